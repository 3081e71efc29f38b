// Private header of the kernel code generator (hip_codegen.hpp is its interface): the model types, small helpers
// and the Generator class, whose member functions are defined in hip_codegen.cpp (driver) and codegen_*.cpp, one
// file per part of the generator:
//   codegen_model.cpp      the model of a kernel group: operands, storages and views, what each kernel reads of what
//                          earlier kernels wrote, contraction ordering
//   codegen_schedule.cpp   the schedule: register tiles and lane order, kernels applied in the registers of their
//                          producers, phases, LDS tiles and their placement, batch and workgroup size
//   codegen_bodies.cpp     code of one work item: offsets, operand sources, unrolled / looped / lane-shared / matrix
//                          bodies, stores
//   codegen_reduction.cpp  the reduction schedule (few outputs, long contraction) and the kernel-parameter helpers
//   codegen_transpose.cpp  the transpose schedule (32 x 32 tiles through LDS)
//   codegen_operator.cpp   the operator schedules (a dense operator applied to every entry, on the FP64 matrix cores)
//   codegen_product.cpp    the product schedule (products of element matrices on the FP64 matrix cores)
//   codegen_chain.cpp      emission of the fused chain kernel: phases, prefetch, item loops, LDS copy-out
#ifndef ACRO_HIP_CODEGEN_IMPL_HPP
#define ACRO_HIP_CODEGEN_IMPL_HPP

#include "hip_codegen.hpp"
#include <algorithm>
#include <cctype>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <functional>
#include <map>
#include <numeric>
#include <set>
#include <sstream>
#include "Error.hpp"

namespace acro
{
namespace codegen
{


// One occurrence of a variable in a kernel.
struct VarRef
{
    int uvar = -1;
    std::vector<int> idx;     // loop id of every dimension
    std::vector<int> ext;     // extent of every dimension
    std::vector<long> stride;  // row-major element stride of every dimension
    long size = 1;
    bool repeated = false;    // some index occurs in two dimensions
};

struct Sub
{
    std::string text;
    VarRef out;
    std::vector<VarRef> in;
    char op = '=';            // '=', '+' or '-'
    std::vector<int> outIdx;  // distinct loop ids of the output
    std::vector<int> contr;   // contraction loop ids, first-appearance order
    // schedule
    std::vector<int> lane;    // loop ids enumerated by the work items (last one fastest)
    std::vector<int> tile;    // loop ids kept in registers by one work item
    std::vector<int> wantedTile;  // the register tile asked for by the step that built this kernel (empty: the cost model's)
    bool loopMode = false;    // contraction as counted loops instead of unrolled code
    bool fusedWithPrev = false;
    std::vector<char> forwardedIn;  // per input occurrence: served from the registers of an earlier kernel of the chain
    // 0: contraction.  1: the output is the inverse of the operand's trailing matrix, 2: its determinant.
    int matrixOp = 0;
    int matrixN = 0;
    // > 0: the kernel has one output per batch entry; that many adjacent lanes share its contraction and add their
    // partial sums through lane exchanges
    int splitLanes = 0;
    bool forwardedOld = false;  // the old value of a += / -= output is the previous kernel's result, in registers
    bool flatItems = false;     // one work item per output, numbered as the output lies in memory (no register tile)
    int phase = 0;              // barrier-separated phase the kernel runs in
    long laneCount = 1, tileCount = 1, contrCount = 1;
};

// An operand of the group: a unique variable (by name) or, in positional mode, one occurrence.
struct UVarInfo
{
    std::string name;
    std::vector<int> dims;
    long size = 0;
    bool written = false;
    int firstWrite = -1;
    int lastUse = -1;
    bool consistent = true;       // same shape and batch positions in every occurrence
    std::vector<int> batchDims;   // dimensions carrying the batch index
    bool anyRepeated = false;
    // the storage this operand is a view of
    int storage = -1;
    long viewOffset = 0;          // first element inside the storage
    std::vector<int> fixed;       // leading indices of the storage that the view fixes
    bool plainView = true;        // the view is "leading indices fixed, all trailing dimensions kept"
    bool isVirtual = false;       // intermediate of a factorised kernel: lives in LDS only, no kernel parameter
    bool isStagedCopy = false;    // ... that is a plain copy of an operand (StageReusedOperands)
};

// A tensor's memory: what kernel parameters point to, what LDS tiles mirror and what stores are elided for.
struct Storage
{
    std::vector<int> dims;        // extents of the root tensor
    std::vector<long> stride;     // its row-major strides
    std::vector<int> members;     // operands that are views of it
    bool written = false;
    bool transient = true;        // every member is marked transient
    int batchDim = -1;            // root dimension carrying the batch index
    bool elementLocal = true;     // every member carries the batch index exactly once, at batchDim
    bool anyRepeated = false;
    int firstWrite = -1;          // kernel numbers
    // LDS residency of the per-batch-entry tile
    bool wantLds = false;
    bool inLds = false;
    int tileSize = 0;             // doubles per batch entry
    std::vector<int> ldsStride;   // per root dimension (0 for the batch dimension)
    int ldsOffset = 0;            // in doubles, start of the NB tiles
    int liveTo = -1;              // last kernel that reads the tile from LDS
    int phaseFrom = 0, phaseTo = 0;  // lifetime in barrier-separated phases (fused kernels share a phase)
    bool elide = false;           // no store to device memory
    bool staged = false;          // small input without batch index: every workgroup copies it to LDS before it starts
    bool copyOutOnly = false;     // result that no kernel reads back: its tile only serves to write it out in whole lines
};

inline long product(const std::vector<int> &ids, const std::vector<int> &extent)
{
    long p = 1;
    for (int i : ids) p *= extent[i];
    return p;
}

inline bool has(const std::vector<int> &v, int x)
{
    return std::find(v.begin(), v.end(), x) != v.end();
}

inline std::string str(long v)
{
    return std::to_string(v);
}

inline uint64_t hashString(const std::string &s)
{
    uint64_t h = 1469598103934665603ull;
    for (unsigned char c : s)
    {
        h ^= c;
        h *= 1099511628211ull;
    }
    return h;
}

inline int envInt(const char *name, int otherwise = 0)
{
    const char *v = std::getenv(name);
    return v ? std::atoi(v) : otherwise;
}

class Generator
{
  public:
    // max_virtual_tile: largest partial result (doubles per batch entry) a reordered single kernel may keep in LDS;
    // 0 = evaluate single kernels as written.
    Generator(const DimensionedMultiKernel &mk_, const HipCodegenOptions &opt_, long max_virtual_tile)
        : mk(mk_), opt(opt_), factorise(max_virtual_tile > 0), maxVirtualTile(max_virtual_tile)
    {
    }

    // The factorised form of a kernel was planned but its intermediates did not all stay on chip: the caller
    // generates the kernel again as written.
    bool factorisationAbandoned = false;
    HipKernelPlan Run();

  private:
    const DimensionedMultiKernel &mk;
    const HipCodegenOptions &opt;
    const bool factorise;
    const long maxVirtualTile;
    bool factorised = false;

    int nidx = 0;
    std::vector<std::string> idxName;
    std::vector<int> extent;
    std::vector<Sub> subs;
    std::vector<UVarInfo> uvars;
    std::set<int> reshaped;  // whole tensors whose dimensions were split by StageReusedOperands: their storage has the split extents
    std::vector<Storage> stores;
    // Per kernel and input occurrence: every entry it reads has been written to the storage's tile by an earlier
    // kernel of the group (so it can be served from LDS); per kernel: the same for the old value of a += output.
    std::vector<std::vector<bool>> readCovered;
    std::vector<bool> oldCovered;
    int batch = -1;
    long E = 1;
    int NB = 1, NT = 128;
    int ldsDoubles = 0;
    bool extentsConsistent = true;
    bool batchUniform = false;  // one batch entry per workgroup: the batch index is a scalar
    double busyLanes = 1.0;     // share of busy lanes in the wavefronts that the chosen batching issues
    bool lightWorkgroups = false;  // the batch was raised because a workgroup would have moved too few bytes
    bool entriesFastest = false;   // the work items of a workgroup are numbered with the batch entry fastest
    bool wide = false;          // 64-bit device-memory offsets

    // Literal of a device-memory stride or offset, and the type such offsets are computed in.
    std::string Lit(long v) const { return std::to_string(v) + (wide ? "L" : ""); }
    const char *OffsetType() const { return wide ? "long" : "int"; }

    // ------------------------------------------------------------------------------------------ model
    // Operand numbering: unique variables by name, or one operand per occurrence in positional mode.
    bool Positional() const { return opt.positional && mk.GetNumKernels() == 1; }
    int NumOperands() const { return Positional() ? mk.Kernels[0]->GetNumVars() : mk.GetNumUVars(); }
    int OperandOf(int ki, int vari) const { return Positional() ? vari + 1 : mk.GetUVari(ki, vari); }
    std::pair<int, int> FirstOccurrence(int u) const;
    void BuildModel();

    // --------------------------------------------------------------------------- contraction ordering
    // A kernel with three or more operands, written as one big sum
    // ("M_e_i_j_k_l_m_n = B_q_i B_q_l B_r_j B_r_m B_s_k B_s_n W_e_q_r_s": 64 terms of 7 factors for each of 729
    // outputs), is evaluated as a chain of smaller contractions when that takes far fewer multiply-adds: a
    // contraction index is summed as soon as every operand carrying it has been multiplied in, and the partial
    // result becomes the operand of the next step.  The partial results are tensors of the generator's own: one
    // tile per batch entry in LDS, never a kernel parameter.  The steps then run through the same machinery as a
    // user-written multi-kernel group.  The order of the steps is the cheapest (in multiply-adds) among those whose
    // every intermediate carries the batch index and fits in LDS; nothing changes unless the gain is large, because
    // one lane already shares partial sums between the outputs of its pencil.
    static constexpr double kFactoriseMinWork = 8192.0;   // multiply-adds per batch entry as written
    static constexpr double kFactoriseMinGain = 4.0;

    struct FactorStep
    {
        std::vector<int> group;   // operand ids multiplied in this step (inputs: 0..n-1, result of step t: n + t)
        std::vector<int> summed;  // loop ids summed in this step
        std::vector<int> result;  // loop ids of the result, in storage order
    };
    double NonBatchVolume(const std::set<int> &ids) const;
    void FactoriseSearch(const Sub &orig, std::vector<int> &live, std::vector<std::vector<int>> &idxOf, std::vector<int> &remaining, double cost, std::vector<FactorStep> &steps, double &best, long &bestSlowest, std::vector<FactorStep> &bestSteps, long &visits) const;
    void FactoriseKernels();
    bool ProductThenRowSums(int ki, const Sub &orig, std::vector<Sub> &result, int &counter);
    bool StageReusedOperands(int ki, const Sub &orig, std::vector<Sub> &result, int &counter);
    bool FactoriseKernel(int ki, const Sub &orig, bool alone, std::vector<Sub> &result, int &counter);
    void BuildStorages();
    bool Covered(const Storage &st, const std::vector<int> &fixed, const std::vector<std::vector<int>> &written) const;
    void AnalyseCoverage();
    bool CheckFusable(std::string &why);

    // --------------------------------------------------------------------------------------- schedule
    bool IsPureInput(int uvar) const { return !stores[uvars[uvar].storage].written; }
    bool IsUniform(const Sub &s, const VarRef &r, const std::vector<int> &tile) const;
    double AccessCostPerItem(const Sub &s, const std::vector<int> &tile) const;
    long LoadsPerItem(const Sub &s, const std::vector<int> &tile) const;
    long WaveFootprint(const Sub &s, const std::vector<int> &tile) const;
    double LinesPerInstruction(const Sub &s, const VarRef &r, const std::vector<int> &lanes) const;

    static constexpr long kUnrollBudget = 8192;   // multiply-adds emitted per work item (before hoisting)
    static constexpr long kMaxUnrolledContraction = 512;  // terms of one unrolled sum
    static constexpr long kMaxTile = 32;
    static constexpr long kMaxLiveValues = 160;   // loaded operands + accumulators held by one lane
    static constexpr long kPrefetchDoubles = 48;  // per lane, held in registers from kernel entry to their phase
    void ChooseTiles();
    bool ChooseLoopTile(Sub &s, const std::vector<int> &mid) const;
    void ForcedTile(int k, const std::vector<int> &mid, std::vector<int> &tile) const;
    void SetLanes(Sub &s);
    bool ForwardableFrom(const Sub &q, const VarRef &r, const std::vector<int> &lane) const;
    bool ChainOperandsFromRegisters(int k, int chainStart, const std::vector<int> &lane, std::vector<char> &fwd) const;
    void ForwardAlongChain(int k, int chainStart);
    int ChainStartOf(int k) const;
    void PlanFusion();
    bool ViewsOverlap(int ua, int ub) const;
    bool KernelsIndependent(int ka, int kb) const;
    void AssignPhases();
    bool FromRegisters(int k, int v) const;

    int PhaseOf(int k) const { return subs[k].phase; }
    void ComputeLdsWishes();
    void ChooseCopyOutTile();

    // A small operand that does not depend on the batch entry but whose address depends on the lane
    // ("A_e_i = B_i_j X_e_j" with one lane per i: lane i walks along row i of B, 512 bytes from its neighbour's) cannot
    // be read with scalar loads, and read from device memory every load instruction touches 64 lines, which the
    // memory pipeline works through one by one (measured 3 % of the HBM peak for that kernel with a 64 x 64 B).  Every
    // workgroup copies such an operand into LDS once, with coalesced loads, and its lanes read it there; the stride of
    // the lanes in LDS is made odd so that they fall into different banks.
    static constexpr long kMaxStagedDoubles = 4096;
    void ChooseStagedInputs();

    // Doubles of LDS that a storage's tiles take in a workgroup of nb batch entries.
    int LdsNeed(const Storage &st, int nb) const { return st.tileSize * (st.staged ? 1 : nb); }
    int PlaceLds(int nb);
    int PlaceLdsFromBothEnds(int nb);
    void ChooseBatching();
    bool EntriesAreFastest() const;
    void ChooseEntriesFastest();
    static long ConflictCycles(const std::vector<long> &addr);
    std::vector<long> LaneAddresses(const Sub &s, const VarRef &r, int nb) const;
    long LdsCostOfStorage(int si, int nb) const;
    void SetLdsStrides(Storage &st, const std::vector<int> &pad, int padEntry) const;
    void PadLdsTiles(int budgetDoubles, bool stagedCopiesOnly);

    // --------------------------------------------------------------------------------------- emission
    std::ostringstream out;

    // Kernel parameters are storages; an operand addresses its storage at viewOffset.
    std::string PtrName(int uvar) const { return "T" + str(uvars[uvar].storage); }
    int GatherSlot(int uvar) const;
    int NumGatherSlots() const;
    std::string GlobalRead(int uvar, const std::string &offset, bool streamedOnce = false) const;
    bool StreamedOnce(int k, int v) const;
    std::string ConstPtrName(int uvar) const { return "C" + str(uvars[uvar].storage); }
    const Storage &StoreOf(int uvar) const { return stores[uvars[uvar].storage]; }
    int LdsStride(int uvar, size_t d) const;
    long LdsViewOffset(int uvar) const;
    std::string IdxVar(int id) const { return "i_" + idxName[id]; }
    std::string RuntimeOffset(const VarRef &r, const Sub &s, bool lds) const;
    long LiteralOffset(const VarRef &r, const Sub &s, bool lds, const std::vector<int> &value) const;

    // Where an input occurrence of kernel k is read from.
    enum Source
    {
        kFromRegisters,
        kFromConstant,
        kFromLds,
        kFromGlobal
    };
    Source SourceOf(int k, int v) const;
    std::string ScalarBase(const VarRef &r) const;

    // Results that the kernels of a chain have left in registers: (operand, literal offset) -> register name.
    typedef std::map<std::pair<int, long>, std::string> ForwardMap;

    struct Body
    {
        std::vector<std::string> bases;    // run-time base offsets
        std::vector<std::string> loads;    // operand loads
        std::vector<std::string> compute;  // partial sums and outputs
        std::vector<std::string> stores;
        std::map<std::string, std::string> loadMemo;
        std::map<std::string, std::string> sumMemo;
        int counter = 0;
        // Loads of per-entry pure inputs from device memory, in order of first use: (memo key, right-hand side).
        // They are what a prefetch at kernel entry would issue.
        std::vector<std::pair<std::string, std::string>> globalLoads;
    };
    bool Prefetchable(int k, int v) const;
    std::string OperandExpr(int k, int v, const std::vector<int> &value, Body &body, const ForwardMap &forwarded);
    std::string PartialSum(int k, int depth, std::vector<int> &value, Body &body, const std::vector<int> &level, const ForwardMap &forwarded);
    void EmitBases(int k, Body &body);

    // Is the output variable's tile already on chip before kernel k (needed by += and -=)?
    bool OldValueInLds(int k) const { return StoreOf(subs[k].out.uvar).inLds && oldCovered[k]; }
    bool StoreIsDead(int k) const;

    bool StoresToGlobal(int k) const { return !StoreOf(subs[k].out.uvar).elide && !StoreIsDead(k); }
    bool StreamsOut(int k) const;
    double WaveStoreLineCoverage(int k, int entries = 0) const;
    bool WritesDominate() const;
    bool SplitLanesTakePairs(int k) const;
    std::string GlobalStore(int k, const std::string &gaddr, const std::string &value) const;
    bool NeedsLdsCopy(int k) const;
    bool CopiesOutFromLds(int k) const;
    void EmitUnrolledBody(int k, ForwardMap &forwarded, std::vector<std::string> &lines, const std::map<std::string, std::string> *preloaded = nullptr, std::vector<std::pair<std::string, std::string>> *globalLoads = nullptr);
    void EmitMatrixBody(int k, Body &body, ForwardMap &forwarded);
    void EmitSplitLanesBody(int k, std::vector<std::string> &lines);
    void EmitLoopBody(int k, std::vector<std::string> &lines);

    // ------------------------------------------------------------------------------ reduction schedule
    // A single kernel with few output entries and a very long contraction ("S_i_j = A_n_i_j B_n" with n = 2^20):
    // mapping lanes to outputs would leave the device idle, so the flattened contraction range is split over
    // workgroups and over the lanes of a workgroup.  Lane (slice, output entry) accumulates a private partial sum
    // over its share, the workgroup adds its slices in LDS and writes one partial per output entry to a scratch
    // buffer, and a second, single-workgroup kernel adds the per-workgroup partials in a fixed order (no
    // floating-point atomics: results are reproducible from run to run).
    static constexpr long kReductionMinContraction = 2048;
    static constexpr long kReductionMaxOutputs = 128;
    static constexpr int kReductionLanes = 256;
    bool UseReductionSchedule() const;
    bool UseReductionFallback() const;
    bool ReductionServes(const Sub &s) const;
    std::string FullOffset(const VarRef &r) const;
    int NumParamStores() const;
    void FillParams(HipKernelPlan &plan, bool honour_elision) const;
    std::string ParamList() const;
    void EmitReduction(HipKernelPlan &plan);
    bool UseTransposeSchedule() const;

    // "A_I_J = B_N_I C_N_J [W_N]": the I x J matrix of sums over a long leading range N
    struct GramShape
    {
        const VarRef *b = nullptr, *c = nullptr, *w = nullptr;
        long rows = 0, cols = 0, range = 0;
        bool swapped = false;   // the result is stored as J x I
    };
    bool GramPattern(GramShape &g) const;
    bool UseGramSchedule() const;
    void EmitGram(HipKernelPlan &plan);
    void EmitTranspose(HipKernelPlan &plan);

    // "A_e_r_c = R_e_{r,k} C_e_{k,c}": products of element matrices on the FP64 matrix cores (codegen_product.cpp)
    struct ProductShape
    {
        const VarRef *row = nullptr, *col = nullptr;   // the factor that carries the result's row / column index
        bool rowKFast = false, colKFast = false;       // the contracted index is the factor's fastest dimension
        long M = 0, N = 0, K = 0, E = 0;
        bool pairMap = false;                          // the terms of a step are permuted so that 16-byte loads feed two steps
        int rowMode = 0;                               // how the row factor reaches the registers, see ProductPattern
        long steps = 0, TI = 0, TJ = 0, NBE = 1, ldsPerEntry = 0;
    };
    bool ProductPattern(const Sub &s, ProductShape &p) const;
    bool UseProductSchedule() const;
    void EmitProduct(HipKernelPlan &plan);

    // Products of matrices too large for one workgroup, with or without a batch index (codegen_product.cpp).
    struct TiledProductShape
    {
        const VarRef *row = nullptr, *col = nullptr;
        bool rowKFast = false, colKFast = false, batched = false;
        long M = 0, N = 0, K = 0, E = 1;
        long W = 0, TJ = 0, tilesM = 0, panels = 0, KC = 16;   // strips per workgroup, blocks per strip, tiles per entry, terms per chunk
        long splits = 1;                                        // shares of the contracted range (more than one: partial sums through scratch)
    };
    bool TiledProductPattern(const Sub &s, TiledProductShape &p) const;
    bool UseTiledProductSchedule() const;
    void EmitTiledProduct(HipKernelPlan &plan);

    // ------------------------------------------------------------------------------ operator schedule
    // One dense operator applied to every batch entry: "A_e_i = B_i_j X_e_j" with B too large for scalar operands or a
    // register tile (16 <= rows, columns; at most 4 096 entries), also with several row or column indices
    // ("A_e_i1_i2 = B_i1_i2_j1_j2 X_e_j1_j2") and with several leading indices numbering the entries
    // ("A_e_q_i = B_i_j X_e_q_j").  The generic schedule stages B in LDS and gives a lane one row and one
    // entry, which is bound by the 64 LDS reads per output (17 % of the HBM peak for 64 x 64).  Two variants:
    // rows a multiple of 16 and columns a multiple of 8 go to the FP64 matrix cores (EmitOperatorMatrixCores, 72 %;
    // the operator may then also be stored transposed, "B_j_i").  Otherwise a lane keeps its
    // row for four entries at a time, so one LDS read feeds four multiply-adds; the entry number is uniform in a
    // wavefront, so X is read with scalar loads, and the lanes of a wavefront write consecutive outputs (43 %).
    // Taking the entries' vectors into registers first and handing them round with readlane was slower (216 us).
    static constexpr int kOperatorEntriesPerLane = 4;

    // The kernels that the operator schedules see: the group's kernels, with pointwise kernels folded into the operator
    // kernel whose transient result they rescale ("U = B X" followed by "V = U D" reads as "V = B X D").
    mutable std::vector<Sub> opKernels;
    mutable bool opKernelsReady = false;
    void FoldPointwiseKernels() const;
    int NumOpKernels() const;
    const Sub &OpKernel(int k) const;

    struct OperatorShape
    {
        const VarRef *op = nullptr, *x = nullptr;
        long rows = 0, cols = 0, entries = 0;
        // An operator too large for LDS is applied in blocks of rows, one launch per block: `blockRows` rows at a
        // time (0: whole).  The emitter then sees `rows` rows starting at `rowOffset` of `allRows`.
        long blockRows = 0, rowOffset = 0, allRows = 0;
        bool transposed = false;   // the operator is stored with the contracted indices first: "B_j_i"
        // the operator's dimensions in any other order: per row index and per column index (fastest first) what to
        // divide the row / column number by, its extent and its stride in the operator
        bool mixed = false;
        struct Term
        {
            long div, ext, stride;
        };
        std::vector<Term> rowTerms, colTerms;
        // component indices between the result's row indices: where row number and component number go in an entry
        bool outMixed = false;
        std::vector<Term> outRowTerms, outCompTerms;
        bool cores = false;        // sizes and alignment suit the FP64 matrix cores
        bool pairs = false;        // the entries' vectors (and weights of their shape) come in 16-byte loads
        bool trailing = false;     // the entries are the fastest dimension: "A_i_e = B_i_j X_j_e"
        // > 1: the result and the vectors carry that many components behind the operator's indices
        // ("A_e_i_k = B_i_j X_e_j_k"): entry (e, k) has its vector elements and its outputs `comp` doubles apart
        long comp = 1;
        // Pointwise factors beside the operator and the vectors (matrix-core variant only): one value per entry
        // "W_e", per output "W_e_i", per row "W_i" scale the result; per vector element "W_e_j" or per column
        // "W_j" scale the entries' vectors as they are loaded.
        std::vector<const VarRef *> perEntry, perOutput, perRow, perElement, perColumn;
    };
    bool OperatorPattern(OperatorShape &o, int k = 0, bool alone = true) const;
    bool UseOperatorSequence() const;
    bool OperatorPair(OperatorShape &first, OperatorShape &second) const;
    bool UseOperatorSchedule() const;


    int opSub = 0;            // the kernel that the operator emitters work on
    int opBlock = 0;          // ... and the block of rows, for an operator applied in blocks
    bool opSequence = false;  // ... as one of several launches
    void EmitOperator(HipKernelPlan &plan);
    void EmitOperatorMatrixCores(HipKernelPlan &plan, const OperatorShape &shape, const OperatorShape *next = nullptr, int nextSub = -1);
    void EmitOperatorEntriesFastest(HipKernelPlan &plan, const OperatorShape &shape);
    void EmitOperatorComponents(HipKernelPlan &plan, const OperatorShape &shape);
    bool ComponentsTogether(const OperatorShape &o) const;
    std::string OperatorEntry(const OperatorShape &shape, const std::string &row, const std::string &j, long allRows) const;
    void Emit(HipKernelPlan &plan);
};

}  // namespace codegen
}  // namespace acro

#endif
