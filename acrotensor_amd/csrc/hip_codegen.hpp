// Kernel code generator of the "HIP" policy: DimensionedMultiKernel -> fixed-size HIP C++ source for gfx950.
// Replaces the reference's CUDA text generator (exec/CudaExecutor.cpp:111-702) with a different schedule,
// designed for 64-wide wavefronts and HBM-bound finite-element chains:
//
//  * One workgroup owns NB consecutive values of the batch index (the largest index shared as an outer index by
//    every kernel of the group - the "element" index) and runs every kernel of the group on them, separated by
//    workgroup barriers.  Nothing is exchanged between workgroups.
//  * Inside a kernel a lane owns one "pencil": fixed values of the lane indices and ALL values of the tile
//    indices.  Contraction and tile loops are fully unrolled; every operand entry is loaded once per pencil and
//    partial sums that do not depend on an inner index are hoisted (sum factorisation inside the lane).
//  * Small operands that do not vary with the lane (basis matrices) are read through the constant address space,
//    i.e. with scalar loads into SGPRs, and feed the FMAs as scalar operands.
//  * An output that a later kernel of the group consumes stays in LDS (one tile per batch entry); its store to
//    device memory is skipped when the tensor is marked transient.  A kernel without contraction whose operand
//    was just produced with the same index set is applied in registers (no LDS round trip).
//    More generally a kernel whose work items can be those of the previous kernel, and that reads that kernel's
//    results (or those of the kernels it was applied after) entry by entry, runs in the same registers, also when it
//    contracts over the producer's register tile.
//  * A kernel with three or more operands written as one big sum is evaluated as a chain of smaller contractions
//    (the cheapest elimination order whose partial results fit in LDS) when that saves at least 4x the multiply-adds.
//  * Matrix kernels (TensorKernel::Function "inv" / "det": what the engine turns recorded batched inverses and
//    determinants into) take one work item per matrix and follow the host formulas term by term.
//  * Register tiles are chosen by loads per output, weighted by how the lanes reach device memory (lines touched per
//    load instruction, cache footprint of a wavefront); batch entries with few outputs get one output per lane; a
//    kernel whose dominant operand streams along the contraction shares each output between 2 - 16 lanes that add
//    their partial sums by DPP exchanges; small invariant operands with lane-dependent addresses are staged in LDS.
//  * A single kernel with few outputs and a long contraction runs the "reduction schedule": the contraction range
//    is split over workgroups and lanes, partial sums are added in a fixed order by a second one-workgroup kernel.
//  * A single kernel that only permutes the dimensions of one operand, with different long fastest dimensions on the
//    two sides, moves tiles of 32 x 32 entries through LDS ("transpose schedule").
//  * A dense operator of up to 4 096 entries applied to every batch entry ("A_e_i = B_i_j X_e_j", also stored
//    transposed, with several leading indices numbering the entries, or with the entries as the fastest dimension,
//    "A_i_e = B_i_j X_j_e") runs the "operator schedule" on the FP64
//    matrix cores: 16 entries per wavefront and trip through v_mfma_f64_16x16x4, the operator in LDS in operand order
//    and padded with zeros to whole 16 x 4 blocks; pointwise factors per entry, output, row, vector element or
//    column stay in the same launch; a second operator applied to a transient result runs in the same kernel, the
//    intermediate passing from the result layout to the operand layout through a per-wavefront piece of LDS.
//    A larger operator is applied in blocks of rows that fit LDS, one launch per block; results of operators whose
//    rows 16 does not divide leave through LDS as one contiguous range per trip.
//  * Products of element matrices ("A_e_i_j = B_e_i_k C_e_k_j") copy their per-entry operands to LDS tiles with the
//    lanes along memory and compute from the tiles; output indices of even extent are split in two so that a lane owns
//    a 2 x 2 block of outputs.
//  * "A_i_j = B_n_i C_n_j" with more than 64 outputs runs the "Gram schedule": four rows of the range per
//    v_mfma_f64_16x16x4, up to 16 blocks of 16 x 16 sums per wavefront, partial matrices added by a second kernel.
//  * A kernel whose tensors all have the batch index as their fastest dimension numbers its work items with the entry
//    fastest, so that a wavefront reads consecutive entries.
//  * A streaming group whose workgroups would move less than 2.5 KB takes more batch entries per workgroup.
//  * Contractions too long to unroll fall back to counted loops with the same lane mapping.
//
// Experiment switches (environment, read when a kernel is generated; defaults are what measured best on MI355X):
//   ACRO_HIP_NB / ACRO_HIP_NT   batch entries per workgroup / lanes per workgroup (default: chosen per kernel)
//   ACRO_HIP_MERGE=-1           one phase per chain instead of sharing phases between independent kernels
//   ACRO_HIP_PREFETCH=-1        no prefetch of later phases' streaming inputs at kernel entry
//   ACRO_HIP_NT_STORE=-1        ordinary instead of non-temporal stores for results that stream out
//   ACRO_HIP_LDS_PAD=1|2        pad LDS tile strides against bank conflicts (2: even if a resident workgroup is lost)
//   ACRO_HIP_PACK=1|-1          1: pick batch / workgroup size for wavefront utilisation also when one batch entry per
//                               workgroup would do; -1: never (default: only for groups that batch several entries)
//   ACRO_HIP_PERSIST=<n>        persistent grid of n workgroups per CU looping over the batch
//   ACRO_HIP_PIPELINE=1         with ACRO_HIP_PERSIST: streaming inputs stay in registers across iterations and are
//                               requested one iteration ahead
//   ACRO_HIP_FACTORISE=-1|2     -1: evaluate multi-operand kernels as written instead of as a chain of steps;
//                               2: reorder whenever a chain is cheaper at all (default: only large kernels, 4x gain)
//   ACRO_HIP_LDS_COPY_OUT=-1    stored results that also live in LDS are written by the lanes that computed them instead
//                               of by the workgroup from the LDS tiles
//   ACRO_HIP_FORWARD=-1         only a pointwise kernel directly after its producer is applied in that kernel's registers
//                               (no contractions over the producer's register tile, no matrix kernels joined to readers)
//   ACRO_HIP_FOOTPRINT=-1       register tiles by loads per output alone (no weight for uncoalesced streaming loads, no
//                               cache-footprint term, no one-output-per-lane rule for tiny batch entries)
//   ACRO_HIP_FORCE_TILE="8:;3:q,r"  kernel 8 of the group takes the empty register tile, kernel 3 the tile (q, r)
//   ACRO_HIP_COLLAPSE=-1        offsets are sums over every lane index (runs of lane indices that an operand lays out in
//                               the lanes' own order are not collapsed into one multiple of the item number)
//   ACRO_HIP_WRITE_BATCH=-1     write-heavy launches whose results leave through LDS tiles keep their batch size
//                               (default: twice the batch entries in workgroups of 512 lanes)
//   ACRO_HIP_OPERATOR_COMPONENTS=-1  operators applied to vectors with trailing component indices ("A_e_i_k = B_i_j X_e_j_k")
//                               run through the generic schedule, not on the matrix cores
//   ACRO_HIP_COPY_OUT_TILE=-1|2 -1: results are always stored by the lanes that computed them; 2: an LDS tile that the workgroup
//                               writes out in whole lines only for a kernel on its own whose lanes each hold a long run of outputs
//                               (default: also for the last kernel of any group whose store instructions would fill less than
//                               30 % of the lines they touch).  ACRO_HIP_COPY_OUT_MAX=<doubles per batch entry> (default 2048)
//   ACRO_HIP_ROW_SUMS=-1        an element matrix times an element vector with rows that are no multiple of four doubles, and
//                               one to three short sums per entry (dot products, row sums), run as written (lanes along the
//                               rows) instead of as products into LDS followed by row sums
//   ACRO_HIP_PREFETCH_FIRST=-1 / ACRO_HIP_PREFETCH_CLAMP=-1 / ACRO_HIP_PREFETCH_PASSES=-1
//                               the first phase's operands are not requested ahead of the prefetched ones / prefetch loads of
//                               partly filled passes stay behind a branch / a first phase of several passes keeps its item loop
//   ACRO_HIP_LDS_BOTH_ENDS=-1   LDS tiles are always placed first-fit from the bottom (default: from both ends of the region
//                               when that lets one more workgroup live on a compute unit)
//   ACRO_HIP_LOOP_TILE=-1       kernels far above the machine balance keep their unrolled body or a plain counted loop (default:
//                               counted loops around a register tile, see ChooseLoopTile)
//   ACRO_HIP_STAGE_ENTRIES=-1   products of element matrices read their operands from device memory (no copies to LDS tiles first)
//   ACRO_HIP_STAGE_ENTRIES=2    ... are staged, but their output indices are not split into blocks (one output or one row per lane)
//   ACRO_HIP_STAGE_TRANSPOSED=-1 ... and the copy of a factor whose fastest dimension is contracted keeps the operand's layout
//   ACRO_HIP_SPLIT_FIVE=-1      ... and extents divisible by five only are not split in five
//   ACRO_HIP_STAGE_MOST=<n>     ... at most n staged values per entry (default 8000; 2048: matrices up to 32 x 32 only)
//   ACRO_HIP_STAGE_WHOLE_LINES=<n> / =-1  tiny products (fewer than 64 outputs per entry) whose operands' entries are powers of two
//                               of doubles are staged from n outputs per entry on (16) / never
//   ACRO_HIP_STAGE=-1           small invariant operands with lane-dependent addresses stay in device memory (not staged in LDS)
//   ACRO_HIP_SPLIT_PAIRS=-1     lanes that share a contraction take its terms one at a time also where they have few of them
//   ACRO_HIP_SPLIT_LANES=-1     one lane per batch entry also for kernels with one output per entry (no lane exchanges)
//   ACRO_HIP_WAVE_UNIFORM=-1    no readfirstlane on the batch entry of wavefronts that hold items of one entry only
//   ACRO_HIP_TRANSPOSE=-1|2     -1: permutations with long fastest dimensions on both sides run as ordinary kernels (no LDS
//                               tiles); 2: LDS tiles only where both dimensions have 32 entries or more (no rectangular tiles)
//   ACRO_HIP_OPERATOR=-1        a dense operator applied to every batch entry runs through the generic schedule (operator staged
//                               in LDS, one entry per lane) instead of the operator schedule
//   ACRO_HIP_LIGHT=-1           streaming groups whose workgroups move less than 2.5 KB keep their batch size (no extra
//                               passes to bring a workgroup to 8 KB)
//   ACRO_HIP_ENTRIES_FASTEST=-1 tensors with the batch index last: work items numbered entry by entry all the same
//   ACRO_HIP_GRAM=-1            "A_i_j = B_n_i C_n_j" with more than 64 outputs does not take the Gram schedule (matrix cores, two launches)
//   ACRO_HIP_OPERATOR_ANY_ORDER=-1  operators whose dimensions are neither rows by columns nor columns by rows: generic schedule
//   ACRO_HIP_OPERATOR_COMPONENTS=2  vectors with components: always entries (entry, component), never the components of an entry together
//   ACRO_HIP_OPERATOR_BLOCKS=-1 operators of more than 4 096 entries are not applied in blocks of rows (generic schedule instead)
//   ACRO_HIP_OPERATOR_STAGE_OUT=-1  results of operators whose rows 16 does not divide are stored by the lanes that hold them
//   ACRO_HIP_OPERATOR_FOLD=-1   a pointwise kernel that rescales an operator kernel's transient result is not folded into it
//   ACRO_HIP_OPERATOR_PAIR=-1   two operator-shaped kernels with a transient intermediate are not joined into one matrix-core kernel
//   ACRO_HIP_OPERATOR_SEQUENCE=-1  groups of several large operator-shaped kernels run as one fused chain kernel instead of one
//                               matrix-core launch per kernel
//   ACRO_HIP_OPERATOR_SMALL=-1  operators below 16 rows and 16 columns applied to vectors of even length take the operator schedule
//                               from five rows on, as they did before the generic schedule overtook it there
//   ACRO_HIP_OPERATOR_FEW_ROWS=<n>  operators of two to four rows take the operator schedule from n columns on (default 16; 0: never)
//   ACRO_HIP_OPERATOR_MFMA=-1   the operator schedule never uses the FP64 matrix cores (a lane keeps its row for four entries,
//                               whose vectors come through scalar loads, whatever the operator's sizes)
//   ACRO_HIP_RED_PENCIL=-1      split contractions: one lane per (slice, output entry) also when there are few outputs
//   ACRO_HIP_RED_WIDE=-1        sums over a long index with more than 128 outputs keep the generic schedule
//   ACRO_HIP_RED_FALLBACK=-1    a long contraction that no schedule takes and that the generic plan leaves to few lanes keeps
//                               the generic plan instead of being shared out over workgroups
//   ACRO_HIP_FACTORISE_PAIRS=-1 a kernel of two operands is not taken apart where an operand carries a contraction index alone
//   ACRO_HIP_SPLIT_ORDER=-1     a contraction shared by lanes is numbered as the kernel names its indices, not as they lie in
//                               the streaming operand
//   ACRO_HIP_NT_LOADS=-1 / ACRO_HIP_RED_NT=-1 / ACRO_HIP_GRAM_NT=-1 / ACRO_HIP_PRODUCT_NT=-1
//                               no non-temporal hint on operands that are read once in whole lines (chain, reduction, Gram
//                               and product schedules)
//   ACRO_HIP_RED_ROWS=-1        split contractions of few long rows: all outputs in every workgroup, NT / outputs lanes along a row
//   ACRO_HIP_ONE_PASS=1         split contractions: the workgroup that finishes last adds the per-workgroup partials
//                               instead of a second kernel (measured 18.4 against 16.3 us: the device-scope release
//                               writes back the XCD's L2 once per workgroup)
//   ACRO_HIP_RED_GROUPS=<n> / ACRO_HIP_RED_UNROLL=<n>
//                               split contractions where a lane owns whole slices: number of workgroups (default 256, one per
//                               compute unit) and slices a lane requests before it adds them (default 1)
//   ACRO_HIP_PRODUCT=-1 / =2    products of two element matrices never / whenever they fit take the product schedule on the
//                               matrix cores (default: from 17 rows or columns on, except sizes up to 36 that 2, 3 or 5 divide)
//   ACRO_HIP_PRODUCT_FROM=<n> / ACRO_HIP_PRODUCT_TO=<n>   smallest and largest "larger of rows and columns" it takes (17, 64)
//   ACRO_HIP_PRODUCT_ENTRIES=<n>  entries per workgroup of the product schedule (default: up to 4 wavefronts, 8 192 LDS values)
//   ACRO_HIP_PRODUCT_DIRECT=-1  the row factor always passes through LDS, also where lanes could load their operands directly
//   ACRO_HIP_COPY_OUT_COVERAGE=<percent>  share of the touched lines below which the last kernel's stores leave through an
//                               LDS tile (default 30);  ACRO_HIP_COPY_OUT_WRITERS=-1: launches whose stores dominate no
//                               longer do so below 95 %
//   ACRO_HIP_WRITE_BATCH_FROM=<n>  write-heavy launches that copy out of LDS tiles double their batch from this batch size on (1)
//   ACRO_HIP_NT_COPY_OUT=-1     copies out of LDS tiles use non-temporal stores only for tiles of at most 20 KB
//   ACRO_HIP_NT_STORE=2         non-temporal stores from registers also in launches that hold more than 20 KB of LDS per workgroup
//   ACRO_HIP_OPERATOR_GROUPS=<n>  workgroups of the matrix-core operator kernel (default: 256 - 1 024 by the operator's size)
//   ACRO_HIP_GRAM_GROUPS=<n>    workgroups of the Gram schedule's first kernel (default: 256 where the blocks of outputs are whole, else 512)
//   ACRO_HIP_PRODUCT_VECTOR=-1 / =2  an element matrix applied to an element vector never takes the product schedule / takes it
//                               whatever its row length (default: rows of 25 - 128 doubles that are no multiple of four, 16 - 128 rows)
//   ACRO_HIP_COPY_OUT_RUN=<n>   a kernel on its own whose lanes each hold a run of n or more consecutive outputs writes them out
//                               through an LDS tile (default 4)
//   ACRO_HIP_XCD_RUN=-1 / =<n>  fused launches that read an operand through an index map number their workgroups as the hardware
//                               deals them / in runs of n per XCD (default 16)
//   ACRO_HIP_TILED_PRODUCT=-1   large matrix products (more than 64 rows or columns or 128 terms per entry, or no batch index) keep
//                               the generic schedule;  ACRO_HIP_TILED_PRODUCT_FROM=<n>: smallest "larger of rows and columns" (65)
//   ACRO_HIP_TILED_PRODUCT_CHUNK=<terms> / _STRIPS=<n> / _BLOCKS=<n> / _WAVES=<n>
//                               terms per chunk (16), most strips per workgroup and blocks per strip (8, 8), waves per SIMD asked of
//                               the compiler (none)
//   ACRO_HIP_TILED_PRODUCT_SPLIT=-1 / =<n>  never share out the contracted range / share it out n ways
//   ACRO_HIP_TILED_PRODUCT_VGPR_FORM=-1  launches of few workgroups are compiled like the others (default: for at least two
//                               wavefronts per SIMD, which keeps the matrix instruction's accumulators in ordinary vector registers)
//   ACRO_HIP_TILED_PRODUCT_HALF=-1 / _PREFER=<n>  few tiles keep eight strips per workgroup (default: four) / blocks per strip
//                               that the split of the columns prefers (4)
//   ACRO_HIP_TILED_PRODUCT_XCD=-1  the tiles of an entry are numbered as the hardware deals them (default: an entry's two to four
//                               tiles on one XCD, so that the strips they share pass through one L2)
//   ACRO_HIP_TILED_PRODUCT_OPERATOR=<entries>  a product without a batch index one of whose factors has at most this many entries
//                               is left to the operator schedule (4 096);  ACRO_HIP_TILED_PRODUCT_OPERATOR_MID=<entries>: up to
//                               this many entries, with at most 96 columns, the operator schedule goes first where it applies (8 192)
#ifndef ACRO_HIP_CODEGEN_HPP
#define ACRO_HIP_CODEGEN_HPP

#include <string>
#include <utility>
#include <vector>
#include "DimensionedMultiKernel.hpp"

namespace acro
{

// Where an operand lives: operands that are views (leading-index slices) of one tensor share a storage number;
// offset is the view's first element inside that tensor and root_dims the tensor's own extents.
struct HipOperandView
{
    int storage = -1;
    long offset = 0;
    std::vector<int> root_dims;
};

struct HipCodegenOptions
{
    // Per operand: the executor allows the store to device memory to be dropped (transient tensor).
    std::vector<bool> transient;
    // Per operand (empty: every operand is a tensor of its own).  Views of one storage may be written under one
    // name and read under another inside a fused launch; the generator resolves them exactly.
    std::vector<HipOperandView> views;
    // False when two unique variables overlap in device memory and one of them is written: pointers are then
    // not declared restrict and nothing is read through the constant address space.
    bool noalias = true;
    // Single kernels only: every variable occurrence is a separate operand even when two occurrences share a
    // name (the caller bound them to different tensors).  transient is then indexed by occurrence: output, then
    // inputs in order.
    bool positional = false;
    int force_nb = 0;  // 0 = choose
    int force_nt = 0;  // 0 = choose
    // Per operand (empty: none): >= 0 says that the operand is never materialised: entry i of it is entry map[i] of a
    // source vector (a FlatIndexedScatter recorded in the same multi-kernel launch whose result is transient).  The
    // value numbers the (map, source) pair among the extra kernel parameters.  Only for operands that are read, never
    // written, by the group, and not in positional mode.
    std::vector<int> gathered;
    // True: no schedule that uses the FP64 matrix cores (the operator and Gram schedules) is chosen.  The executor asks
    // for this after a matrix-core kernel has come out of the compiler with private memory (register spills) that the
    // schedule's register-relief switch did not remove: such a kernel is never launched.
    bool no_matrix_cores = false;
};

// One kernel launch of a plan.  params: >= 0 is an index into HipKernelPlan::param_occurrence (a storage's device
// pointer), -1 is the plan's scratch buffer, -2 - 2 g the index map (const int *) and -3 - 2 g the source vector
// (const double *) of gathered-operand pair g.
struct HipLaunch
{
    std::string function_name;
    unsigned grid = 0;
    unsigned grid_y = 1;  // > 1: the work items of one batch entry are spread over this many workgroups
    unsigned block = 0;
    std::vector<int> params;
};

struct HipKernelPlan
{
    bool fusable = false;        // false: the group must be run as one launch per kernel
    std::string why_not;         // reason when !fusable
    std::string module_name;
    std::string source;            // one translation unit defining every function of `launches`
    std::vector<HipLaunch> launches;  // executed in order on the library's stream
    // Device scratch the launches share (partial sums of split contractions and their arrival counter).  The
    // executor zeroes it once, when it allocates it; the kernels leave the counter at zero when they finish.
    size_t scratch_doubles = 0;
    // Kernel parameter i is the device pointer of a storage: the device pointer of the tensor bound to this
    // (kernel number, variable number) occurrence (variable number -1 is that kernel's output) minus param_offset[i]
    // elements (the occurrence may be a view into the storage).
    std::vector<std::pair<int, int>> param_occurrence;
    std::vector<long> param_offset;
    std::vector<bool> stored;      // per parameter: the kernel writes it to device memory
    // Parameters that must be set to zero before the launch: an output assigned with "=" whose index list repeats
    // an index ("A_i_i = B_i") is only written on its diagonal by the kernel, while assignment means zero-fill
    // followed by accumulation (reference exec/CPUInterpretedExecutor.cpp:63-67).
    struct ZeroFill
    {
        int param;    // storage parameter
        long offset;  // first element
        long count;   // number of elements
    };
    std::vector<ZeroFill> zero_fills;
    int lds_bytes = 0;
    int nb = 0;
    bool gathers_applied = false;  // the source reads gathered operands through their maps (HipCodegenOptions::gathered)
    // Kernels of `source` that hold matrix-core accumulators: they keep nothing in private memory by design, and a
    // code object that reports private memory for one of them has register spills, which the compiler has been seen to
    // get wrong around those accumulators.  register_relief_macro, when not empty, names a preprocessor switch of
    // the source that trades registers for LDS reads.
    std::vector<std::string> matrix_core_functions;
    std::string register_relief_macro;
    std::string schedule;          // human readable schedule summary (also a comment in the source)
};

HipKernelPlan GenerateHipKernel(const DimensionedMultiKernel &mk, const HipCodegenOptions &options);

}  // namespace acro

#endif
