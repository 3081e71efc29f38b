// Kernel code generator, the product schedule: products of element matrices on the FP64 matrix cores,
// "A_e_i_j = B_e_i_k C_e_k_j" with either factor stored either way round.
#include "hip_codegen_impl.hpp"

namespace acro
{
namespace codegen
{

// "A_e_r_c (=|+=|-=) R_e_{r,k} C_e_{k,c}": every batch entry holds an M x K and a K x N matrix (each stored with the
// contracted index last or first) and receives their M x N product, all three contiguous per entry.  The reference
// maps a thread to an output and loops over k (exec/CudaExecutor.cpp:193-263); the staged vector-ALU schedule of this
// generator does the same out of LDS tiles, where every multiply-add reads one or both of its factors from LDS: from
// 33 x 33 on it is bound by LDS (55 x 55: 22 % of the HBM peak, 63 x 63: 32 %), and these sizes carry as much
// arithmetic as traffic.  v_mfma_f64_16x16x4 multiplies a 16 x 4 block by a 4 x 16 block per instruction with one
// operand value per lane each.
//
// A wavefront owns a strip of 16 rows of one entry's result.  It loads its strip of the row factor straight from
// device memory in the layout the instruction wants (lane = row + 16 * term group), 16 bytes per lane where the
// contracted index is the fastest dimension (the two doubles go to two successive steps: the terms of a step are
// permuted, k = 8 [s / 2] + 2 g + s mod 2, which a sum does not mind).  The column factor is needed by every strip:
// the wavefronts of an entry load it once, each a share of its 16-column blocks, also in instruction layout, and
// leave it in LDS fragment by fragment, so that the reads in the multiply loop are 64 consecutive doubles (no bank
// conflicts).  Rows and columns past the end read the last valid one (their results are not stored), terms past
// the end read as zero.  The accumulators (register q of a lane: row 4 q + lane / 16, column lane % 16 of the block)
// go to a tile in LDS in the result's memory order, and the workgroup writes the tiles of its entries, one contiguous
// range of the result, in whole lines with non-temporal stores.
auto Generator::ProductPattern(const Sub &s, ProductShape &p) const -> bool
{
    if (envInt("ACRO_HIP_PRODUCT") < 0 || opt.no_matrix_cores || batch < 0 || !opt.noalias || NumGatherSlots() > 0) return false;
    if (mk.GetNumKernels() != 1 || s.matrixOp != 0 || s.out.repeated || s.in.size() != 2 || s.contr.size() != 1) return false;
    // (an element matrix applied to an element vector, "A_e_r = R_e_r_k X_e_k", is the product with a single column)
    const bool vectorForm = s.out.idx.size() == 2;
    if ((s.out.idx.size() != 3 && !vectorForm) || s.out.idx[0] != batch) return false;
    const int k = s.contr[0], r = s.out.idx[1], c = vectorForm ? -1 : s.out.idx[2];
    for (const auto &v : s.in)
    {
        if (vectorForm && !v.repeated && v.idx.size() == 2 && v.idx[0] == batch && v.idx[1] == k && !p.col && v.uvar != s.out.uvar &&
            !(uvars[v.uvar].storage >= 0 && uvars[v.uvar].storage == uvars[s.out.uvar].storage))
        {
            p.col = &v;
            p.colKFast = true;
            continue;
        }
        if (v.repeated || v.idx.size() != 3 || v.idx[0] != batch) return false;
        // (the pattern is also asked for while the model is being built, before storages are known)
        if (v.uvar == s.out.uvar || (uvars[v.uvar].storage >= 0 && uvars[v.uvar].storage == uvars[s.out.uvar].storage)) return false;
        const bool kLast = v.idx[2] == k, kFirst = v.idx[1] == k;
        if (!kLast && !kFirst) return false;
        const int other = kLast ? v.idx[1] : v.idx[2];
        if (other == r && !p.row)
        {
            p.row = &v;
            p.rowKFast = kLast;
        }
        else if (other == c && !p.col)
        {
            p.col = &v;
            p.colKFast = kLast;
        }
        else
            return false;
    }
    if (!p.row || !p.col) return false;
    p.M = extent[r];
    p.N = vectorForm ? 1 : extent[c];
    p.K = extent[k];
    p.E = extent[batch];
    if (vectorForm)
    {
        // Rows that are no whole number of 32-byte pieces (27 x 27, 25 x 25, 45 x 45): with the lanes along the rows a
        // wavefront reads its matrices in pieces of a row that start anywhere in a line (47 - 59 % of the HBM peak with
        // any of the vector-ALU schedules).  Here every strip of 16 rows is one contiguous range read front to back, and
        // the 15 unused columns of the matrix instruction cost nothing that shows: 27 x 27 needs 14 instructions per
        // entry, 48 us of matrix time for 127 us of memory time.  Rows of a multiple of four doubles keep the lanes that
        // share a contraction (69 - 76 %).
        if (!p.rowKFast || envInt("ACRO_HIP_PRODUCT_VECTOR") < 0) return false;
        // (rotated tensors, % of the HBM peak, two-step vector-ALU schedule / this one: 27 x 27 57 / 67, 25 x 25 58 / 63,
        // 31 x 31 57 / 70, 45 x 45 59 / 70, 63 x 63 58 / 73, 64 x 27 60 / 74, 27 x 45 58 / 72; short rows the other way
        // round: 21 x 21 62 / 52, 17 x 17 60 / 38, 13 x 13 59 / 56, 9 x 9 63 / 35)
        if ((p.K % 4 == 0 && envInt("ACRO_HIP_PRODUCT_VECTOR") < 2) || p.K < 25 || p.K > 128 || p.M < 16 || p.M > 128) return false;
    }
    // From 17 rows or columns on (up to 16 x 16 the staged schedule has a lane per output and is bound by memory);
    // a wavefront holds one strip of at most eight column blocks, an entry at most eight strips.
    const long lo = envInt("ACRO_HIP_PRODUCT_FROM", 17), hi = envInt("ACRO_HIP_PRODUCT_TO", 64);
    if (!vectorForm && (std::max(p.M, p.N) < lo || p.M > hi || p.N > hi || p.K > 128 || p.K < 8 || p.M < 8 || p.N < 8)) return false;
    // Up to 36 x 36 the staged vector-ALU schedule is as fast or a little faster where it can give a lane a block of
    // outputs, i.e. where both extents have a divisor 2, 3 or 5 (rotated buffers, % of the HBM peak, staged / here:
    // 20 x 20 75 / 71, 24 x 24 75 / 72, 25 x 25 74 / 71, 28 x 28 74 / 73, 33 x 33 67 / 64, 36 x 36 71 / 70; without such
    // a divisor 17 x 17 59 / 67, 31 x 31 42 / 71, 37 x 37 37 / 70; larger: 40 x 40 69 / 69, 45 x 45 67 / 69, 48 x 48 69 / 70,
    // 53 x 53 28 / 68, 55 x 55 23 / 68, 56 x 56 58 / 69, 63 x 63 32 / 67, 64 x 64 15 / 70).
    // Blocks of 3 x 3 are the staged schedule's weakest, and up to 32 x 32 (two strips of two blocks here) extents that only
    // three divides do better on the matrix cores: 21 x 21 64 / 70, 27 x 27 61 / 71, 27 x 27 x 9 terms 54 / 73,
    // 21 x 33 x 27 terms 69 / 72.
    auto blocks = [](long n) { return n % 2 == 0 || n % 3 == 0 || n % 5 == 0; };
    auto byThreeOnly = [](long n) { return n % 3 == 0 && n % 2 != 0 && n % 5 != 0; };
    // Whole blocks of 16 (32 x 32, 32 x 16) leave nothing of the matrix instruction unused and take it too: 32 x 32 72 / 74,
    // with the second factor transposed 61 / 73, with both 67 / 73.
    const bool staged = std::max(p.M, p.N) <= 36 && blocks(p.M) && blocks(p.N) &&
                        !(std::max(p.M, p.N) <= 32 && (byThreeOnly(p.M) || byThreeOnly(p.N))) && !(p.M % 16 == 0 && p.N % 16 == 0);
    if (!vectorForm && staged && envInt("ACRO_HIP_PRODUCT") < 2) return false;
    // A side of fewer than 16 leaves half and more of the matrix instruction's columns (or rows) empty; where the staged
    // schedule can hold both factors in LDS it is ahead then (from HBM, % of the HBM peak, here / staged: 64 x 8 by 8 x 8
    // 57 / 76, 48 x 8 by 8 x 8 58 / 74, 64 x 8 by 8 x 12 60 / 71, 8 x 8 by 8 x 64 78 / 84, 12 x 8 by 8 x 48 77 / 80,
    // 64 x 32 by 32 x 8 68 / 80, 40 x 16 by 16 x 10 68 / 75; 8 x 32 by 32 x 64 80 / 76).
    // (measured up to 32 terms)
    if (!vectorForm && std::min(p.M, p.N) < 16 && p.K <= 32 && (p.M + p.N) * p.K <= 4000 && envInt("ACRO_HIP_PRODUCT") < 2) return false;
    p.TI = (p.M + 15) / 16;
    p.TJ = (p.N + 15) / 16;
    if (p.TI > 8 || p.TJ > 8) return false;
    // The row factor goes into registers strip by strip, each wavefront its own 16 rows.  Straight from device memory
    // where a wavefront's loads fall on whole lines: rows of a multiple of 128 bytes read along the contracted index in
    // pairs (mode 0), or blocks of 16 rows read across it, 128 contiguous bytes per term (mode 1).  Otherwise (mode 2)
    // the strip, one contiguous range of device memory, is read front to back and passes through a piece of LDS of the
    // wavefront's own, which the column factor's fragments take over afterwards.
    // (View offsets are known only once the model is complete, and whether the schedule applies must not depend on
    // them: the size test takes the larger footprint.)
    p.rowMode = !p.rowKFast ? 1 : (p.K % 16 == 0 && uvars[p.row->uvar].viewOffset % 2 == 0 && envInt("ACRO_HIP_PRODUCT_DIRECT") >= 0 ? 0 : 2);
    p.pairMap = p.rowMode == 0;
    p.steps = p.pairMap ? 2 * ((p.K + 7) / 8) : (p.K + 3) / 4;
    const long stepsMost = 2 * ((p.K + 7) / 8);
    if (std::max<long>(std::max(p.TI, p.TJ) * stepsMost * 64, p.M * p.N) * 8 > 64 * 1024) return false;
    const long perEntry = std::max<long>(std::max<long>(p.rowMode == 2 ? p.TI : 0, p.TJ) * p.steps * 64, p.M * p.N);
    // entries per workgroup: up to four wavefronts, 64 KB of LDS (fragments of the factors, then the result tiles)
    p.NBE = std::max<long>(1, std::min<long>(4 / p.TI, (64 * 1024 / 8) / perEntry));
    if (envInt("ACRO_HIP_PRODUCT_ENTRIES") > 0) p.NBE = std::min<long>(envInt("ACRO_HIP_PRODUCT_ENTRIES"), (64 * 1024 / 8) / perEntry);
    p.NBE = std::min(p.NBE, p.E);
    p.ldsPerEntry = perEntry;
    return true;
}

auto Generator::UseProductSchedule() const -> bool
{
    ProductShape p;
    return subs.size() == 1 && ProductPattern(subs[0], p);
}

auto Generator::EmitProduct(HipKernelPlan &plan) -> void
{
    const Sub &s = subs[0];
    ProductShape p;
    ProductPattern(s, p);
    const long M = p.M, N = p.N, K = p.K, E = p.E, TI = p.TI, TJ = p.TJ, steps = p.steps, NBE = p.NBE;
    const long NW = NBE * TI, NT = NW * 64, MN = M * N, LT = TI * 64;   // LT: lanes that share an entry
    const long groups = (E + NBE - 1) / NBE;
    const long ldsDoublesHere = NBE * p.ldsPerEntry;
    const std::string dimName = mk.GetDimensionedNameString();
    char hex[32];
    std::snprintf(hex, sizeof(hex), "%016llx",
                  static_cast<unsigned long long>(hashString(dimName + "/product/" + (Positional() ? "p" : "u") + str(NBE) +
                                                             str(p.rowMode))));
    plan.module_name = std::string("acro_prod_") + hex;

    std::ostringstream sched;
    sched << "product schedule on the FP64 matrix cores: " << M << " x " << K << " by " << K << " x " << N << " per entry (row factor "
          << (p.rowKFast ? "with the contracted index last" : "with the contracted index first")
          << (p.rowMode == 2 ? ", strips through LDS" : ", read straight into registers") << "; column factor "
          << (p.colKFast ? "with the contracted index last" : "with the contracted index first") << ", through LDS), " << TI
          << " strips of 16 rows x " << TJ << " blocks of 16 columns, " << steps << " steps of four terms" << (p.pairMap ? " (terms in pairs)" : "")
          << ", " << NBE << (NBE == 1 ? " entry" : " entries") << " per workgroup of " << NT << " lanes, LDS " << ldsDoublesHere * 8
          << " bytes, results written out through LDS\n  [0] " << s.text << "\n";
    plan.schedule = sched.str();
    out << "// Generated by the acrotensor HIP code generator for gfx950.\n";
    {
        std::istringstream lines(plan.schedule);
        std::string l;
        while (std::getline(lines, l)) out << "// " << l << "\n";
    }
    const std::string R = PtrName(p.row->uvar), C = PtrName(p.col->uvar), A = PtrName(s.out.uvar);
    const long rOff = uvars[p.row->uvar].viewOffset, cOff = uvars[p.col->uvar].viewOffset, aOff = uvars[s.out.uvar].viewOffset;

    // term of step s for term group g, and step / group of term k
    auto termOf = [&](const std::string &step) {
        return p.pairMap ? "(8 * ((" + step + ") / 2) + 2 * g + (" + step + ") % 2)" : "(4 * (" + step + ") + g)";
    };
    const std::string stepOfK = p.pairMap ? "(2 * (k / 8) + k % 2)" : "(k / 4)";
    const std::string groupOfK = p.pairMap ? "((k % 8) / 2)" : "(k % 4)";

    // A factor's matrix of one entry is one contiguous range of device memory: the lanes of the entry read it front to
    // back from the line boundary at or before its first double, 16 bytes each, and put every value where the matrix
    // instruction will want it: fragment (block of 16 rows or columns, step), term group, and within the group of 16
    // a place that depends on row and term (acro_place), which spreads the values that a wavefront writes at once, a
    // run along either dimension of the matrix, over the banks (the readers undo the permutation).
    struct Staged
    {
        std::string ptr, name;
        long offset, rows, kFast, base, blocks;
    };
    std::vector<Staged> staged;
    staged.push_back({C, "c", cOff, N, p.colKFast ? 1 : 0, 0, TJ});
    // the strip of the row factor (mode 2): 16 rows of K doubles, read by the one wavefront that owns it
    long stripIts = 0;
    if (p.rowMode == 2)
    {
        long lead = 0;
        for (long en = 0; en < 16; ++en)
            for (long st = 0; st < TI; ++st) lead = std::max(lead, (rOff + (en * M + 16 * st) * K) % 16);
        stripIts = ((16 * K + lead + 1) / 2 + 63) / 64;
    }
    // 16-byte pieces per lane: the matrix and the most doubles that can lie between a line boundary and its first one
    auto itsOf = [&](const Staged &f) {
        long lead = 0;
        for (long en = 0; en < 16; ++en) lead = std::max(lead, (f.offset + en * f.rows * K) % 16);
        return ((f.rows * K + lead + 1) / 2 + LT - 1) / LT;
    };

    // loads of the factors of the workgroup's entries into registers (no branches around the single loads: all of them
    // are in flight together.  A pair that would reach past the end of the tensor is replaced by the last whole pair,
    // whose values are then not used; the last double of a tensor of odd length is read on its own.)
    auto emitLoads = [&](const std::string &eg, const std::string &ind) {
        out << ind << "{\n";
        out << ind << "    const long en = (" << eg << ") * " << NBE << " + slot < " << E << " ? (" << eg << ") * " << NBE << " + slot : " << E - 1 << ";\n";
        for (const Staged &f : staged)
        {
            const long size = f.rows * K, tensorEnd = f.offset + E * size, lastPair = (tensorEnd - 2) & ~1L;
            out << ind << "    const long " << f.name << "First = (" << f.offset << "L + en * " << size << "L) & ~15L;\n";
            out << "#pragma unroll\n" << ind << "    for (int it = 0; it < " << itsOf(f) << "; ++it)\n" << ind << "    {\n";
            out << ind << "        const long at = " << f.name << "First + 2 * (it * " << LT << " + lt);\n";
            // (factors that are whole 128-byte lines per entry are read once, by load instructions that take whole lines:
            // with the non-temporal hint 32 x 32 products 73.5 -> 78 % of the HBM peak from HBM, 48 x 48 72 -> 76 %, 64 x 64
            // 72 -> 75 %, re-launched on tensors that the memory-side cache holds in part 86 -> 82 %; factors whose entries
            // share lines, and the vectors of the operator schedule, which a wavefront reads in 64-byte pieces, lose by it)
            const bool nt = envInt("ACRO_HIP_PRODUCT_NT") >= 0 && size % 16 == 0 && f.offset % 16 == 0;
            out << ind << "        " << f.name << "v[it] = " << (nt ? "__builtin_nontemporal_load(" : "*") << "reinterpret_cast<const acro_pair *>(" << f.ptr << " + (at < " << lastPair << "L ? at : " << lastPair << "L))" << (nt ? ")" : "") << ";\n";
            if (tensorEnd % 2 != 0)
                out << ind << "        if (at == " << tensorEnd - 1 << "L) " << f.name << "v[it].x = " << f.ptr << "[" << tensorEnd - 1 << "L];\n";
            out << ind << "    }\n";
        }
        if (p.rowMode == 2)
        {
            const long tensorEnd = rOff + E * M * K, lastPair = (tensorEnd - 2) & ~1L;
            out << ind << "    const long rFirst = (" << rOff << "L + (en * " << M << " + 16 * strip) * " << K << "L) & ~15L;\n";
            out << "#pragma unroll\n" << ind << "    for (int it = 0; it < " << stripIts << "; ++it)\n" << ind << "    {\n";
            out << ind << "        const long at = rFirst + 2 * (it * 64 + lane);\n";
            const bool nt = envInt("ACRO_HIP_PRODUCT_NT") >= 0 && (M * K) % 16 == 0 && rOff % 16 == 0;
            out << ind << "        rv[it] = " << (nt ? "__builtin_nontemporal_load(" : "*") << "reinterpret_cast<const acro_pair *>(" << R << " + (at < " << lastPair << "L ? at : " << lastPair << "L))" << (nt ? ")" : "") << ";\n";
            if (tensorEnd % 2 != 0)
                out << ind << "        if (at == " << tensorEnd - 1 << "L) rv[it].x = " << R << "[" << tensorEnd - 1 << "L];\n";
            out << ind << "    }\n";
        }
        else
        {
            out << ind << "    const double *rm = " << R << " + " << rOff << "L + en * " << M * K << "L;\n";
            out << ind << "    const int m = 16 * strip + c < " << M << " ? 16 * strip + c : " << M - 1 << ";\n";
            if (p.rowKFast)
            {
                out << "#pragma unroll\n" << ind << "    for (int u = 0; u < " << steps / 2 << "; ++u)\n" << ind << "    {\n";
                out << ind << "        const int k = 8 * u + 2 * g;\n";
                out << ind << "        acro_pair v = {0.0, 0.0};\n";
                out << ind << "        if (k < " << K << ") v = *reinterpret_cast<const acro_pair *>(rm + m * " << K << " + k);\n";
                out << ind << "        a[2 * u] = v.x;\n" << ind << "        a[2 * u + 1] = v.y;\n" << ind << "    }\n";
            }
            else
            {
                out << "#pragma unroll\n" << ind << "    for (int s = 0; s < " << steps << "; ++s)\n" << ind << "    {\n";
                out << ind << "        const int k = " << termOf("s") << ";\n";
                out << ind << "        a[s] = k < " << K << " ? rm[k * " << M << " + m] : 0.0;\n" << ind << "    }\n";
            }
        }
        out << ind << "}\n";
    };

    out << "typedef double acro_double4 __attribute__((ext_vector_type(4)));\n";
    out << "typedef double acro_pair __attribute__((ext_vector_type(2)));\n";
    // the place of (row or column x, term k) within its group of 16: x and k each go through v -> v / 2 + 8 (v mod 2),
    // so that 16 lanes that write every second x at one k, or every second k at one x (the halves of 16-byte pieces
    // along either dimension), and 16 lanes that read 16 consecutive x at one k all fall on different banks
    // (runs of odd length change the parity of x or k from one row to the next, and there the plain rotation by x + k
    // measured faster: 53 x 53 68 against 61 % of the HBM peak, 34 x 34 the other way round 65 against 72 %)
    out << "__device__ static inline int acro_place(int x, int k) { return ((x >> 1) + 8 * (x & 1) + (k >> 1) + 8 * (k & 1)) & 15; }\n";
    out << "__device__ static inline int acro_place_odd(int x, int k) { return (x + k) & 15; }\n";
    const std::string rowPlace = K % 2 == 0 ? "acro_place" : "acro_place_odd";
    const std::string colPlace = (p.colKFast ? K : N) % 2 == 0 ? "acro_place" : "acro_place_odd";
    out << "\nextern \"C\" __global__ __launch_bounds__(" << NT << ") void " << plan.module_name << "(" << ParamList() << ")\n{\n";
    out << "    __shared__ double lds[" << ldsDoublesHere << "];\n";
    out << "    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, c = lane & 15, g = lane >> 4;\n";
    out << "    const int slot = wave / " << TI << ", strip = wave % " << TI << ", lt = strip * 64 + lane;   // lt: lane among those of the entry\n";
    out << "    double *frag = lds + slot * " << p.ldsPerEntry << ";\n";
    for (const Staged &f : staged) out << "    acro_pair " << f.name << "v[" << itsOf(f) << "];\n";
    if (p.rowMode == 2) out << "    acro_pair rv[" << stripIts << "];\n";
    out << "    double a[" << steps << "];\n";
    emitLoads("(long)blockIdx.x", "    ");
    out << "    {\n";
    out << "        const long e0 = (long)blockIdx.x * " << NBE << ";\n";
    out << "        const long e = e0 + slot < " << E << " ? e0 + slot : " << E - 1 << ";   // (a slot past the last entry repeats it; nothing of it is stored)\n";
    // terms past the end read as zero: the places of the last step(s) whose term does not exist
    long np = 0;
    std::string sOfW, gOfW;
    if (p.pairMap && K % 8 != 0)
    {
        np = 2 * (4 - (K % 8) / 2);
        sOfW = str(steps - 2) + " + w % 2";
        gOfW = str((K % 8) / 2) + " + w / 2";
    }
    else if (!p.pairMap && K % 4 != 0)
    {
        np = 4 - K % 4;
        sOfW = str(steps - 1);
        gOfW = str(K % 4) + " + w";
    }
    if (p.rowMode == 2)
    {
        // ---- the strip: to the fragments of this wavefront's block of rows, and from there into its registers
        out << "        {\n            double *fr = frag + strip * " << steps * 64 << ";\n";
        out << "            const long base = " << rOff << "L + (e * " << M << " + 16 * strip) * " << K << "L;\n";
        out << "            const int lead = (int)(base - (base & ~15L));   // doubles between the line boundary and the strip\n";
        out << "            const int size = (" << M << " - 16 * strip < 16 ? " << M << " - 16 * strip : 16) * " << K << ";\n";
        out << "#pragma unroll\n            for (int it = 0; it < " << stripIts << "; ++it)\n            {\n";
        out << "#pragma unroll\n                for (int h = 0; h < 2; ++h)\n                {\n";
        out << "                    const int j = 2 * (it * 64 + lane) + h - lead;\n";
        out << "                    if (j < 0 || j >= size) continue;\n";
        out << "                    const int x = j / " << K << ", k = j % " << K << ";\n";
        out << "                    fr[" << stepOfK << " * 64 + " << groupOfK << " * 16 + " << rowPlace << "(x, k)] = h == 0 ? rv[it].x : rv[it].y;\n";
        out << "                }\n            }\n";
        if (np > 0)
        {
            out << "            for (int z = lane; z < " << np * 16 << "; z += 64)\n            {\n";
            out << "                const int w = z / 16;\n";
            out << "                fr[(" << sOfW << ") * 64 + (" << gOfW << ") * 16 + (z & 15)] = 0.0;\n            }\n";
        }
        // (a wavefront's LDS accesses complete in program order: no workgroup barrier between its writes and its reads)
        out << "            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, \"wavefront\");\n            __builtin_amdgcn_wave_barrier();\n";
        out << "#pragma unroll\n            for (int s = 0; s < " << steps << "; ++s) a[s] = fr[s * 64 + g * 16 + " << rowPlace << "(c, " << termOf("s") << ")];\n";
        out << "        }\n";
        out << "        __syncthreads();   // every strip is in registers: the column factor's fragments take the place\n";
    }
    // ---- staged values to their fragments
    for (const Staged &f : staged)
    {
        const long size = f.rows * K;
        out << "        {\n            double *fr = frag + " << f.base << ";\n";
        out << "            const long base = " << f.offset << "L + e * " << size << "L;\n";
        out << "            const int lead = (int)(base - (base & ~15L));   // doubles between the line boundary and the matrix\n";
        out << "#pragma unroll\n            for (int it = 0; it < " << itsOf(f) << "; ++it)\n            {\n";
        out << "#pragma unroll\n                for (int h = 0; h < 2; ++h)\n                {\n";
        out << "                    const int j = 2 * (it * " << LT << " + lt) + h - lead;\n";
        out << "                    if (j < 0 || j >= " << size << ") continue;\n";
        if (f.kFast)
            out << "                    const int x = j / " << K << ", k = j % " << K << ";\n";
        else
            out << "                    const int k = j / " << f.rows << ", x = j % " << f.rows << ";\n";
        out << "                    fr[((x / 16) * " << steps << " + " << stepOfK << ") * 64 + " << groupOfK << " * 16 + " << colPlace << "(x, k)] = h == 0 ? "
            << f.name << "v[it].x : " << f.name << "v[it].y;\n";
        out << "                }\n            }\n";
        if (np > 0)
        {
            out << "            for (int z = lt; z < " << f.blocks * np * 16 << "; z += " << LT << ")\n            {\n";
            out << "                const int blk = z / " << np * 16 << ", w = (z / 16) % " << np << ";\n";
            out << "                fr[(blk * " << steps << " + " << sOfW << ") * 64 + (" << gOfW << ") * 16 + (z & 15)] = 0.0;\n            }\n";
        }
        out << "        }\n";
    }
    out << "        acro_double4 acc[" << TJ << "];\n";
    out << "#pragma unroll\n        for (int J = 0; J < " << TJ << "; ++J) acc[J] = acro_double4{0.0, 0.0, 0.0, 0.0};\n";
    out << "        __syncthreads();\n";
    out << "#pragma unroll\n        for (int s = 0; s < " << steps << "; ++s)\n        {\n";
    out << "            const int k = " << termOf("s") << ";   // this lane's term in step s\n";
    out << "#pragma unroll\n            for (int J = 0; J < " << TJ << "; ++J)\n";
    out << "                acc[J] = __builtin_amdgcn_mfma_f64_16x16x4f64(a[s], frag[(J * " << steps << " + s) * 64 + g * 16 + " << colPlace << "(16 * J + c, k)], acc[J], 0, 0, 0);\n";
    out << "        }\n";
    out << "        __syncthreads();   // every fragment has been read: the tiles of the results take their place\n";
    out << "        {\n";
    out << "            double *tile = lds + slot * " << MN << ";\n";
    out << "#pragma unroll\n            for (int J = 0; J < " << TJ << "; ++J)\n";
    out << "#pragma unroll\n                for (int q = 0; q < 4; ++q)\n                {\n";
    out << "                    const int m = 16 * strip + 4 * q + g, n = 16 * J + c;\n";
    out << "                    if (m < " << M << " && n < " << N << ") tile[m * " << N << " + n] = acc[J][q];\n";
    out << "                }\n        }\n";
    out << "        __syncthreads();\n";
    out << "        {   // LDS tiles -> device memory: the entries of the workgroup are one contiguous range; 16 bytes per lane, whole lines per instruction\n";
    out << "            const int count = (int)(" << E << " - e0 < " << NBE << " ? " << E << " - e0 : " << NBE << ") * " << MN << ";\n";
    out << "            const long base = " << aOff << "L + e0 * " << MN << "L, first = base & ~15L;\n";
    const bool streams = s.op == '=' && envInt("ACRO_HIP_NT_STORE") >= 0;
    const std::string combine = s.op == '=' ? "" : (s.op == '+' ? "+" : "-");
    out << "            for (int i = threadIdx.x; 2 * i < count + 15; i += " << NT << ")\n            {\n";
    out << "                const long at = first + 2 * i;\n";
    out << "                const int j = (int)(at - base);\n";
    out << "                if (j >= 0 && j + 1 < count)\n                {\n";
    out << "                    acro_pair v = {lds[j], lds[j + 1]};\n";
    out << "                    acro_pair *d = reinterpret_cast<acro_pair *>(" << A << " + at);\n";
    if (s.op == '=')
        out << "                    " << (streams ? "__builtin_nontemporal_store(v, d);" : "*d = v;") << "\n";
    else
        out << "                    *d = *d " << combine << " v;\n";
    out << "                }\n                else\n                {\n";
    for (int h = 0; h < 2; ++h)
    {
        const std::string jj = h == 0 ? "j" : "j + 1", aa = h == 0 ? "at" : "at + 1";
        out << "                    if (" << jj << " >= 0 && " << jj << " < count) " << A << "[" << aa << "] = "
            << (s.op == '=' ? "" : A + "[" + aa + "] " + combine + " ") << "lds[" << jj << "];\n";
    }
    out << "                }\n            }\n";
    out << "        }\n";
    out << "    }\n}\n";

    plan.source = out.str();
    plan.nb = static_cast<int>(NBE);
    plan.lds_bytes = static_cast<int>(ldsDoublesHere * 8);
    FillParams(plan, false);
    HipLaunch launch;
    launch.function_name = plan.module_name;
    launch.grid = static_cast<unsigned>(groups);
    launch.block = static_cast<unsigned>(NT);
    for (int si = 0; si < NumParamStores(); ++si) launch.params.push_back(si);
    plan.launches.push_back(launch);
}

// ---------------------------------------------------------------------------------------------- tiled products
// Matrix products beyond what one workgroup can hold: "A_e_r_c (=|+=|-=) R_e_{r,k} C_e_{k,c}" with more than 64 rows or
// columns or more than 128 terms, and the same without a batch index ("A_i_j = B_i_k C_k_j", a plain matrix product).
// The reference gives every output a thread that walks the contracted index through device memory
// (exec/CudaExecutor.cpp:193-263); so did the generic schedule here (128 x 128 per entry: 6 % of the HBM peak,
// 2 048 x 2 048 unbatched: 4.8 TFLOP/s).
//
// A workgroup of W wavefronts owns a tile of 16 W rows by 16 TJ columns of one entry's result: wavefront w the strip of 16
// rows number w, TJ accumulator blocks of v_mfma_f64_16x16x4.  The contracted index is walked in chunks of KC terms.  Per
// chunk the workgroup reads a 16 W x KC piece of the row factor and a KC x 16 TJ piece of the column factor, each lane
// single doubles with the lanes along the factor's fastest dimension, into registers; writes them to LDS in the order
// the instruction wants its operands (fragment = block of 16 rows or columns and step of four terms; within a group of
// 16 the place (x + k) mod 16, which keeps the 16 lanes that write a run along either dimension, and the 16 that read,
// on different banks); and requests the next chunk before it multiplies this one, so that device memory is busy while
// the matrix cores are.  Rows, columns and terms past the end are zero in LDS; results past the end are not stored.
// Result register q of a lane holds row 4 q + lane / 16 and column lane % 16 of its block: a store instruction
// writes four runs of 128 bytes.
auto Generator::TiledProductPattern(const Sub &s, TiledProductShape &p) const -> bool
{
    if (envInt("ACRO_HIP_TILED_PRODUCT") < 0 || opt.no_matrix_cores || !opt.noalias || NumGatherSlots() > 0) return false;
    if (mk.GetNumKernels() != 1 || s.matrixOp != 0 || s.out.repeated || s.in.size() != 2 || s.contr.size() != 1) return false;
    const size_t rank = s.out.idx.size();
    if (rank != 2 && rank != 3) return false;
    p.batched = rank == 3;
    const int entry = p.batched ? s.out.idx[0] : -1;   // (need not be the index that the other schedules would batch over)
    const int k = s.contr[0], r = s.out.idx[rank - 2], c = s.out.idx[rank - 1];
    for (const auto &v : s.in)
    {
        if (v.repeated || v.idx.size() != rank || (p.batched && v.idx[0] != entry)) return false;
        if (v.uvar == s.out.uvar || (uvars[v.uvar].storage >= 0 && uvars[v.uvar].storage == uvars[s.out.uvar].storage)) return false;
        const bool kLast = v.idx[rank - 1] == k, kFirst = v.idx[rank - 2] == k;
        if (!kLast && !kFirst) return false;
        const int other = kLast ? v.idx[rank - 2] : v.idx[rank - 1];
        if (other == r && !p.row)
        {
            p.row = &v;
            p.rowKFast = kLast;
        }
        else if (other == c && !p.col)
        {
            p.col = &v;
            p.colKFast = kLast;
        }
        else
            return false;
    }
    if (!p.row || !p.col) return false;
    p.M = extent[r];
    p.N = extent[c];
    p.K = extent[k];
    p.E = p.batched ? extent[entry] : 1;
    // (fewer than 16 rows or columns only with a long contracted range and 64 outputs or more: most of a matrix
    // instruction is padding then, but memory bounds such a product, and the reduction schedule takes only some of them
    // (15 x 15 and 8 x 31 outputs over 10^6 terms were left to the generic schedule, which gives the range to single lanes:
    // 110 ms); where both apply they measure alike (8 x 32 here 181 us, 4 x 32 there 155 us, 16 x 8 there 378 us))
    const bool longRange = p.K >= 1024 && p.M * p.N >= 64 && std::min(p.M, p.N) >= 2;
    if (((p.M < 16 || p.N < 16) && !longRange) || p.K < 16 || p.M * p.K >= (1L << 31) || p.N * p.K >= (1L << 31) || p.M * p.N >= (1L << 31)) return false;
    // (smaller matrices per entry have the schedules above; an unbatched product must be worth a launch of its own)
    const long from = envInt("ACRO_HIP_TILED_PRODUCT_FROM", 65);
    if (p.batched && std::max(p.M, p.N) < from && p.K <= 128) return false;
    // (... or have a long contracted range, which the generic schedule would give to single lanes: 32 x 32 outputs over
    // 10^6 terms 102 ms there, 0.1 % of the HBM peak)
    if (!p.batched && p.M * p.N < 64 * 64 && p.K < 1024) return false;
    // (one factor small enough for LDS in one piece: that is a dense operator applied to many vectors, "A_e_i = B_i_j X_e_j",
    // which the operator schedule streams at 64 - 86 % of the HBM peak)
    if (!p.batched && std::min(p.M, p.N) * p.K <= envInt("ACRO_HIP_TILED_PRODUCT_OPERATOR", 4096)) return false;
    // strips per workgroup and blocks per strip: as even a split of the result as eight of each allow
    const long strips = (p.M + 15) / 16, blocks = (p.N + 15) / 16;
    // The split wastes as little of the matrix instruction on padding as it can.  Among equals: four blocks per strip
    // rather than more (32 accumulator registers: two workgroups of eight wavefronts fit a compute unit, and one starts
    // or drains while the other multiplies; with eight blocks one fits.  128 x 128 x 128 per entry: 52 against 43 % of
    // the HBM peak).
    auto split = [](long units, long lo, long hi, long preferred, long &parts, long &each) {
        double best = 1e30;
        for (long n = lo; n <= hi; ++n)
        {
            const long m = (units + n - 1) / n;
            const double cost = static_cast<double>(m * n) * (n > preferred ? 1.15 : 1.0) - 1e-3 * n;
            if (units <= n && n > units) continue;   // (never more than there is)
            if (cost < best)
            {
                best = cost;
                parts = m;
                each = n;
            }
        }
        if (units < lo)
        {
            parts = 1;
            each = units;
        }
    };
    const long mostW = envInt("ACRO_HIP_TILED_PRODUCT_STRIPS") > 0 ? envInt("ACRO_HIP_TILED_PRODUCT_STRIPS") : 8;
    const long mostJ = envInt("ACRO_HIP_TILED_PRODUCT_BLOCKS") > 0 ? envInt("ACRO_HIP_TILED_PRODUCT_BLOCKS") : 8;
    split(blocks, std::min<long>(3, mostJ), mostJ, envInt("ACRO_HIP_TILED_PRODUCT_PREFER", 4), p.panels, p.TJ);
    // (strips: up to 12 of them, four per workgroup rather than more: 128^3 per entry 57 -> 59 %, 125^3 45 -> 48 %, 192^3
    // 30.5 -> 38 %; from 13 on, as many as possible: 256^3 31.5 against 30.4 %, and the large products without a batch index)
    split(strips, std::min<long>(4, mostW), mostW, strips <= 12 ? 4 : 8, p.tilesM, p.W);
    // (few workgroups, a product without a batch index of moderate size: tiles of half the height fill the device better;
    // 1 024 x 1 024 x 1 024: 14.5 -> 31.6 TFLOP/s)
    if (p.E * p.tilesM * p.panels < 512 && p.W > 4 && mostW > 4 && envInt("ACRO_HIP_TILED_PRODUCT_HALF") >= 0) split(strips, 4, 4, 4, p.tilesM, p.W);
    p.KC = envInt("ACRO_HIP_TILED_PRODUCT_CHUNK") > 0 ? envInt("ACRO_HIP_TILED_PRODUCT_CHUNK") : 16;
    if (p.KC % 4 != 0 || p.KC > 64) return false;
    if (p.K < p.KC) p.KC = 16;   // (the end of a range is read as its last chunk's worth of terms)
    // Few tiles (normal equations "A_i_j = B_n_i C_n_j" with many columns, a product of two wide matrices, any product
    // without a batch index up to some 1 000 rows and columns): a workgroup passes through its chunks one after the
    // other, about a microsecond each while it has a SIMD to itself, and most of the device idles.  The contracted range
    // is split over workgroups as well, each writes its tile of partial sums to the scratch buffer, and a second kernel
    // adds them in a fixed order (reproducible, no atomics).  Every share costs a tile of partial sums written and read
    // (some 3 TB/s, they stay in the caches), so the number of shares balances the two, and a second launch (some 4 us) must
    // be worth it: no more shares than make three workgroups per compute unit (what its registers hold), at least two chunks each, at most 64 MB of
    // partial sums.  512 x 512 x 512: 34.6 -> 17.9 us, 256 x 256 x 256: 18.1 -> 9.9 us, 768 x 768 x 768: 52 -> 35 us,
    // 512 x 512 x 2048: 127 -> 35 us, 128 x 128 x 8192: 497 -> 20 us.
    p.splits = 1;
    const long groups = p.E * p.tilesM * p.panels, chunks = (p.K + p.KC - 1) / p.KC;
    const long asked = envInt("ACRO_HIP_TILED_PRODUCT_SPLIT");
    if (asked > 0) p.splits = std::min<long>(asked, chunks);
    else if (groups < 512 && chunks >= 4 && asked == 0)
    {
        // microseconds, roughly: one per chunk, the partial sums at 3 TB/s, four for the second launch
        const double perShare = 16.0 * static_cast<double>(p.E * p.M * p.N) / 3.0e6;
        const long most = std::min<long>(std::min<long>((768 + groups - 1) / groups, chunks / 2), 256);
        double best = static_cast<double>(chunks);
        for (long n = 2; n <= most; ++n)
        {
            const double cost = static_cast<double>((chunks + n - 1) / n) + static_cast<double>(n) * perShare + 4.0;
            if (cost < best - 1.0)
            {
                best = cost;
                p.splits = n;
            }
        }
    }
    while (p.splits > 1 && p.splits * p.E * p.M * p.N > (1L << 23)) --p.splits;
    return true;
}

auto Generator::UseTiledProductSchedule() const -> bool
{
    TiledProductShape p;
    return subs.size() == 1 && TiledProductPattern(subs[0], p);
}

auto Generator::EmitTiledProduct(HipKernelPlan &plan) -> void
{
    const Sub &s = subs[0];
    TiledProductShape p;
    TiledProductPattern(s, p);
    const long M = p.M, N = p.N, K = p.K, E = p.E, W = p.W, TJ = p.TJ, KC = p.KC, KS = KC / 4, NT = 64 * W;
    const long tiles = p.tilesM * p.panels, groups = tiles * E, splits = p.splits;
    const long span = ((K + splits - 1) / splits + KC - 1) / KC * KC;   // terms per share of the contracted range
    const long rowTile = 16 * W * KC, colTile = 16 * TJ * KC;
    const long UA = (rowTile + NT - 1) / NT, UB = (colTile + NT - 1) / NT;
    const std::string dimName = mk.GetDimensionedNameString();
    char hex[32];
    std::snprintf(hex, sizeof(hex), "%016llx",
                  static_cast<unsigned long long>(hashString(dimName + "/tiled-product/" + (Positional() ? "p" : "u") + str(KC) + "/" + str(W) + "/" + str(TJ) + "/" + str(splits))));
    plan.module_name = std::string("acro_tprod_") + hex;

    std::ostringstream sched;
    sched << "tiled product schedule on the FP64 matrix cores: " << M << " x " << K << " by " << K << " x " << N
          << (p.batched ? " per entry, " + str(E) + " entries" : std::string(", no batch index")) << " (row factor "
          << (p.rowKFast ? "with the contracted index last" : "with the contracted index first") << ", column factor "
          << (p.colKFast ? "with the contracted index last" : "with the contracted index first") << "), tiles of " << 16 * W << " rows x "
          << 16 * TJ << " columns (" << p.tilesM << " x " << p.panels << " per entry), chunks of " << KC << " terms through "
          << (UA + UB) * NT * 8 << " bytes of LDS, " << groups * splits << " workgroups of " << NT << " lanes";
    if (splits > 1) sched << ", the contracted range in " << splits << " shares of " << span << " terms whose partial sums a second kernel adds";
    // Few workgroups per compute unit: a wavefront has its SIMD almost to itself, and what it issues beside the matrix
    // instructions shows.  Allowed all 512 registers of a SIMD lane (one wavefront per SIMD is enough for a workgroup of
    // 256 lanes), the compiler keeps the accumulators in the accumulation half of the register file inside the loop and in
    // the other half around its back edge, 64 copies per chunk; asked for at least two wavefronts per SIMD it has 256
    // registers, all of them ordinary ones, uses about 100 and makes no copies.  512^3 16.5 -> 15.4 us, 1 024^3 54 -> 47 us,
    // 1 536^3 183 -> 157 us, 144 x 128 x 100 000 105 -> 94 us; with many workgroups per compute unit the copies hide behind
    // other wavefronts and the other form loses a little (128^3 per entry 56.5 -> 54.6 % of the HBM peak), so those are
    // left to the compiler.
    // Not for products that memory bounds (fewer than 9.8 operations per byte of the factors: 64 x 64 x 500 000 130 -> 157 us)
    // nor for short ranges (128^3 on 16 entries: 8.7 -> 10.4 us).
    const bool vgprForm = groups * splits <= 1024 && W <= 4 && M * N >= 40 * (M + N) && K >= 256 && envInt("ACRO_HIP_TILED_PRODUCT_VGPR_FORM") >= 0;
    if (vgprForm) sched << ", at least two wavefronts per SIMD asked of the compiler";
    sched << "\n  [0] " << s.text << "\n";
    plan.schedule = sched.str();
    out << "// Generated by the acrotensor HIP code generator for gfx950.\n";
    {
        std::istringstream lines(plan.schedule);
        std::string l;
        while (std::getline(lines, l)) out << "// " << l << "\n";
    }
    const std::string R = PtrName(p.row->uvar), C = PtrName(p.col->uvar), A = PtrName(s.out.uvar);
    const long rOff = uvars[p.row->uvar].viewOffset, cOff = uvars[p.col->uvar].viewOffset, aOff = uvars[s.out.uvar].viewOffset;
    // Non-temporal stores where a store instruction's four runs of 16 doubles are whole lines; rows that 16 does not divide
    // start anywhere in a line, and the pieces of a line then meet in L2 (125 x 125: 36 -> 40 % of the HBM peak, 65 x 65 39 -> 42 %).
    const bool streams = s.op == '=' && envInt("ACRO_HIP_NT_STORE") >= 0 && N % 16 == 0 && aOff % 16 == 0;

    out << "typedef double acro_double4 __attribute__((ext_vector_type(4)));\n";
    out << "\nextern \"C\" __global__ __launch_bounds__(" << NT << ") ";
    if (envInt("ACRO_HIP_TILED_PRODUCT_WAVES") > 0) out << "__attribute__((amdgpu_waves_per_eu(" << envInt("ACRO_HIP_TILED_PRODUCT_WAVES") << "))) ";
    else if (vgprForm) out << "__attribute__((amdgpu_waves_per_eu(2))) ";
    const std::string fMain = splits > 1 ? plan.module_name + "_partial" : plan.module_name, fFinal = plan.module_name + "_final";
    out << "void " << fMain << "(" << ParamList() << (splits > 1 ? ", double *__restrict__ scratch" : "") << ")\n{\n";
    // (padded to a whole number of values per lane: lanes without a value of the tile write into the padding, no branch)
    out << "    __shared__ double fragA[" << UA * NT << "];\n";
    out << "    __shared__ double fragB[" << UB * NT << "];\n";
    out << "    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, c = lane & 15, g = lane >> 4;\n";
    if (splits > 1)
    {
        out << "    const int split = blockIdx.x / " << groups << ";\n    const long group = blockIdx.x % " << groups << ";\n";
        out << "    const int kBegin = split * " << span << ", kEnd = kBegin + " << span << " < " << K << " ? kBegin + " << span << " : " << K << ";\n";
    }
    else if (tiles > 1 && tiles <= 4 && p.batched && envInt("ACRO_HIP_TILED_PRODUCT_XCD") >= 0)
    {
        // The tiles of an entry read the same strips of the factors.  Hardware deals consecutive workgroup ids round-robin
        // to the eight XCDs, each with an L2 of its own: numbered as they come, the tiles of an entry would each fetch
        // their factors through another L2.  Workgroup b is on XCD b % 8 and is that XCD's number b / 8; the tiles of an
        // entry take consecutive numbers of one XCD.  (Rotated tensors, % of the HBM peak: 125^3 per entry 41 -> 44,
        // 216^3 26.5 -> 28, 100^3 37 -> 38.5, 128^3 53 -> 54; with eight tiles per entry, 256^3, 28 -> 26: left as it comes.)
        const long whole = groups / (8 * tiles) * (8 * tiles);
        out << "    const long b_ = blockIdx.x;\n";
        out << "    const long group = b_ >= " << whole << "L ? b_ : ((b_ / 8) / " << tiles << " * 8 + b_ % 8) * " << tiles << " + (b_ / 8) % " << tiles << ";\n";
        out << "    const int kBegin = 0, kEnd = " << K << ";\n";
    }
    else
        out << "    const long group = blockIdx.x;\n    const int kBegin = 0, kEnd = " << K << ";\n";
    out << "    const long e = group / " << tiles << ";\n";
    out << "    const int tile = (int)(group % " << tiles << "), r0 = tile / " << p.panels << " * " << 16 * W << ", c0 = tile % " << p.panels
        << " * " << 16 * TJ << ";\n";
    out << "    const double *Rm = " << R << " + " << rOff << "L + e * " << M * K << "L;\n";
    out << "    const double *Cm = " << C << " + " << cOff << "L + e * " << K * N << "L;\n";
    out << "    double *Am = " << A << " + " << aOff << "L + e * " << M * N << "L;\n";
    // Where this lane's values of a chunk come from and go to (the same for every chunk but for the term offset).  Rows and
    // columns past the end of the matrices read the last row or column instead: what they contribute to are results past
    // the end, which are not stored.  Lanes without a value of the tile (a tile of fewer values than a whole number per
    // lane) read the tile's first value and write into the padding of the LDS arrays.  So the loop has no lane-dependent
    // condition, and its loads take a scalar base that moves with the chunk plus a 32-bit offset per lane
    // (1 024 x 1 024 x 1 024 in 256 workgroups: 137 -> 75 other vector instructions per chunk, 67.6 -> 51.5 us).
    out << "    unsigned aFrom[" << UA << "], bFrom[" << UB << "];\n    int aTo[" << UA << "], bTo[" << UB << "];\n";
    out << "#pragma unroll\n    for (int u = 0; u < " << UA << "; ++u)\n    {\n";
    out << "        const int i = threadIdx.x + " << NT << " * u, v = i < " << rowTile << " ? i : 0;\n";
    if (p.rowKFast)
        out << "        const int kk = v % " << KC << ", rr = v / " << KC << ";\n";
    else
        out << "        const int rr = v % " << 16 * W << ", kk = v / " << 16 * W << ";\n";
    out << "        const int row = r0 + rr < " << M << " ? r0 + rr : " << M - 1 << ";\n";
    out << "        aFrom[u] = " << (p.rowKFast ? "row * " + str(K) + " + kk" : "kk * " + str(M) + " + row") << ";\n";
    out << "        aTo[u] = i < " << rowTile << " ? ((rr / 16) * " << KS << " + kk / 4) * 64 + (kk % 4) * 16 + ((rr + kk) & 15) : i;\n";
    out << "    }\n";
    out << "#pragma unroll\n    for (int u = 0; u < " << UB << "; ++u)\n    {\n";
    out << "        const int i = threadIdx.x + " << NT << " * u, v = i < " << colTile << " ? i : 0;\n";
    if (p.colKFast)
        out << "        const int kk = v % " << KC << ", cc = v / " << KC << ";\n";
    else
        out << "        const int cc = v % " << 16 * TJ << ", kk = v / " << 16 * TJ << ";\n";
    out << "        const int col = c0 + cc < " << N << " ? c0 + cc : " << N - 1 << ";\n";
    out << "        bFrom[u] = " << (p.colKFast ? "col * " + str(K) + " + kk" : "kk * " + str(N) + " + col") << ";\n";
    out << "        bTo[u] = i < " << colTile << " ? ((cc / 16) * " << KS << " + kk / 4) * 64 + (kk % 4) * 16 + ((cc + kk) & 15) : i;\n";
    out << "    }\n";
    const std::string aStep = p.rowKFast ? "k0" : "(long)k0 * " + str(M);
    const std::string bStep = p.colKFast ? "k0" : "(long)k0 * " + str(N);
    // One copy of a chunk's fragments in LDS and two barriers per chunk (before the fragments are overwritten and after).
    // Measured against that and not kept: two halves of LDS, the next chunk written to one while the other is
    // multiplied, one barrier per chunk (80^3 per entry 57 -> 62 %, 128 x 128 x 2^18 37 -> 41 TFLOP/s, but 128^3 per entry
    // 53 -> 50 %, 2 048^3 58 -> 53 TFLOP/s); two chunks on their way in two sets of registers (4 096^3 62 -> 53 TFLOP/s):
    // neither the barriers nor the latency of the loads is what these kernels wait for.
    out << "    double ra[" << UA << "], rb[" << UB << "];\n";
    auto emitLoads = [&](const std::string &ind, const std::string &k0) {
        // (no branches around the loads and no use of their values here, so that all of them are in flight together and
        // stay so while the chunk before is multiplied)
        out << ind << "{\n" << ind << "    const int k0 = " << k0 << ";\n";
        out << ind << "    const double *rk = Rm + " << aStep << ", *ck = Cm + " << bStep << ";\n";
        out << "#pragma unroll\n" << ind << "    for (int u = 0; u < " << UA << "; ++u) ra[u] = rk[aFrom[u]];\n";
        out << "#pragma unroll\n" << ind << "    for (int u = 0; u < " << UB << "; ++u) rb[u] = ck[bFrom[u]];\n";
        out << ind << "}\n";
    };
    auto emitProducts = [&](const std::string &ind) {
        // (Reading the next step's fragments from LDS before this step's products, the order held by scheduling barriers,
        // changed nothing: 4 096^3 61 -> 59 TFLOP/s, 128^3 per entry 53 -> 49 %.  The wavefronts of a SIMD hide each other's
        // LDS latency already.)
        out << "#pragma unroll\n" << ind << "for (int s = 0; s < " << KS << "; ++s)\n" << ind << "{\n";
        out << ind << "    const int at = s * 64 + g * 16 + ((c + 4 * s + g) & 15);\n";
        out << ind << "    const double a = fragA[wave * " << KS * 64 << " + at];\n";
        out << "#pragma unroll\n" << ind << "    for (int J = 0; J < " << TJ << "; ++J)\n";
        out << ind << "        acc[J] = __builtin_amdgcn_mfma_f64_16x16x4f64(a, fragB[J * " << KS * 64 << " + at], acc[J], 0, 0, 0);\n";
        out << ind << "}\n";
    };
    // The whole chunks of the range run in the loop.  What is left of a range that is no whole number of chunks is read as
    // the range's last 16 terms (the factors have at least that many), and the terms among them that the loop has added
    // already become zero on their way to LDS: both factors', so that a NaN or an infinity there stays out.
    const bool tail = K % KC != 0 || (splits > 1 && span % KC != 0);
    out << "    const int kWhole = kBegin + (kEnd - kBegin) / " << KC << " * " << KC << ";   // where the whole chunks end\n";
    emitLoads("    ", "kBegin < kWhole ? kBegin : kEnd - " + str(KC));
    out << "    acro_double4 acc[" << TJ << "];\n";
    out << "#pragma unroll\n    for (int J = 0; J < " << TJ << "; ++J) acc[J] = acro_double4{0.0, 0.0, 0.0, 0.0};\n";
    out << "    for (int kc = kBegin; kc < kWhole; kc += " << KC << ")\n    {\n";
    out << "#pragma unroll\n        for (int u = 0; u < " << UA << "; ++u) fragA[aTo[u]] = ra[u];\n";
    out << "#pragma unroll\n        for (int u = 0; u < " << UB << "; ++u) fragB[bTo[u]] = rb[u];\n";
    out << "        __syncthreads();\n";
    emitLoads("        ", "kc + " + str(KC) + " < kWhole ? kc + " + str(KC) + " : kEnd - " + str(KC));
    emitProducts("        ");
    out << "        __syncthreads();\n";
    out << "    }\n";
    if (tail)
    {
        out << "    if (kWhole < kEnd)\n    {\n";
        out << "        const int done = kWhole - (kEnd - " << KC << ");   // terms of the last 16 that the loop has added\n";
        out << "#pragma unroll\n        for (int u = 0; u < " << UA << "; ++u)\n        {\n";
        out << "            const int i = threadIdx.x + " << NT << " * u, v = i < " << rowTile << " ? i : 0;\n";
        out << "            fragA[aTo[u]] = " << (p.rowKFast ? "v % " + str(KC) : "v / " + str(16 * W)) << " >= done ? ra[u] : 0.0;\n        }\n";
        out << "#pragma unroll\n        for (int u = 0; u < " << UB << "; ++u)\n        {\n";
        out << "            const int i = threadIdx.x + " << NT << " * u, v = i < " << colTile << " ? i : 0;\n";
        out << "            fragB[bTo[u]] = " << (p.colKFast ? "v % " + str(KC) : "v / " + str(16 * TJ)) << " >= done ? rb[u] : 0.0;\n        }\n";
        out << "        __syncthreads();\n";
        emitProducts("        ");
        out << "    }\n";
    }
    out << "#pragma unroll\n    for (int J = 0; J < " << TJ << "; ++J)\n";
    out << "#pragma unroll\n        for (int q = 0; q < 4; ++q)\n        {\n";
    out << "            const int m = r0 + 16 * wave + 4 * q + g, n = c0 + 16 * J + c;\n";
    if (M % (16 * W) != 0 || N % (16 * TJ) != 0) out << "            if (m >= " << M << " || n >= " << N << ") continue;\n";
    if (splits > 1)
    {
        out << "            scratch[((long)split * " << E << " + e) * " << M * N << "L + (long)m * " << N << " + n] = acc[J][q];\n";
        out << "        }\n}\n";
        // ---- the partial sums of all shares, added in a fixed order: one lane per output, or 4 or 16 lanes where the
        // outputs alone are too few lanes to keep the loads of many shares in flight (64 x 64 outputs in 256 shares:
        // 27 -> 6 us); the lanes of an output add their sums through LDS, in a fixed order again
        const long O = E * M * N;
        long P = 1;
        while (P < 16 && O * P < 65536 && 4 * P * 2 <= splits) P *= 4;
        const long each = 256 / P;
        out << "\nextern \"C\" __global__ __launch_bounds__(256) void " << fFinal << "(double *" << (opt.noalias ? "__restrict__ " : "")
            << "result, const double *__restrict__ scratch)\n{\n";
        if (P == 1)
        {
            out << "    const long o = (long)blockIdx.x * 256 + threadIdx.x;\n";
            out << "    if (o >= " << O << "L) return;\n";
            out << "    double t = 0.0;\n";
            out << "#pragma unroll 8\n    for (int w = 0; w < " << splits << "; ++w) t += scratch[w * " << O << "L + o];\n";
        }
        else
        {
            out << "    __shared__ double red[256];\n";
            out << "    const long o = (long)blockIdx.x * " << each << " + threadIdx.x % " << each << ";\n";
            out << "    const int part = threadIdx.x / " << each << ";\n";
            out << "    double t = 0.0;\n";
            out << "    if (o < " << O << "L)\n    {\n";
            out << "#pragma unroll 8\n        for (int w = part; w < " << splits << "; w += " << P << ") t += scratch[w * " << O << "L + o];\n    }\n";
            out << "    red[threadIdx.x] = t;\n    __syncthreads();\n";
            out << "    if (part != 0 || o >= " << O << "L) return;\n";
            out << "    t = red[threadIdx.x];\n";
            out << "#pragma unroll\n    for (int q = 1; q < " << P << "; ++q) t += red[threadIdx.x + " << each << " * q];\n";
        }
        const std::string dst = "result[" + str(aOff) + "L + o]";
        if (s.op == '=')
            out << "    " << dst << " = t;\n";
        else
            out << "    " << dst << " = " << dst << (s.op == '+' ? " + t;\n" : " - t;\n");
        out << "}\n";
    }
    else
    {
        out << "            double *d = Am + (long)m * " << N << " + n;\n";
        if (s.op == '=')
            out << "            " << (streams ? "__builtin_nontemporal_store(acc[J][q], d);" : "*d = acc[J][q];") << "\n";
        else
            out << "            *d " << (s.op == '+' ? "+=" : "-=") << " acc[J][q];\n";
        out << "        }\n";
        out << "}\n";
    }

    plan.source = out.str();
    plan.nb = 1;
    plan.lds_bytes = static_cast<int>((UA + UB) * NT * 8);
    FillParams(plan, false);
    HipLaunch launch;
    launch.function_name = fMain;
    launch.grid = static_cast<unsigned>(groups * splits);
    launch.block = static_cast<unsigned>(NT);
    for (int si = 0; si < NumParamStores(); ++si) launch.params.push_back(si);
    if (splits > 1) launch.params.push_back(-1);
    plan.launches.push_back(launch);
    if (splits > 1)
    {
        plan.scratch_doubles = static_cast<size_t>(splits * E * M * N);
        HipLaunch fin;
        fin.function_name = fFinal;
        long P = 1;   // (lanes per output, as in the kernel above)
        while (P < 16 && E * M * N * P < 65536 && 4 * P * 2 <= splits) P *= 4;
        fin.grid = static_cast<unsigned>((E * M * N + 256 / P - 1) / (256 / P));
        fin.block = 256;
        fin.params.push_back(uvars[s.out.uvar].storage);
        fin.params.push_back(-1);
        plan.launches.push_back(fin);
    }
}

}  // namespace codegen
}  // namespace acro
