// Kernel code generator, the Gram schedule: many outputs contracted over a long leading range, "A_i_j = B_n_i C_n_j".
#include "hip_codegen_impl.hpp"

namespace acro
{
namespace codegen
{

// "A_I_J = B_N_I C_N_J [W_N]": both operands carry the whole contraction range N as their leading dimensions, in the
// same order, and a group of output indices each behind it; the result is the I x J (or J x I) matrix of sums over N
// (normal equations, mass matrices of a global basis, moments of the batch).  A tall-skinny matrix product: with more
// outputs than the reduction schedule takes, the generic schedule gives every output a lane that walks the whole
// range with a stride of a row (64 x 64 over 2^20 rows: 113 ms).  Here a wavefront takes four rows of N at a time,
// reads them with the lanes along the rows, and adds the 16 x 16 blocks of outputs with v_mfma_f64_16x16x4; the
// arithmetic of 64 x 64 outputs takes about as long on the FP64 matrix cores as its rows take to arrive from HBM.
auto Generator::GramPattern(GramShape &g) const -> bool
{
    if (subs.size() != 1 || NumGatherSlots() > 0 || envInt("ACRO_HIP_GRAM") < 0 || opt.no_matrix_cores) return false;
    const Sub &s = subs[0];
    if (s.out.repeated || s.matrixOp != 0 || s.contr.empty() || (s.in.size() != 2 && s.in.size() != 3)) return false;
    if (s.contrCount < kReductionMinContraction) return false;
    const size_t nc = s.contr.size();
    // the two matrices, and an optional weight per row of N
    for (const auto &r : s.in)
    {
        if (r.repeated || r.uvar == s.out.uvar || uvars[r.uvar].storage == uvars[s.out.uvar].storage) return false;
        if (r.idx.size() < nc) return false;
        for (size_t d = 0; d < nc; ++d)
        {
            if (!has(s.contr, r.idx[d]) || r.idx[d] != s.in[0].idx[d]) return false;
        }
        for (size_t d = nc; d < r.idx.size(); ++d)
        {
            if (has(s.contr, r.idx[d])) return false;
        }
        if (r.idx.size() == nc)
        {
            if (g.w) return false;
            g.w = &r;
        }
        else if (!g.b)
            g.b = &r;
        else if (!g.c)
            g.c = &r;
        else
            return false;
    }
    if (!g.b || !g.c) return false;
    const std::vector<int> I(g.b->idx.begin() + nc, g.b->idx.end()), J(g.c->idx.begin() + nc, g.c->idx.end());
    for (int id : I)
    {
        if (has(J, id)) return false;
    }
    std::vector<int> ij = I, ji = J;
    ij.insert(ij.end(), J.begin(), J.end());
    ji.insert(ji.end(), I.begin(), I.end());
    if (s.out.idx != ij && s.out.idx != ji) return false;
    g.swapped = s.out.idx != ij;
    g.rows = product(I, extent);
    g.cols = product(J, extent);
    g.range = s.contrCount;
    const long tiles = ((g.rows + 15) / 16) * ((g.cols + 15) / 16);
    // (up to 64 outputs a lane of the reduction schedule owns whole rows of the range and keeps them all, 8 x 8: 75 % of
    // the HBM peak; beyond that it would read every value once per output, 12 x 12: 12 %, here 73 %.  A wavefront holds
    // at most 16 blocks of 16 x 16 sums.)
    if (g.rows * g.cols <= 64 || tiles > 16) return false;
    return true;
}

auto Generator::UseGramSchedule() const -> bool
{
    GramShape g;
    return GramPattern(g);
}

auto Generator::EmitGram(HipKernelPlan &plan) -> void
{
    const Sub &s = subs[0];
    GramShape g;
    GramPattern(g);
    const long nI = g.rows, nJ = g.cols, N = g.range, O = nI * nJ;
    const long TI = (nI + 15) / 16, TJ = (nJ + 15) / 16;
    const long groups = (N + 3) / 4;                      // four rows of N per instruction
    // One workgroup of four wavefronts per CU, or two: each wavefront strides over the groups of rows.  Whole blocks of
    // outputs, four or more of them: one (the loop then has no selects for a second wavefront to hide, and with 16
    // blocks only one wavefront fits a SIMD anyway, so 512 workgroups ran as two rounds of 256); outputs that 16 does
    // not divide, and a single block: two.  512 MB of operands, tensors rotated, % of the HBM peak with 256 / 512 / 768
    // workgroups: 64 x 64 63 / 55 / 49, 64 x 48 68 / 60 / 56, 64 x 32 72 / 61 / 61, 32 x 32 71 / 64 / 61; 48 x 40 56 / 64 / 50,
    // 40 x 40 54 / 63 / 49, 24 x 24 60 / 65 / 59, 16 x 16 66 / 70 / 62, 12 x 12 63 / 65 / 59.
    const bool wholeBlocks = nI % 16 == 0 && nJ % 16 == 0 && TI * TJ >= 4;
    const long G = envInt("ACRO_HIP_GRAM_GROUPS") > 0 ? envInt("ACRO_HIP_GRAM_GROUPS") : std::max<long>(1, std::min<long>(wholeBlocks ? 256 : 512, groups / 16));

    const std::string dimName = mk.GetDimensionedNameString();
    char hex[32];
    std::snprintf(hex, sizeof(hex), "%016llx",
                  static_cast<unsigned long long>(hashString(dimName + "/gram/" + (opt.noalias ? "n" : "a") + (Positional() ? "p" : "u"))));
    plan.module_name = std::string("acro_gram_") + hex;
    const std::string fPartial = plan.module_name + "_partial", fFinal = plan.module_name + "_final";

    std::ostringstream sched;
    sched << "Gram schedule on the FP64 matrix cores: " << nI << " x " << nJ << " outputs" << (g.swapped ? " (stored transposed)" : "")
          << ", sums over " << N << " rows, four rows per v_mfma_f64_16x16x4, " << TI * TJ << " blocks per wavefront, " << G
          << " workgroups of 256 lanes, partials added in a fixed order by a second kernel\n  [0] " << s.text << "\n";
    plan.schedule = sched.str();
    out << "// Generated by the acrotensor HIP code generator for gfx950.\n";
    {
        std::istringstream lines(plan.schedule);
        std::string l;
        while (std::getline(lines, l)) out << "// " << l << "\n";
    }
    const std::string B = PtrName(g.b->uvar), C = PtrName(g.c->uvar);
    out << "typedef double acro_double4 __attribute__((ext_vector_type(4)));\n";
    out << "\nextern \"C\" __global__ __launch_bounds__(256) void " << fPartial << "(" << ParamList() << ", double *__restrict__ scratch)\n{\n";
    out << "    __shared__ double sums[" << O << "];\n";
    out << "    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r = lane & 15, k = lane >> 4;\n";
    out << "    acro_double4 acc[" << TI << "][" << TJ << "];\n";
    out << "#pragma unroll\n    for (int ti = 0; ti < " << TI << "; ++ti)\n";
    out << "#pragma unroll\n        for (int tj = 0; tj < " << TJ << "; ++tj) acc[ti][tj] = acro_double4{0.0, 0.0, 0.0, 0.0};\n";
    // A wavefront takes four or eight groups of four rows per step, all their loads first, and requests the next step's rows before
    // it multiplies this step's: with two wavefronts per SIMD the loads of one step would otherwise wait out their
    // whole latency between two bursts of arithmetic.
    // (64 x 64 outputs: 533 / 280 / 249 / 294 us with 1 / 2 / 4 / 8 groups per step; 32 x 32: 260 / - / 194 / 203 us)
    // (48 x 40 with a weight per row: 157 us with 2 groups, 181 us with 4)
    const long U = TI + TJ >= 8 ? 4 : std::max<long>(1, 16 / (TI + TJ));
    const long stride = G * 4;
    // Two forms of the loads of a step: `fetch` serves any rows (rows past the end of the range read as zero, their
    // addresses fall back to row 0), `fetchInside` only rows that all exist: no selects on the loaded values, which the
    // first form needs one or two of per value.  The main loop takes two steps per turn, the operands of the one in the
    // registers that the other has just used up (no copies), and runs while both steps' rows are inside the range; the
    // steps near the end go one at a time through `fetch`.  With one wavefront per SIMD (16 blocks of sums are 128
    // registers, the operands of two steps as many again) nothing else hides those instructions: 64 x 64 over 2^20 rows
    // 54 -> 70 % of the HBM peak with both changes and one workgroup per CU, 5.8 -> 2.4 other vector instructions per
    // matrix instruction.
    for (int inside = 0; inside < 2; ++inside)
    {
        out << "    auto " << (inside ? "fetchInside" : "fetch") << " = [&](long g0, double (&bq)[" << U << "][" << TI << "], double (&cq)[" << U << "][" << TJ << "]) {\n";
        out << "#pragma unroll\n        for (int u = 0; u < " << U << "; ++u)\n        {\n";
        out << "            const long n = (g0 + u * " << stride << ") * 4 + k;\n";
        const std::string row = inside ? "n" : "(inRange ? n : 0)";
        const std::string ok = inside ? "" : "inRange";
        if (!inside) out << "            const bool inRange = n < " << N << ";\n";
        out << "            const double *b = " << B << " + " << Lit(uvars[g.b->uvar].viewOffset) << " + " << row << " * " << nI << " + r;\n";
        out << "            const double *c = " << C << " + " << Lit(uvars[g.c->uvar].viewOffset) << " + " << row << " * " << nJ << " + r;\n";
        auto guarded = [&](long extentHere, const std::string &t, const std::string &load) {
            std::string cond = ok;
            if (extentHere % 16 != 0) cond += (cond.empty() ? "" : " && ") + std::string("16 * ") + t + " + r < " + str(extentHere);
            return cond.empty() ? load : "(" + cond + ") ? " + load + " : 0.0";
        };
        // (rows of whole 128-byte lines, each read by one group of 16 lanes once: with the non-temporal hint 32 x 32 outputs
        // over 2^21 rows 77 -> 85 % of the HBM peak, 64 x 64 71 -> 76 %, 16 x 48 73 -> 79 %)
        const bool ntB = envInt("ACRO_HIP_GRAM_NT") >= 0 && nI % 16 == 0 && g.b->uvar != g.c->uvar, ntC = envInt("ACRO_HIP_GRAM_NT") >= 0 && nJ % 16 == 0 && g.b->uvar != g.c->uvar;
        out << "#pragma unroll\n            for (int ti = 0; ti < " << TI << "; ++ti) bq[u][ti] = " << guarded(nI, "ti", ntB ? "__builtin_nontemporal_load(&b[16 * ti])" : "b[16 * ti]") << ";\n";
        out << "#pragma unroll\n            for (int tj = 0; tj < " << TJ << "; ++tj) cq[u][tj] = " << guarded(nJ, "tj", ntC ? "__builtin_nontemporal_load(&c[16 * tj])" : "c[16 * tj]") << ";\n";
        if (g.w)
        {
            out << "            const double w = " << PtrName(g.w->uvar) << "[" << Lit(uvars[g.w->uvar].viewOffset) << " + " << row << "];\n";
            // on the side with fewer blocks
            if (TI <= TJ)
                out << "#pragma unroll\n            for (int ti = 0; ti < " << TI << "; ++ti) bq[u][ti] *= w;\n";
            else
                out << "#pragma unroll\n            for (int tj = 0; tj < " << TJ << "; ++tj) cq[u][tj] *= w;\n";
        }
        out << "        }\n    };\n";
    }
    auto emitProducts = [&](const std::string &bName, const std::string &cName, const std::string &ind) {
        out << "#pragma unroll\n" << ind << "for (int u = 0; u < " << U << "; ++u)\n";
        out << "#pragma unroll\n" << ind << "    for (int ti = 0; ti < " << TI << "; ++ti)\n";
        out << "#pragma unroll\n" << ind << "        for (int tj = 0; tj < " << TJ << "; ++tj)\n";
        out << ind << "            acc[ti][tj] = __builtin_amdgcn_mfma_f64_16x16x4f64(" << bName << "[u][ti], " << cName << "[u][tj], acc[ti][tj], 0, 0, 0);\n";
    };
    const long step = U * stride, fullGroups = N / 4;   // groups of four rows that all exist
    out << "    double bv[" << U << "][" << TI << "], cv[" << U << "][" << TJ << "], bn[" << U << "][" << TI << "], cn[" << U << "][" << TJ << "];\n";
    out << "    long g0 = (long)blockIdx.x * 4 + wave;\n";
    out << "    fetch(g0, bv, cv);\n";
    // (the last group that the second fetch of a turn touches is g0 + 2 * step + (U - 1) * stride)
    out << "    for (; g0 + " << 2 * step + (U - 1) * stride << " < " << fullGroups << "; g0 += " << 2 * step << ")\n    {\n";
    out << "        fetchInside(g0 + " << step << ", bn, cn);\n";
    emitProducts("bv", "cv", "        ");
    out << "        fetchInside(g0 + " << 2 * step << ", bv, cv);\n";
    emitProducts("bn", "cn", "        ");
    out << "    }\n";
    out << "    for (; g0 < " << groups << "; g0 += " << step << ")\n    {\n";
    out << "        fetch(g0 + " << step << ", bn, cn);\n";
    emitProducts("bv", "cv", "        ");
    out << "#pragma unroll\n        for (int u = 0; u < " << U << "; ++u)\n        {\n";
    out << "#pragma unroll\n            for (int ti = 0; ti < " << TI << "; ++ti) bv[u][ti] = bn[u][ti];\n";
    out << "#pragma unroll\n            for (int tj = 0; tj < " << TJ << "; ++tj) cv[u][tj] = cn[u][tj];\n";
    out << "        }\n    }\n";
    // The four wavefronts add their blocks in LDS one after the other (a fixed order), in the result's memory order:
    // register q of a lane holds output row 4 q + lane / 16 and column lane % 16 of its block.
    out << "    for (int turn = 0; turn < 4; ++turn)\n    {\n";
    out << "        if (wave == turn)\n        {\n";
    out << "#pragma unroll\n            for (int ti = 0; ti < " << TI << "; ++ti)\n";
    out << "#pragma unroll\n                for (int tj = 0; tj < " << TJ << "; ++tj)\n";
    out << "#pragma unroll\n                    for (int q = 0; q < 4; ++q)\n                    {\n";
    out << "                        const int i = 16 * ti + 4 * q + k, j = 16 * tj + r;\n";
    if (nI % 16 != 0 || nJ % 16 != 0)
        out << "                        if (i >= " << nI << " || j >= " << nJ << ") continue;\n";
    const std::string at = g.swapped ? "j * " + str(nI) + " + i" : "i * " + str(nJ) + " + j";
    out << "                        if (turn == 0) sums[" << at << "] = acc[ti][tj][q];\n";
    out << "                        else sums[" << at << "] += acc[ti][tj][q];\n";
    out << "                    }\n        }\n        __syncthreads();\n    }\n";
    out << "    for (int o = threadIdx.x; o < " << O << "; o += 256) scratch[(long)blockIdx.x * " << O << " + o] = sums[o];\n";
    out << "}\n";

    // ---- the partials of all workgroups, added in a fixed order: 64 outputs per workgroup, four lanes each
    const long finishGroups = (O + 63) / 64;
    out << "\nextern \"C\" __global__ __launch_bounds__(256) void " << fFinal << "(double *" << (opt.noalias ? "__restrict__ " : "")
        << "result, const double *__restrict__ scratch)\n{\n";
    out << "    __shared__ double red[256];\n";
    out << "    const int o = blockIdx.x * 64 + (threadIdx.x & 63), part = threadIdx.x >> 6;\n";
    out << "    double t = 0.0;\n";
    out << "    if (o < " << O << ")\n    {\n";
    out << "#pragma unroll 8\n";
    out << "        for (long w = part; w < " << G << "; w += 4) t += scratch[w * " << O << " + o];\n    }\n";
    out << "    red[threadIdx.x] = t;\n    __syncthreads();\n";
    out << "    if (part == 0 && o < " << O << ")\n    {\n";
    out << "        t = ((red[threadIdx.x] + red[threadIdx.x + 64]) + red[threadIdx.x + 128]) + red[threadIdx.x + 192];\n";
    const std::string dst = "result[" + Lit(uvars[s.out.uvar].viewOffset) + " + o]";
    if (s.op == '=')
        out << "        " << dst << " = t;\n";
    else
        out << "        " << dst << " = " << dst << (s.op == '+' ? " + t;\n" : " - t;\n");
    out << "    }\n}\n";

    plan.source = out.str();
    plan.scratch_doubles = static_cast<size_t>(G * O);
    plan.nb = 1;
    plan.lds_bytes = static_cast<int>(O * 8);
    FillParams(plan, false);
    const int S = static_cast<int>(stores.size());
    HipLaunch partial;
    partial.function_name = fPartial;
    partial.grid = static_cast<unsigned>(G);
    partial.block = 256;
    for (int si = 0; si < S; ++si) partial.params.push_back(si);
    partial.params.push_back(-1);
    plan.launches.push_back(partial);
    HipLaunch fin;
    fin.function_name = fFinal;
    fin.grid = static_cast<unsigned>(finishGroups);
    fin.block = 256;
    fin.params.push_back(uvars[s.out.uvar].storage);
    fin.params.push_back(-1);
    plan.launches.push_back(fin);
}

}  // namespace codegen
}  // namespace acro
