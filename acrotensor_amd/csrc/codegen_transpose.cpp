// Kernel code generator, the transpose schedule (32 x 32 tiles through LDS).
#include "hip_codegen_impl.hpp"

namespace acro
{
namespace codegen
{

// ------------------------------------------------------------------------------ transpose schedule
// A single kernel that only permutes the dimensions of one operand, with different, long fastest dimensions on
// the two sides ("A_i_j = B_j_i" with 8 192 x 8 192 entries): whichever side the lanes follow, the other side
// moves 8 bytes per 128-byte line (17 % of the HBM peak for that kernel).  Instead a workgroup moves a tile of
// 32 x 32 entries through LDS: it reads rows of 32 consecutive entries along the operand's fastest dimension,
// and writes rows of 32 consecutive entries along the output's.  The tile's rows are 33 doubles apart in LDS, so
// that the transposed read is free of bank conflicts.
auto Generator::UseTransposeSchedule() const -> bool
{
    if (subs.size() != 1 || envInt("ACRO_HIP_TRANSPOSE") < 0 || !opt.noalias || NumGatherSlots() > 0) return false;
    const Sub &s = subs[0];
    if (s.matrixOp != 0 || s.in.size() != 1 || !s.contr.empty() || s.out.repeated || s.in[0].repeated) return false;
    if (s.in[0].uvar == s.out.uvar || s.in[0].idx.size() != s.out.idx.size() || s.out.idx.size() < 2) return false;
    const int a = s.in[0].idx.back(), b = s.out.idx.back();
    if (a == b) return false;
    if (extent[a] >= 32 && extent[b] >= 32)
    {
        // Small matrices per entry ("A_e_i_j = B_e_j_i", 40 x 40 to 100 x 100): a lane per element writes along the rows
        // of the result and reads down the columns of an operand that the caches hold for the whole entry, which beats
        // tiles of 32 x 32 that such extents fill badly (40 x 40: 37 -> 90 % of the HBM peak, 45 x 45 31 -> 89 %,
        // 64 x 64 78 -> 87 %, 64 x 100 59 -> 85 %, 100 x 100 44 -> 60 %; 32 x 32 stays, 80 against 70 %, and so does
        // 200 x 200, 64 against 37 %).
        const long na = extent[a], nb = extent[b];
        const double filled = static_cast<double>(na * nb) / static_cast<double>(((na + 31) / 32 * 32) * ((nb + 31) / 32 * 32));
        const size_t n = s.out.idx.size();
        bool perEntry = n > 2 && envInt("ACRO_HIP_TRANSPOSE") < 3 && s.out.idx[n - 2] == a && s.in[0].idx[n - 2] == b;
        for (size_t d = 0; perEntry && d + 2 < n; ++d) perEntry = s.out.idx[d] == s.in[0].idx[d];
        if (perEntry && na * nb > 1024 && (na * nb <= 4096 || (na * nb <= 10000 && filled < 0.8))) return false;
        return true;
    }
    // One side short (a matrix of 2^22 x 16): tiles of 16 x 64 (8 x 128) entries, see EmitTranspose.
    const int shorter = std::min(extent[a], extent[b]), longer = std::max(extent[a], extent[b]);
    return envInt("ACRO_HIP_TRANSPOSE") < 2 && shorter >= 8 && longer >= 256;
}

auto Generator::EmitTranspose(HipKernelPlan &plan) -> void
{
    const Sub &s = subs[0];
    const VarRef &in = s.in[0];
    const int a = in.idx.back(), b = s.out.idx.back();
    auto strideOf = [](const VarRef &r, int id) {
        for (size_t d = 0; d < r.idx.size(); ++d)
        {
            if (r.idx[d] == id) return r.stride[d];
        }
        return 0L;
    };
    std::vector<int> rest;
    for (int id : s.out.idx)
    {
        if (id != a && id != b) rest.push_back(id);
    }
    const long na = extent[a], nbb = extent[b], nrest = product(rest, extent);
    // entries per side of a tile: 32 x 32 (64 measured 55.4 against 58.7 % of the HBM peak for 8 192 x 8 192); where one
    // side has fewer than 32 entries the tile takes the next power of two of them and 1 024 entries in all, so that the
    // long side is read or written in runs of 512 or 1 024 bytes (2^22 x 16 -> 16 x 2^22: 34.6 % of the HBM peak one
    // entry per lane; see the schedule comment for what it runs as now)
    auto pow2ceil = [](long n) { int p = 1; while (p < n) p *= 2; return p; };
    const int TA = na >= 32 ? (nbb >= 32 ? 32 : 1024 / pow2ceil(nbb)) : pow2ceil(na);
    const int TB = nbb >= 32 ? 1024 / TA : pow2ceil(nbb);
    const long tilesA = (na + TA - 1) / TA, tilesB = (nbb + TB - 1) / TB;
    const long groups = tilesA * tilesB * nrest;
    ACROBATIC_ASSERT(groups < (1L << 31), "HIP generator: too many tiles for one launch of the transpose schedule.");
    for (const auto &st : stores)
    {
        long entries = 1;
        for (int d : st.dims) entries *= d;
        if (entries >= (1L << 31) - 1) wide = true;
    }

    const std::string dimName = mk.GetDimensionedNameString();
    char hex[32];
    std::snprintf(hex, sizeof(hex), "%016llx",
                  static_cast<unsigned long long>(hashString(dimName + "/transpose/" + (Positional() ? "p" : "u"))));
    plan.module_name = std::string("acro_tr_") + hex;
    std::ostringstream sched;
    sched << "transpose schedule: tiles of " << TA << " x " << TB << " entries over (" << idxName[a] << ", " << idxName[b] << ") through LDS, "
          << groups << " workgroups of 256 lanes\n  [0] " << s.text << "\n";
    plan.schedule = sched.str();

    out << "// Generated by the acrotensor HIP code generator for gfx950.\n";
    {
        std::istringstream lines(plan.schedule);
        std::string l;
        while (std::getline(lines, l)) out << "// " << l << "\n";
    }
    out << "\nextern \"C\" __global__ __launch_bounds__(256) void " << plan.module_name << "(" << ParamList() << ")\n{\n";
    out << "    __shared__ double tile[" << TB << " * " << TA + 1 << "];\n";
    out << "    long g = blockIdx.x;\n";
    // Tiles along a are taken in turn, and each starts at another tile along b: workgroups that run together then
    // write (and read) different column blocks.  With rows a power of two apart every tile of one column block
    // falls on the same memory channels (8 192 x 8 192: 57 % of the HBM peak in plain order, 65 % this way; the
    // diagonal along a instead, or shifted only every 8 tiles: 64 %, 60 %; tiles of 16 / 64 entries: 62 / 54 %).
    out << "    const int ta = (int)(g % " << tilesA << "); g /= " << tilesA << ";\n";
    out << "    const int tb = (int)((g % " << tilesB << " + ta) % " << tilesB << "); g /= " << tilesB << ";\n";
    std::string inBase = Lit(uvars[in.uvar].viewOffset), outBase = Lit(uvars[s.out.uvar].viewOffset);
    for (int j = static_cast<int>(rest.size()) - 1; j >= 0; --j)
    {
        const std::string name = IdxVar(rest[j]);
        out << "    const int " << name << " = (int)(g % " << extent[rest[j]] << "); g /= " << extent[rest[j]] << ";\n";
        inBase += " + " + name + " * " + Lit(strideOf(in, rest[j]));
        outBase += " + " + name + " * " + Lit(strideOf(s.out, rest[j]));
    }
    out << "    const " << OffsetType() << " inBase = " << inBase << ", outBase = " << outBase << ";\n";
    // the operand's rows run along a, the tile keeps them as rows (TA + 1 doubles apart)
    out << "    {\n        const int lx = threadIdx.x & " << TA - 1 << ", ly = threadIdx.x / " << TA << ";\n";
    out << "        for (int y = ly; y < " << TB << "; y += " << 256 / TA << ")\n        {\n";
    out << "            const int ia = ta * " << TA << " + lx, ib = tb * " << TB << " + y;\n";
    // every entry is read once and written once: neither side is worth keeping in the caches (non-temporal stores
    // 8 192 x 8 192 64.9 -> 68.8 % of the HBM peak, 2^22 x 16 69.5 -> 74.5 %; loads as well 69.8 %, 75.1 %)
    const bool streams = envInt("ACRO_HIP_NT_STORE") >= 0;
    const std::string src = PtrName(in.uvar) + "[inBase + ia * " + Lit(strideOf(in, a)) + " + ib * " + Lit(strideOf(in, b)) + "]";
    out << "            if (ia < " << na << " && ib < " << nbb << ") tile[y * " << TA + 1 << " + lx] = "
        << (streams ? "__builtin_nontemporal_load(&" + src + ")" : src) << ";\n        }\n    }\n";
    out << "    __syncthreads();\n";
    // the output's rows run along b: lane lx takes column lx of the tile's rows
    out << "    {\n        const int lx = threadIdx.x & " << TB - 1 << ", ly = threadIdx.x / " << TB << ";\n";
    out << "        for (int y = ly; y < " << TA << "; y += " << 256 / TB << ")\n        {\n";
    out << "            const int ia = ta * " << TA << " + y, ib = tb * " << TB << " + lx;\n";
    out << "            if (ia < " << na << " && ib < " << nbb << ")\n            {\n";
    const std::string dst = PtrName(s.out.uvar) + "[outBase + ia * " + Lit(strideOf(s.out, a)) + " + ib * " + Lit(strideOf(s.out, b)) + "]";
    if (s.op == '=' && streams)
        out << "                __builtin_nontemporal_store(tile[lx * " << TA + 1 << " + y], &" << dst << ");\n";
    else if (s.op == '=')
        out << "                " << dst << " = tile[lx * " << TA + 1 << " + y];\n";
    else
        out << "                " << dst << " = " << dst << (s.op == '+' ? " + " : " - ") << "tile[lx * " << TA + 1 << " + y];\n";
    out << "            }\n        }\n    }\n}\n";

    plan.source = out.str();
    plan.nb = 1;
    plan.lds_bytes = TB * (TA + 1) * 8;
    FillParams(plan, false);
    HipLaunch launch;
    launch.function_name = plan.module_name;
    launch.grid = static_cast<unsigned>(groups);
    launch.block = 256;
    for (int si = 0; si < NumParamStores(); ++si) launch.params.push_back(si);
    plan.launches.push_back(launch);
}

}  // namespace codegen
}  // namespace acro
