// Kernel code generator, the schedule: register tiles and lane order, kernels applied in the registers of their producers, phases, LDS tiles and their placement, batch and workgroup size.
#include "hip_codegen_impl.hpp"

namespace acro
{
namespace codegen
{

// Operand can be read with scalar loads: never written here, no aliasing, small, and its address does not
// depend on the lane (only on tile / contraction indices, which are literals or uniform loop counters).
auto Generator::IsUniform(const Sub &s, const VarRef &r, const std::vector<int> &tile) const -> bool
{
    if (!opt.noalias || !IsPureInput(r.uvar) || GatherSlot(r.uvar) >= 0) return false;
    bool carriesBatch = false;
    for (int id : r.idx)
    {
        if (id == batch)
        {
            if (!batchUniform) return false;
            carriesBatch = true;
            continue;
        }
        if (!has(tile, id) && !has(s.contr, id)) return false;
    }
    // What one workgroup reads must be small enough to live in the scalar cache.
    const long perEntry = carriesBatch ? r.size / extent[batch] : r.size;
    return perEntry <= 4096;
}

// Loads per work item as LoadsPerItem counts them, except for streaming inputs (never written by the group,
// addressed through the batch index) whose lanes are far apart in memory: their loads are counted as the 16-byte
// instructions they become, each weighing as many times more as it touches more than 16 lines (four times what
// a coalesced one touches), if that is more than the plain count.  Measured with one lane per 4 x 4 matrix product against one lane per row: 44.6 against 88.7 % of the HBM
// peak; "A_e_i = B_e_i_j C_e_j" with 8 x 8: 38.1 against 75.8 %.
auto Generator::AccessCostPerItem(const Sub &s, const std::vector<int> &tile) const -> double
{
    std::vector<int> lanes;
    for (int id : s.out.idx)
    {
        if (id != batch && !has(tile, id) && !has(lanes, id)) lanes.push_back(id);
    }
    double cost = 0.0;
    for (const auto &r : s.in)
    {
        if (IsUniform(s, r, tile)) continue;
        std::set<int> seen;
        long n = 1;
        for (int id : r.idx)
        {
            if ((has(tile, id) || has(s.contr, id)) && seen.insert(id).second) n *= extent[id];
        }
        const bool streams = IsPureInput(r.uvar) && has(r.idx, batch);
        if (!streams)
        {
            cost += static_cast<double>(n);
            continue;
        }
        // trailing dimensions that the work item walks through are contiguous: pairs become 16-byte loads
        long chunk = 1;
        for (size_t d = r.idx.size(); d-- > 0;)
        {
            const int id = r.idx[d];
            if (id == batch || has(lanes, id)) break;
            chunk *= r.ext[d];
        }
        const double instructions = static_cast<double>(n) / chunk * ((chunk + 1) / 2);
        cost += std::max(static_cast<double>(n), instructions * LinesPerInstruction(s, r, lanes) / 16.0);
    }
    return cost;
}

auto Generator::LoadsPerItem(const Sub &s, const std::vector<int> &tile) const -> long
{
    long loads = 0;
    for (const auto &r : s.in)
    {
        if (IsUniform(s, r, tile)) continue;
        std::set<int> seen;
        long n = 1;
        for (int id : r.idx)
        {
            if ((has(tile, id) || has(s.contr, id)) && seen.insert(id).second) n *= extent[id];
        }
        loads += n;
    }
    return loads;
}

// Doubles of streaming operands (inputs that carry the batch index) that one wavefront keeps coming back to: an
// operand whose fastest dimension is not a lane index is read by each lane in pieces, so the lines that one load
// instruction touches are touched again by the lane's next loads and have to stay in the CU's 32 KB vector cache
// in between.  ("A_e_i = B_e_i_j C_e_j" with one lane per entry: 64 lanes x 576 bytes.)
auto Generator::WaveFootprint(const Sub &s, const std::vector<int> &tile) const -> long
{
    std::vector<int> lanes;
    for (int id : s.outIdx)
    {
        if (id != batch && !has(tile, id)) lanes.push_back(id);
    }
    const long perEntry = std::max<long>(1, product(lanes, extent));
    const long entriesPerWave = batch < 0 ? 1 : std::max<long>(1, 64 / perEntry);
    long footprint = 0;
    for (const auto &r : s.in)
    {
        if (!IsPureInput(r.uvar) || !has(r.idx, batch) || IsUniform(s, r, tile) || has(lanes, r.idx.back())) continue;
        std::set<int> seen;
        long perItem = 1, laneSpan = 1;
        for (int id : r.idx)
        {
            if (id == batch || !seen.insert(id).second) continue;
            (has(lanes, id) ? laneSpan : perItem) *= extent[id];
        }
        footprint += std::min<long>(64, laneSpan * entriesPerWave) * perItem;
    }
    return footprint;
}

// Average number of 128-byte lines that one load (or store) instruction of the first wavefront touches for
// occurrence r, the 64 work items being numbered as the emitted code numbers them (batch entries slowest, the
// last lane index fastest).  Four lines is a fully coalesced access; an operand read in pieces of 8 bytes at a
// stride of 72 touches 36, and the memory pipeline works through them one by one.
auto Generator::LinesPerInstruction(const Sub &s, const VarRef &r, const std::vector<int> &lanes) const -> double
{
    std::vector<int> literal;  // tile and contraction indices of the occurrence
    for (int id : r.idx)
    {
        if (id != batch && !has(lanes, id) && !has(literal, id)) literal.push_back(id);
    }
    const long combos = product(literal, extent), perEntry = std::max<long>(1, product(lanes, extent));
    const long step = std::max<long>(1, combos / 32);  // a sample of the literal offsets is enough
    std::vector<int> value(nidx, 0);
    double total = 0.0;
    long counted = 0;
    for (long c = 0; c < combos; c += step, ++counted)
    {
        long rem = c;
        for (int j = static_cast<int>(literal.size()) - 1; j >= 0; --j)
        {
            value[literal[j]] = static_cast<int>(rem % extent[literal[j]]);
            rem /= extent[literal[j]];
        }
        std::set<long> lines;
        for (long w = 0; w < 64; ++w)
        {
            const long b = w / perEntry;
            if (b > 0 && (batch < 0 || b >= E)) break;
            long rest = w % perEntry;
            for (int j = static_cast<int>(lanes.size()) - 1; j >= 0; --j)
            {
                value[lanes[j]] = static_cast<int>(rest % extent[lanes[j]]);
                rest /= extent[lanes[j]];
            }
            if (batch >= 0) value[batch] = static_cast<int>(b);
            long a = 0;
            for (size_t d = 0; d < r.idx.size(); ++d) a += static_cast<long>(value[r.idx[d]]) * r.stride[d];
            lines.insert(a >> 4);
        }
        total += static_cast<double>(lines.size());
    }
    return counted > 0 ? total / static_cast<double>(counted) : 1.0;
}

// A kernel far above the machine balance (hundreds of multiply-adds per double that moves) is bound by instruction
// issue, not by memory, and a long contraction written out term by term keeps every operand of every term in a
// register of its own (3D stiffness assembly step: 270 loads + 25 results per work item, 256 registers, spills).
// Such a kernel runs its contraction as counted loops around a register tile: per term the operands that do not
// depend on the tile are loaded and multiplied once, and every tile entry takes one multiply-add, with its own
// operands from scalar registers where they do not depend on the lanes.  The tile is the candidate with the fewest
// instructions per output; among equals the one made of the output's slowest dimensions, so that the lanes keep
// the fastest ones and stores stay contiguous.  (Stiffness step S = B1 B2 F1 with 225 terms and 15 625 outputs per
// element: 3 832 us with one output per lane, 1 644 us unrolled with the tile (i1, j1), see the schedule comment
// of the generated kernel for what it runs as now.)
auto Generator::ChooseLoopTile(Sub &s, const std::vector<int> &mid) const -> bool
{
    if (envInt("ACRO_HIP_LOOP_TILE") < 0 || batch < 0 || !opt.noalias) return false;
    if (s.matrixOp != 0 || s.out.repeated || s.flatItems || s.contrCount < 32 || mid.empty()) return false;
    const long nin = static_cast<long>(s.in.size());
    double moved = static_cast<double>(s.out.size) / static_cast<double>(E);
    for (const auto &r : s.in)
    {
        if (r.repeated || r.uvar == s.out.uvar) return false;
        if (has(r.idx, batch)) moved += static_cast<double>(r.size) / static_cast<double>(E);
    }
    const double outputs = static_cast<double>(product(mid, extent));
    const double macs = outputs * static_cast<double>(s.contrCount) * static_cast<double>(std::max<long>(1, nin - 1));
    if (macs < 64.0 * moved) return false;
    // Where every operand carries few of the contraction indices ("M = B_q_i B_q_l B_r_j B_r_m B_s_k B_s_n W_q_r_s"),
    // the unrolled body shares partial sums between the terms of one lane, which a loop cannot: that form stays.
    long carried = 0;
    for (const auto &r : s.in)
    {
        for (int c : s.contr) carried += has(r.idx, c) ? 1 : 0;
    }
    if (10 * carried < 7 * nin * static_cast<long>(s.contr.size())) return false;

    auto perOutput = [&](const std::vector<int> &t) {
        const long tc = product(t, extent);
        long common = 0, commonLoads = 0, perEntry = 1;
        for (const auto &r : s.in)
        {
            bool onTile = false;
            for (int id : r.idx) onTile = onTile || has(t, id);
            const bool uniform = IsUniform(s, r, t);
            if (!onTile)
            {
                ++common;
                if (!uniform) ++commonLoads;
            }
            else
            {
                perEntry += uniform ? 0 : 1;  // its load
                ++perEntry;                    // its multiplication
            }
        }
        if (common == 0) --perEntry;  // nothing to multiply the first tile operand with
        const double perTerm = static_cast<double>(commonLoads + std::max<long>(0, common - 1)) + static_cast<double>(tc * perEntry);
        return perTerm / static_cast<double>(tc);
    };
    const double flat = perOutput({});
    std::vector<std::vector<int>> candidates;
    for (size_t a = 0; a < mid.size(); ++a)
    {
        candidates.push_back({mid[a]});
        for (size_t b = a + 1; b < mid.size(); ++b) candidates.push_back({mid[a], mid[b]});
    }
    double best = 0.5 * flat;  // worth it from half the instructions on
    long bestPosition = 0;
    std::vector<int> tile;
    for (const auto &t : candidates)
    {
        const long tc = product(t, extent);
        if (tc < 2 || tc > kMaxTile || product(mid, extent) / tc < 64) continue;
        long position = 0;
        for (int id : t)
        {
            for (size_t d = 0; d < s.out.idx.size(); ++d)
            {
                if (s.out.idx[d] == id) position += static_cast<long>(d);
            }
        }
        const double cost = perOutput(t);
        if (cost < best - 1e-9 || (std::fabs(cost - best) <= 1e-9 && !tile.empty() && position < bestPosition))
        {
            best = cost;
            bestPosition = position;
            tile = t;
        }
    }
    if (tile.empty()) return false;
    s.tile = tile;
    s.loopMode = true;
    return true;
}

auto Generator::ChooseTiles() -> void
{
    for (auto &s : subs)
    {
        s.splitLanes = 0;
        std::vector<int> mid;
        for (int id : s.outIdx)
        {
            if (id != batch) mid.push_back(id);
        }
        const long nin = static_cast<long>(s.in.size());
        if (s.matrixOp != 0)
        {
            // One work item per matrix: the inverse keeps its row and column index as the register tile, the
            // determinant contracts them.
            s.loopMode = false;
            s.tile.clear();
            if (s.matrixOp == 1) s.tile.assign(s.out.idx.end() - 2, s.out.idx.end());
        }
        else if (ChooseLoopTile(s, mid))
        {
            // counted loops around a register tile
        }
        else if (s.contrCount > kMaxUnrolledContraction || s.contrCount * nin > kUnrollBudget)
        {
            s.loopMode = true;
            s.tile.clear();
        }
        else
        {
            std::vector<std::vector<int>> candidates(1);  // the empty tile
            for (size_t a = 0; a < mid.size(); ++a)
            {
                candidates.push_back({mid[a]});
                for (size_t b = a + 1; b < mid.size(); ++b) candidates.push_back({mid[a], mid[b]});
            }
            double bestScore = 1e300;
            std::vector<int> best;
            for (const auto &t : candidates)
            {
                const long tc = product(t, extent);
                if (tc > kMaxTile || tc * s.contrCount * nin > kUnrollBudget) continue;
                // (the copies of staged operands are made by many lanes per entry: the kernel that reads them keeps at
                // least four, or its workgroups would be mostly idle there)
                bool readsStagedCopy = false;
                for (const auto &r : s.in) readsStagedCopy = readsStagedCopy || uvars[r.uvar].isStagedCopy;
                if (readsStagedCopy && !t.empty() && product(mid, extent) / tc < 4) continue;
                const long loads = LoadsPerItem(s, t);
                // (operands staged in LDS tiles are cheap to read again: the compiler need not keep them all, and a
                // row of outputs per lane halves the reads: 16 x 16 matrix products 77 -> 84 % of the HBM peak)
                bool allStaged = tc <= 16;
                for (const auto &r : s.in) allStaged = allStaged && (uvars[r.uvar].isStagedCopy || IsUniform(s, r, t));
                if (loads + tc > (allStaged ? 2 * kMaxLiveValues : kMaxLiveValues) && !t.empty()) continue;
                // loads per produced output; a small bias keeps the tile short when nothing is gained
                const double cost = envInt("ACRO_HIP_FOOTPRINT") >= 0 ? AccessCostPerItem(s, t) : static_cast<double>(loads);
                double score = cost / tc + 1e-3 * t.size() + 1e-6 * tc;
                // ... unless the wavefront's working set of partly used lines outgrows its share of the vector cache
                const long footprint = WaveFootprint(s, t);
                if (footprint > 512 && envInt("ACRO_HIP_FOOTPRINT") >= 0) score *= static_cast<double>(footprint) / 512.0;
                if (score < bestScore)
                {
                    bestScore = score;
                    best = t;
                }
            }
            // A kernel on its own whose batch entries are tiny (at most 32 outputs, every operand streaming):
            // one output per lane.  The lanes of a wavefront then share the few lines of a handful of entries and
            // every access is coalesced, which outweighs the extra loads (batched 4 x 4 matrix products: 88.7 %
            // of the HBM peak against 55.5 % with a row per lane and 44.6 % with a product per lane; 3 x 3:
            // 64.6 / 58.5 / 53.8 %).
            bool streamingOnly = subs.size() == 1 && batch >= 0 && envInt("ACRO_HIP_FOOTPRINT") >= 0;
            // (small operands without the batch index do not count: they stay in the caches)
            const bool smallInvariantToo = envInt("ACRO_HIP_ONE_OUTPUT") > 0;
            for (const auto &r : s.in)
                streamingOnly = streamingOnly && (has(r.idx, batch) || (smallInvariantToo && r.size <= 1024)) && !r.repeated;
            const long outputs = product(mid, extent), loadsPerOutput = s.contrCount * nin;
            // (without a contraction, products of the entries' own values "A_e_i_j_k_l = B_e_i_j C_e_k_l", up to 256
            // outputs: 62 -> 84 % of the HBM peak, 16 x 16 outer product 81 -> 87 %; with 512 outputs and more a
            // register tile wins, 73 against 55 %)
            const long flatUpTo = s.contr.empty() ? 256 : 64;
            if (streamingOnly && ((outputs <= 32 && loadsPerOutput <= 16) || (outputs <= flatUpTo && loadsPerOutput <= 4))) best.clear();
            // The same for a tiny product whose operands were copied to LDS tiles first: one output per lane keeps the
            // stores of a wavefront contiguous.
            bool fromStagedCopies = (outputs < 64 || (outputs < 200 && s.wantedTile.empty())) && !s.in.empty();
            for (const auto &r : s.in)
            {
                fromStagedCopies = fromStagedCopies && (uvars[r.uvar].isStagedCopy || !has(r.idx, batch));
                // (matrices: every copy carries an output index; copies that all outputs of an entry share leave the
                // tile to the cost model, "Y_e_i_j = B_q_i B_r_j D_e_q_r U_e_q_r": 60 % with one output per lane,
                // 77 % with a row)
                bool carriesOutput = false;
                for (int id : r.idx) carriesOutput = carriesOutput || has(mid, id);
                if (uvars[r.uvar].isStagedCopy && !carriesOutput) fromStagedCopies = false;
            }
            bool anyStagedCopy = false;
            for (const auto &r : s.in) anyStagedCopy = anyStagedCopy || uvars[r.uvar].isStagedCopy;
            if (fromStagedCopies && anyStagedCopy) best.clear();
            // Entries as the fastest dimension of every tensor: whatever the tile, a wavefront reads 64 consecutive
            // entries per load, so the tile with the fewest loads per output wins (3 x 3 products of such layouts: a
            // lane per entry with all nine outputs, 18 loads, instead of nine lanes with six loads each).
            if (EntriesAreFastest())
            {
                double fewest = 1e300;
                for (const auto &t : candidates)
                {
                    const long tc = product(t, extent);
                    if (tc > kMaxTile || tc * s.contrCount * nin > kUnrollBudget) continue;
                    const long loads = LoadsPerItem(s, t);
                    if (loads + tc > kMaxLiveValues && !t.empty()) continue;
                    const double perOutput = static_cast<double>(loads) / tc;
                    if (perOutput < fewest * (1.0 - 1e-9))
                    {
                        fewest = perOutput;
                        best = t;
                    }
                }
            }
            if (!s.wantedTile.empty() && product(s.wantedTile, extent) * s.contrCount * nin <= kUnrollBudget) best = s.wantedTile;
            ForcedTile(static_cast<int>(&s - subs.data()), mid, best);
            if (s.flatItems) best.clear();
            s.tile = best;
        }
        SetLanes(s);
        // One output per batch entry ("A_e = B_e_i C_e_i", "A_e = B_e_n"): with one lane per entry every lane walks
        // along its own rows, 8 bytes per line and load instruction (55 and 52 % of the HBM peak).  Instead a power
        // of two of adjacent lanes shares the entry: lane c of them takes the terms c, c + lanes, ... of the
        // flattened contraction, so that the lanes of a wavefront read consecutive addresses, and the partial sums
        // are added in a butterfly of lane exchanges (a fixed order: results are reproducible).  The same for a
        // kernel with few outputs per entry and a contraction along the fastest dimension of a streaming operand
        // ("A_e_i = B_e_i_n", "Y_e_i = M_e_i_j X_e_j" with an element matrix of 27 x 27).  Up to 64 rows, or any number
        // of rows of 32 terms and more (65 x 65 62 -> 83 % of the HBM peak, 100 x 100 59 -> 85 %, 200 x 64 72 -> 84 %;
        // 256 x 16 90 -> 88 %, hence not for short rows).
        if (subs.size() == 1 && batch >= 0 && s.matrixOp == 0 && !s.out.repeated && envInt("ACRO_HIP_SPLIT_LANES") >= 0 &&
            !s.contr.empty() && (mid.empty() ? s.contrCount >= 8 : (s.contrCount >= 16 && product(mid, extent) <= (s.contrCount >= 32 ? envInt("ACRO_HIP_SPLIT_LANES_ROWS", 1024) : 64))))
        {
            // the operand that an entry reads most of carries the batch index and the fastest contraction index last
            const VarRef *most = &s.in[0];
            auto perEntry = [&](const VarRef &r) { return has(r.idx, batch) ? r.size / E : r.size; };
            for (const auto &r : s.in)
            {
                // (of two operands of one size, the one that carries the batch index: "A_e = B_i_j C_e_j_i")
                if (perEntry(r) > perEntry(*most) || (perEntry(r) == perEntry(*most) && has(r.idx, batch) && !has(most->idx, batch))) most = &r;
            }
            // (its fastest dimensions may be the contraction indices in another order than the kernel names them, "A_e =
            // B_i_j C_e_j_i": the terms are then numbered as they lie in that operand, 13 -> ... % of the HBM peak)
            std::vector<int> asStored = s.contr;
            if (s.contr.size() > 1 && most->idx.size() >= s.contr.size() && !most->repeated && envInt("ACRO_HIP_SPLIT_ORDER") >= 0)
            {
                const std::vector<int> tail(most->idx.end() - static_cast<long>(s.contr.size()), most->idx.end());
                bool same = true;
                for (int id : s.contr) same = same && has(tail, id);
                if (same) asStored = tail;
            }
            bool streams = has(most->idx, batch) && most->idx.back() == asStored.back();
            // ... and a row of its own for every output: where the outputs of an entry all read the same few values
            // ("Y_e_i_j = B_q_i B_r_j D_e_q_r U_e_q_r") the lanes of an entry would only repeat each other's loads
            // (8.7 % of the HBM peak against 55 % with a row of outputs per lane)
            for (int id : mid) streams = streams && has(most->idx, id);
            if (streams)
            {
                // At most a row of 16 lanes: the exchanges inside a row are register moves, not LDS traffic.  With
                // several outputs per entry a lane should have at least four terms of its own, or the exchanges
                // outweigh the arithmetic (16 x 16 matrix-vector products with one term per lane: 47 % against
                // 59 % unsplit).
                // (one output per entry: one term per lane, or one pair of terms where the lanes can load pairs)
                bool pairable = envInt("ACRO_HIP_SPLIT_PAIRS") >= 0 && s.contr.size() == 1 && s.contrCount % 2 == 0;
                for (const auto &r : s.in)
                {
                    if (has(r.idx, s.contr[0]) && (r.repeated || r.idx.back() != s.contr[0] || r.stride.back() != 1)) pairable = false;
                }
                const long atMost = mid.empty() ? (pairable ? s.contrCount / 2 : s.contrCount) : s.contrCount / 4;
                int lanes = 1;
                while (lanes * 2 <= 16 && lanes * 2 <= atMost) lanes *= 2;
                if (lanes >= (mid.empty() ? 2 : 4))
                {
                    s.tile.clear();
                    s.contr = asStored;
                    SetLanes(s);
                    s.splitLanes = lanes;
                    s.loopMode = true;
                    s.laneCount *= lanes;
                }
            }
        }
    }
}

// Experiment switch ACRO_HIP_FORCE_TILE="8:;3:q,r": kernel 8 of the group gets the empty register tile, kernel 3
// the tile (q, r), whatever the cost model says.  Names that are not output indices of the kernel are ignored.
auto Generator::ForcedTile(int k, const std::vector<int> &mid, std::vector<int> &tile) const -> void
{
    const char *spec = std::getenv("ACRO_HIP_FORCE_TILE");
    if (spec == nullptr) return;
    std::istringstream all(spec);
    std::string item;
    while (std::getline(all, item, ';'))
    {
        const size_t colon = item.find(':');
        if (colon == std::string::npos || std::atoi(item.substr(0, colon).c_str()) != k) continue;
        if (!std::isdigit(static_cast<unsigned char>(item[0]))) continue;
        tile.clear();
        std::istringstream names(item.substr(colon + 1));
        std::string name;
        while (std::getline(names, name, ','))
        {
            for (int id : mid)
            {
                if (idxName[id] == name && !has(tile, id)) tile.push_back(id);
            }
        }
    }
}

auto Generator::SetLanes(Sub &s) -> void
{
    s.lane.clear();
    // Lane order follows the dimension order of the tensor that should see unit-stride lanes: the output
    // when it is stored to device memory, otherwise the largest operand read from device memory.
    const VarRef *order = &s.out;
    const UVarInfo &uo = uvars[s.out.uvar];
    // read again by a later kernel of the group, under this name or as a view of the same storage
    bool readLater = uo.lastUse > uo.firstWrite;
    for (size_t k2 = static_cast<size_t>(&s - subs.data()) + 1; k2 < subs.size() && !readLater; ++k2)
    {
        for (const auto &r : subs[k2].in) readLater = readLater || ViewsOverlap(r.uvar, s.out.uvar);
    }
    const bool out_stays_on_chip = stores[uo.storage].transient && readLater;
    if (out_stays_on_chip)
    {
        const VarRef *big = nullptr;
        for (const auto &r : s.in)
        {
            if (!IsPureInput(r.uvar) || !has(r.idx, batch)) continue;
            if (big == nullptr || r.size > big->size) big = &r;
        }
        if (big != nullptr) order = big;
    }
    auto consider = [&](int id) {
        if (id == batch || has(s.tile, id) || has(s.lane, id) || !has(s.outIdx, id)) return;
        s.lane.push_back(id);
    };
    for (int id : order->idx) consider(id);
    // Output indices that the ordering tensor does not carry go in front (slowest).
    std::vector<int> front;
    for (int id : s.outIdx)
    {
        if (id != batch && !has(s.tile, id) && !has(s.lane, id)) front.push_back(id);
    }
    s.lane.insert(s.lane.begin(), front.begin(), front.end());
    s.laneCount = product(s.lane, extent);
    s.tileCount = product(s.tile, extent);
}

// May operand r of a kernel with lane indices `lane` be taken from the registers in which kernel q left its
// output?  The work item must be the same (same index wherever q's output carries the batch or a lane index) and
// the entry must be named at generation time (a tile or contraction index of the reader elsewhere).
auto Generator::ForwardableFrom(const Sub &q, const VarRef &r, const std::vector<int> &lane) const -> bool
{
    if (r.uvar != q.out.uvar || r.idx.size() != q.out.idx.size()) return false;
    for (size_t d = 0; d < r.idx.size(); ++d)
    {
        const int pid = q.out.idx[d];
        const bool itemDim = pid == batch || has(lane, pid);
        if (itemDim ? r.idx[d] != pid : (r.idx[d] == batch || has(lane, r.idx[d]))) return false;
    }
    return true;
}

// Kernel k is about to join the chain that starts at chainStart, with lane indices `lane`: the kernels of a chain
// run one after the other in the same work item without a barrier, so every operand of k that a kernel of the
// chain writes must be the work item's own entry, taken from registers.  Marks those operands in `fwd`; false
// when some operand would need another work item's result.
auto Generator::ChainOperandsFromRegisters(int k, int chainStart, const std::vector<int> &lane, std::vector<char> &fwd) const -> bool
{
    const Sub &s = subs[k];
    fwd.assign(s.in.size(), 0);
    for (size_t v = 0; v < s.in.size(); ++v)
    {
        const VarRef &r = s.in[v];
        for (int q = k - 1; q >= chainStart; --q)
        {
            if (!ViewsOverlap(subs[q].out.uvar, r.uvar)) continue;
            if (!ForwardableFrom(subs[q], r, lane)) return false;
            fwd[v] = 1;
            break;
        }
    }
    return true;
}

// A kernel whose work items can be those of the previous kernel and that reads results of that kernel (or of
// the kernels it is itself applied after) entry by entry is applied in the same registers: a pointwise kernel
// after a contraction ("U = D T3"), but also a small contraction over the register tile of its producer
// ("D_e_m_n_k = W_k Jdet_e_k Jinv_e_k_n_j Jinv_e_k_m_j" after the inverse and determinant of J_e_k_m_n: one
// work item per (e, k) holds the nine entries of Jinv).
auto Generator::ForwardAlongChain(int k, int chainStart) -> void
{
    Sub &s = subs[k];
    const Sub &p = subs[k - 1];
    if (envInt("ACRO_HIP_FORWARD") < 0 || p.loopMode || s.loopMode || p.out.repeated || s.out.repeated) return;
    if (s.matrixOp == 2 && p.matrixOp == 1 && s.in[0].uvar == p.in[0].uvar && s.in[0].idx == p.in[0].idx)
    {
        // the determinant of the matrix that the previous kernel inverted: that kernel has computed it
        s.fusedWithPrev = true;
        s.forwardedIn.assign(1, 0);
        s.lane = p.lane;
        s.laneCount = p.laneCount;
        return;
    }
    for (int id : p.lane)
    {
        if (!has(s.outIdx, id)) return;
    }
    std::vector<int> tile;
    for (int id : s.out.idx)
    {
        if (id != batch && !has(p.lane, id) && !has(tile, id)) tile.push_back(id);
    }
    if (s.matrixOp == 1 && tile != std::vector<int>(s.out.idx.end() - 2, s.out.idx.end())) return;
    if (s.matrixOp == 2 && !tile.empty()) return;
    const long tc = product(tile, extent);
    if (tc > kMaxTile || tc * s.contrCount * static_cast<long>(s.in.size()) > kUnrollBudget) return;
    std::vector<char> fwd;
    if (!ChainOperandsFromRegisters(k, chainStart, p.lane, fwd)) return;
    if (std::find(fwd.begin(), fwd.end(), 1) == fwd.end()) return;
    for (int q = chainStart; q < k; ++q)
    {
        if (ViewsOverlap(subs[q].out.uvar, s.out.uvar)) return;
        for (const auto &r : subs[q].in)
        {
            if (ViewsOverlap(r.uvar, s.out.uvar)) return;  // other work items may still read what this one would overwrite
        }
    }
    s.fusedWithPrev = true;
    s.forwardedIn = fwd;
    s.lane = p.lane;
    s.laneCount = p.laneCount;
    s.tile = tile;
    s.tileCount = tc;
}

auto Generator::ChainStartOf(int k) const -> int
{
    while (k > 0 && subs[k].fusedWithPrev) --k;
    return k;
}

auto Generator::PlanFusion() -> void
{
    const int K = static_cast<int>(subs.size());
    for (int k = 1; k < K; ++k)
    {
        Sub &s = subs[k];
        const Sub &p = subs[k - 1];
        const int chainStart = ChainStartOf(k - 1);
        // A pointwise kernel over the previous kernel's outputs takes over its lanes and register tile as they are.
        bool pointwise = s.matrixOp == 0 && p.matrixOp == 0 && s.contr.empty() && !p.loopMode && !p.out.repeated && !s.out.repeated;
        if (pointwise)
        {
            std::set<int> a(s.outIdx.begin(), s.outIdx.end()), b(p.outIdx.begin(), p.outIdx.end());
            bool reads = false;
            for (const auto &r : s.in) reads = reads || (r.uvar == p.out.uvar && r.idx == p.out.idx);
            pointwise = a == b && reads && s.out.uvar != p.out.uvar;
        }
        std::vector<char> fwd;
        if (pointwise && ChainOperandsFromRegisters(k, chainStart, p.lane, fwd))
        {
            bool overwrites = false;  // an earlier kernel of the chain reads or writes what this one writes
            for (int q = chainStart; q < k; ++q)
            {
                overwrites = overwrites || ViewsOverlap(subs[q].out.uvar, s.out.uvar);
                for (const auto &r : subs[q].in) overwrites = overwrites || ViewsOverlap(r.uvar, s.out.uvar);
            }
            if (!overwrites)
            {
                s.fusedWithPrev = true;
                s.forwardedIn = fwd;
                s.tile = p.tile;
                s.lane = p.lane;
                s.laneCount = p.laneCount;
                s.tileCount = p.tileCount;
                s.loopMode = false;
                continue;
            }
        }
        ForwardAlongChain(k, chainStart);
    }
    // Accumulation chains ("Y = ...", "Y += ...", "Y += ..."): a kernel that adds into exactly what the previous
    // kernel produced, with the same pencil decomposition, takes the old value from that kernel's registers.
    for (int k = 1; k < K; ++k)
    {
        Sub &s = subs[k];
        const Sub &p = subs[k - 1];
        if (s.fusedWithPrev || s.op == '=' || s.loopMode || p.loopMode || s.out.repeated) continue;
        if (s.out.uvar != p.out.uvar || s.out.idx != p.out.idx || s.tile != p.tile || s.lane != p.lane) continue;
        std::vector<char> fwd;
        if (!ChainOperandsFromRegisters(k, ChainStartOf(k - 1), p.lane, fwd)) continue;
        s.fusedWithPrev = true;
        s.forwardedIn = fwd;
        s.forwardedOld = true;
    }
    AssignPhases();
}

// Two operands address overlapping memory: same storage and neither view's fixed leading indices exclude the
// other's.
auto Generator::ViewsOverlap(int ua, int ub) const -> bool
{
    const UVarInfo &a = uvars[ua], &b = uvars[ub];
    if (a.storage != b.storage) return false;
    if (!a.plainView || !b.plainView) return true;
    const size_t n = std::min(a.fixed.size(), b.fixed.size());
    for (size_t d = 0; d < n; ++d)
    {
        if (a.fixed[d] != b.fixed[d]) return false;
    }
    return true;
}

auto Generator::KernelsIndependent(int ka, int kb) const -> bool
{
    const Sub &a = subs[ka], &b = subs[kb];
    if (ViewsOverlap(a.out.uvar, b.out.uvar)) return false;
    for (const auto &r : b.in)
    {
        if (ViewsOverlap(a.out.uvar, r.uvar)) return false;
    }
    for (const auto &r : a.in)
    {
        if (ViewsOverlap(b.out.uvar, r.uvar)) return false;
    }
    return true;
}

// Chains (a kernel with the kernels applied in its registers) that do not depend on each other share a phase:
// their work items are laid side by side across the workgroup's wavefronts, which shortens the sequence of
// barrier-separated steps one workgroup walks through.
auto Generator::AssignPhases() -> void
{
    const int K = static_cast<int>(subs.size());
    int phase = 0;
    int phaseStart = 0;  // first kernel of the current phase
    for (int k = 0; k < K; ++k)
    {
        if (k > 0 && !subs[k].fusedWithPrev)
        {
            // k opens a new chain: may the whole chain join the current phase?
            int last = k;
            while (last + 1 < K && subs[last + 1].fusedWithPrev) ++last;
            bool join = envInt("ACRO_HIP_MERGE") >= 0 && !subs[k].loopMode;
            for (int a = phaseStart; a < k && join; ++a)
            {
                if (subs[a].loopMode) join = false;
                for (int b = k; b <= last && join; ++b) join = KernelsIndependent(a, b);
            }
            if (!join)
            {
                ++phase;
                phaseStart = k;
            }
        }
        subs[k].phase = phase;
    }
}

auto Generator::FromRegisters(int k, int v) const -> bool
{
    return subs[k].fusedWithPrev && static_cast<size_t>(v) < subs[k].forwardedIn.size() && subs[k].forwardedIn[v] != 0;
}

auto Generator::ComputeLdsWishes() -> void
{
    const int K = static_cast<int>(subs.size());
    for (auto &st : stores)
    {
        st.wantLds = false;
        st.inLds = false;
        st.liveTo = -1;
        st.staged = false;
        st.copyOutOnly = false;
    }
    if (batch < 0) return;
    ChooseStagedInputs();
    ChooseCopyOutTile();
    for (size_t si = 0; si < stores.size(); ++si)
    {
        Storage &st = stores[si];
        if (!st.written || !st.elementLocal || st.anyRepeated) continue;
        // Last kernel that could take entries of this storage from an LDS tile.
        for (int k = st.firstWrite + 1; k < K; ++k)
        {
            const Sub &s = subs[k];
            for (size_t v = 0; v < s.in.size(); ++v)
            {
                if (uvars[s.in[v].uvar].storage != static_cast<int>(si)) continue;
                if (FromRegisters(k, static_cast<int>(v)) || !readCovered[k][v]) continue;
                st.liveTo = k;
            }
            if (uvars[s.out.uvar].storage == static_cast<int>(si) && s.op != '=' && !s.forwardedOld && oldCovered[k])
                st.liveTo = k;
        }
        if (st.liveTo < 0 || st.copyOutOnly) continue;
        st.wantLds = true;
        // Kernels fused into one item loop run without a barrier between them, so LDS lifetimes are counted in
        // phases: a tile read in a phase and a tile written in the same phase must not share storage.
        st.phaseFrom = PhaseOf(st.firstWrite);
        st.phaseTo = PhaseOf(st.liveTo);
    }
}

// A kernel on its own whose work items each write a long run of consecutive outputs ("A_e_i = B_i_j X_e_j" with a
// 27 x 3 operator: one lane per entry, 27 results of 216 bytes each) stores pieces of 16 bytes 216 bytes apart:
// every store instruction of a wavefront touches 64 lines (36 % of the HBM peak).  Its results go to a tile in
// LDS instead, and after a barrier the whole workgroup writes the tiles of its batch entries, one contiguous range
// of the tensor, in whole lines.
auto Generator::ChooseCopyOutTile() -> void
{
    if (envInt("ACRO_HIP_COPY_OUT_TILE") < 0 || envInt("ACRO_HIP_LDS_COPY_OUT") < 0 || envInt("ACRO_HIP_PERSIST") > 0) return;
    // the kernel that writes the group's last result (for a kernel evaluated in steps: its last step)
    const int k = static_cast<int>(subs.size()) - 1;
    const Sub &s = subs[k];
    if (s.loopMode || s.matrixOp != 0 || s.op != '=' || s.out.repeated || s.splitLanes != 0 || s.tile.empty()) return;
    const UVarInfo &u = uvars[s.out.uvar];
    Storage &st = stores[u.storage];
    if (!st.elementLocal || st.anyRepeated || st.members.size() != 1 || st.batchDim != 0 || !u.fixed.empty() || u.viewOffset != 0 || st.transient) return;
    for (int j = 0; j <= k; ++j)
    {
        if (j != k && uvars[subs[j].out.uvar].storage == u.storage) return;
        for (const auto &r : subs[j].in)
        {
            if (uvars[r.uvar].storage == u.storage) return;
        }
    }
    if (st.tileSize > envInt("ACRO_HIP_COPY_OUT_MAX", 2048)) return;
    // the run of consecutive outputs of one work item: the trailing output dimensions that are tile indices
    long run = 1;
    for (size_t d = s.out.idx.size(); d-- > 0;)
    {
        if (!has(s.tile, s.out.idx[d])) break;
        run *= s.out.ext[d];
    }
    // Long runs per lane, or (any group) store instructions that fill less than 30 % of the lines they touch because
    // the register tile sits between the lanes' dimensions: 2D mass assembly "M_e_i1_i2_j1_j2 = B B B B D_e_k1_k2" with
    // lanes (i2, j2) and tile (i1, j1) writes pieces of 32 bytes 128 bytes apart (52 % of the HBM peak; through the
    // tile see the schedule comment).
    bool scattered = false;
    // (a run of four doubles per lane is enough: the lanes' pieces are 32 - 56 bytes long and as far apart, every store
    // instruction touches every line of the wavefront's range, and from HBM that costs more than it does out of the
    // memory-side cache.  Rotated tensors, by the lanes / through the tile: 7 x 9 operator 59 -> 72 %, 7 x 7 59 -> 75 %,
    // 5 x 5 64 -> 75 %, 4 x 4 69 -> 75 %, outer product of two 8-vectors 78 -> 91 %.)
    const long longRun = envInt("ACRO_HIP_COPY_OUT_RUN", 4);
    // (the check for scattered stores covers runs of up to seven, also inside a group, where the rule for long runs does
    // not apply: the p = 6 mass apply ends in runs of seven, 66 against 73 % of the HBM peak)
    if (run < std::max<long>(longRun, 8) && envInt("ACRO_HIP_COPY_OUT_TILE") < 2)
    {
        const int entries = static_cast<int>(std::max<long>(1, 64 / std::max<long>(1, s.laneCount)));
        const double coverage = WaveStoreLineCoverage(k, entries);
        scattered = s.laneCount >= 2 && (coverage < 0.01 * envInt("ACRO_HIP_COPY_OUT_COVERAGE", 30) ||
                                         (coverage < 0.95 && envInt("ACRO_HIP_COPY_OUT_WRITERS") >= 0 && WritesDominate()));
    }
    if (subs.size() != 1 && !scattered) return;
    if (run < longRun && !scattered) return;
    st.copyOutOnly = true;
    st.wantLds = true;
    st.liveTo = k;
    st.phaseFrom = st.phaseTo = PhaseOf(k);
}

auto Generator::ChooseStagedInputs() -> void
{
    if (envInt("ACRO_HIP_STAGE") < 0 || envInt("ACRO_HIP_PERSIST") > 0 || !opt.noalias) return;
    const int K = static_cast<int>(subs.size());
    for (size_t si = 0; si < stores.size(); ++si)
    {
        Storage &st = stores[si];
        if (st.written || st.members.size() != 1 || st.anyRepeated) continue;
        const UVarInfo &u = uvars[st.members[0]];
        if (!u.consistent || !u.batchDims.empty() || !u.plainView || !u.fixed.empty() || u.isVirtual) continue;
        if (GatherSlot(st.members[0]) >= 0) continue;
        if (u.size > kMaxStagedDoubles || u.size < 64) continue;
        bool ok = true, farApart = false;
        int first = -1, last = -1, laneDim = -1;
        for (int k = 0; k < K && ok; ++k)
        {
            const Sub &sk = subs[k];
            for (size_t v = 0; v < sk.in.size() && ok; ++v)
            {
                const VarRef &r = sk.in[v];
                if (uvars[r.uvar].storage != static_cast<int>(si)) continue;
                if (sk.loopMode || sk.matrixOp != 0 || IsUniform(sk, r, sk.tile)) ok = false;
                if (!ok) break;
                if (first < 0)
                {
                    first = k;
                    for (size_t d = 0; d < r.idx.size(); ++d)
                    {
                        if (has(sk.lane, r.idx[d])) laneDim = static_cast<int>(d);  // fastest dimension that a lane index addresses
                    }
                }
                last = k;
                farApart = farApart || LinesPerInstruction(sk, r, sk.lane) >= 16.0;
            }
            if (uvars[sk.out.uvar].storage == static_cast<int>(si)) ok = false;
        }
        if (!ok || !farApart || first < 0 || laneDim < 0) continue;
        st.staged = true;
        st.wantLds = true;
        st.liveTo = last;
        st.phaseFrom = 0;
        st.phaseTo = PhaseOf(last);
        // row-major, with the run of the dimensions faster than the lanes' made odd
        long run = 1;
        st.ldsStride.assign(st.dims.size(), 0);
        for (int d = static_cast<int>(st.dims.size()) - 1; d >= 0; --d)
        {
            if (d == laneDim && run % 2 == 0) run += 1;
            st.ldsStride[d] = static_cast<int>(run);
            run *= st.dims[d];
        }
        st.tileSize = static_cast<int>(run);
    }
}

// First-fit placement of the tiles that are live at the same time; returns doubles needed for nb entries.
auto Generator::PlaceLds(int nb) -> int
{
    std::vector<int> order;
    for (size_t si = 0; si < stores.size(); ++si)
    {
        if (stores[si].wantLds && stores[si].inLds) order.push_back(static_cast<int>(si));
    }
    std::sort(order.begin(), order.end(), [&](int a, int b) {
        if (stores[a].phaseFrom != stores[b].phaseFrom) return stores[a].phaseFrom < stores[b].phaseFrom;
        return a < b;
    });
    int total = 0;
    std::vector<int> placed;
    for (int si : order)
    {
        Storage &u = stores[si];
        const int need = LdsNeed(u, nb);
        int offset = 0;
        bool moved = true;
        while (moved)
        {
            moved = false;
            for (int pj : placed)
            {
                const Storage &p = stores[pj];
                const bool timeOverlap = !(p.phaseTo < u.phaseFrom || u.phaseTo < p.phaseFrom);
                const int pneed = LdsNeed(p, nb);
                const bool spaceOverlap = !(p.ldsOffset + pneed <= offset || offset + need <= p.ldsOffset);
                if (timeOverlap && spaceOverlap)
                {
                    offset = p.ldsOffset + pneed;
                    moved = true;
                }
            }
        }
        u.ldsOffset = offset;
        placed.push_back(si);
        total = std::max(total, offset + need);
    }
    return total;
}

// A second placement for chains: tiles that start in even phases are placed from the bottom, tiles that start in odd
// phases from the top of a region as large as the most that is ever live at once.  Where every tile lives for two
// consecutive phases (a sum-factorised chain) that region is all that is needed, while placing first-fit from the
// bottom leaves holes (p=8 mass apply: 1 900 instead of 2 710 doubles).  Returns the total, or -1 when some tile
// does not fit that way; offsets are only changed on success.
auto Generator::PlaceLdsFromBothEnds(int nb) -> int
{
    std::vector<int> order;
    int lastPhase = 0;
    for (size_t si = 0; si < stores.size(); ++si)
    {
        if (stores[si].wantLds && stores[si].inLds)
        {
            order.push_back(static_cast<int>(si));
            lastPhase = std::max(lastPhase, stores[si].phaseTo);
        }
    }
    std::sort(order.begin(), order.end(), [&](int a, int b) {
        if (stores[a].phaseFrom != stores[b].phaseFrom) return stores[a].phaseFrom < stores[b].phaseFrom;
        return a < b;
    });
    int ceiling = 0;
    for (int ph = 0; ph <= lastPhase; ++ph)
    {
        int live = 0;
        for (int si : order)
        {
            if (stores[si].phaseFrom <= ph && ph <= stores[si].phaseTo) live += LdsNeed(stores[si], nb);
        }
        ceiling = std::max(ceiling, live);
    }
    std::vector<int> placed, offsets;
    auto collides = [&](int si, int offset, int need, int &below, int &above) {
        for (size_t j = 0; j < placed.size(); ++j)
        {
            const Storage &q = stores[placed[j]];
            const int qneed = LdsNeed(q, nb);
            const bool timeOverlap = !(q.phaseTo < stores[si].phaseFrom || stores[si].phaseTo < q.phaseFrom);
            const bool spaceOverlap = !(offsets[j] + qneed <= offset || offset + need <= offsets[j]);
            if (timeOverlap && spaceOverlap)
            {
                below = offsets[j] - need;
                above = offsets[j] + qneed;
                return true;
            }
        }
        return false;
    };
    for (int si : order)
    {
        const int need = LdsNeed(stores[si], nb);
        const bool fromTop = stores[si].phaseFrom % 2 == 1;
        int offset = fromTop ? ceiling - need : 0, below = 0, above = 0;
        while (offset >= 0 && offset + need <= ceiling && collides(si, offset, need, below, above)) offset = fromTop ? below : above;
        if (offset < 0 || offset + need > ceiling) return -1;
        placed.push_back(si);
        offsets.push_back(offset);
    }
    for (size_t j = 0; j < placed.size(); ++j) stores[placed[j]].ldsOffset = offsets[j];
    return ceiling;
}

auto Generator::ChooseBatching() -> void
{
    ComputeLdsWishes();
    long maxLane = 1;
    for (const auto &s : subs) maxLane = std::max(maxLane, s.laneCount);

    NT = opt.force_nt > 0 ? opt.force_nt : envInt("ACRO_HIP_NT");
    if (NT <= 0)
    {
        NT = maxLane > 128 ? 256 : 128;
        // A streaming group (one phase, nothing kept in LDS) with more work items per batch entry than that runs
        // them in one pass of a larger workgroup instead of a loop of passes (geometric-factor setup, 1 000 items:
        // 475.7 -> 457.0 us with 1 024 lanes).  Groups with barriers measured slower that way (p=7 diffusion
        // apply: 1 283 against 940 us), so they keep 256.
        bool streaming = subs.back().phase == 0;
        for (const auto &st : stores) streaming = streaming && !st.wantLds;
        // Not for outputs shared between lanes, whose items are wavefront-sized pieces of rows anyway (64 x 64
        // matrix-vector products: 59 % of the HBM peak with 1 024 lanes, 71 % with 256).
        for (const auto &s : subs) streaming = streaming && s.splitLanes == 0;
        // Larger workgroups leave fewer registers per lane (128 at 1 024 lanes, 256 at 512): size them by the
        // values a lane holds at once.
        long live = 0;
        for (const auto &s : subs) live = std::max(live, s.loopMode ? 8 + s.tileCount : LoadsPerItem(s, s.tile) + s.tileCount);
        const long cap = live <= 48 ? 1024 : (live <= 100 ? 512 : 256);
        if (streaming && maxLane > 256) NT = static_cast<int>(std::min<long>(cap, (maxLane + 63) / 64 * 64));
        // Items that are one output of a few factors each ("A_e_i_j = B_e_i_j C_i_j" with 16 x 32 or 32 x 32): two
        // passes of half as many lanes (512 items: 63 - 72 -> 75 - 79 % of the HBM peak, 1 024: 63 - 75 -> 74 - 79 %).
        bool pointwise = streaming && maxLane > 256 && envInt("ACRO_HIP_LIGHT") < 2;
        for (const auto &s : subs) pointwise = pointwise && s.contr.empty() && s.tile.empty() && s.in.size() <= 3;
        if (pointwise) NT = static_cast<int>(std::min<long>(cap, std::max<long>(256, ((maxLane + 1) / 2 + 63) / 64 * 64)));
    }
    NB = opt.force_nb > 0 ? opt.force_nb : envInt("ACRO_HIP_NB");
    if (NB <= 0)
    {
        // As many batch entries as fit in one pass of the widest kernel, rounded down to a power of two.
        long fit = std::max<long>(1, NT / maxLane);
        NB = 1;
        while (NB * 2 <= fit) NB *= 2;
    }
    if (batch < 0) NB = 1;
    NB = static_cast<int>(std::min<long>(NB, E));

    // Lane utilisation at wavefront granularity (a wavefront with a single busy lane costs as much issue time as
    // a full one).  When the default leaves many lanes idle, look for a batch size / workgroup size that packs
    // wavefronts better; only switch for a clear gain, small workgroups overlap memory latency better.
    if (opt.force_nb <= 0 && opt.force_nt <= 0 && envInt("ACRO_HIP_NB") <= 0 && envInt("ACRO_HIP_NT") <= 0 && batch >= 0)
    {
        auto utilisation = [&](int nb, int nt) {
            double busy = 0.0, issued = 0.0;
            for (const auto &s : subs)
            {
                if (s.fusedWithPrev) continue;
                const long items = static_cast<long>(nb) * s.laneCount;
                const long passes = (items + nt - 1) / nt;
                const long tail = items - (passes - 1) * nt;
                const double weight = static_cast<double>(std::max<long>(1, s.tileCount * s.contrCount));
                busy += weight * items;
                issued += weight * 64.0 * ((passes - 1) * (nt / 64) + (tail + 63) / 64);
            }
            return busy / issued;
        };
        // Share of the arithmetic in kernels that need more than one pass of the workgroup over their items.
        auto multiPassShare = [&](int nb, int nt) {
            double all = 0.0, looped = 0.0;
            for (const auto &s : subs)
            {
                const double work = static_cast<double>(s.laneCount) * std::max<long>(1, s.tileCount * s.contrCount);
                all += work;
                if (static_cast<long>(nb) * s.laneCount > nt) looped += work;
            }
            return all > 0.0 ? looped / all : 0.0;
        };
        // Workgroups that declare much LDS leave few wavefronts resident on a compute unit (160 KB of LDS, handed
        // out in 1280-byte granules, 32 wavefronts at most) and so fewer loads in flight to cover the memory
        // latency; the square root follows the measured rates (p=3 diffusion apply in 256 lanes: 77.3 % of the
        // HBM peak with 32 resident wavefronts, 69.8 % with 12 and fuller wavefronts).
        auto occupancy = [&](int nb, int nt) {
            long bytes = static_cast<long>(PlaceLds(nb)) * 8;
            bytes = std::max<long>(1280, (bytes + 1279) / 1280 * 1280);
            const long groups = std::min<long>(160 * 1024 / bytes, 32 / (nt / 64));
            // wavefronts of a workgroup that have items at all, averaged over the arithmetic
            double all = 0.0, busy = 0.0;
            for (const auto &s : subs)
            {
                const double work = static_cast<double>(s.laneCount) * std::max<long>(1, s.tileCount * s.contrCount);
                all += work;
                busy += work * std::min<long>(nt / 64, (static_cast<long>(nb) * s.laneCount + 63) / 64);
            }
            const double waves = groups * (all > 0.0 ? busy / all : nt / 64.0);
            return std::sqrt(std::min(1.0, waves / 32.0));
        };
        for (auto &st : stores) st.inLds = st.wantLds;
        const double idle = utilisation(NB, NT);
        const double base = idle * occupancy(NB, NT);
        double best = base;
        int bestNB = NB, bestNT = NT;
        // Candidates: up to 16 entries per workgroup.  Kernels that carry at most a quarter of the arithmetic may
        // need several passes (a wide but cheap pointwise kernel should not dictate one entry per workgroup to
        // the narrow, expensive contractions around it); looping the contractions themselves measured slower
        // (p=3 mass apply with 12 entries in 128 lanes: 62.5 % against 76.7 %).  Never smaller workgroups than the
        // default, and everything that wants LDS must still fit.
        for (int nt : {128, 256})
        {
            if (nt < NT) continue;
            for (int nb = 1; nb <= 16 && nb <= E; ++nb)
            {
                if (nb * maxLane > 8L * nt || multiPassShare(nb, nt) > 0.25) break;
                if (PlaceLds(nb) > 64 * 1024 / 8) break;
                const double u = utilisation(nb, nt) * occupancy(nb, nt);
                if (u > best * 1.02)
                {
                    best = u;
                    bestNB = nb;
                    bestNT = nt;
                }
            }
        }
        // A workgroup with one batch entry and at least half of its lanes busy keeps it: the batch index is then
        // uniform, so its share of the address arithmetic is scalar, which measured no worse than fuller
        // wavefronts (p=2 mass assembly).  Groups that batch anyway take the better packing (p=1 mass apply:
        // 8 -> 14 entries per workgroup, 62.9 -> 74.9 % of the HBM peak; p=4: 2 -> 5 entries in 256 lanes,
        // 67.5 -> 72.0 %), and so do groups whose wavefronts would be mostly idle.
        const bool wanted = envInt("ACRO_HIP_PACK") > 0 || (envInt("ACRO_HIP_PACK") == 0 && (NB > 1 || idle < 0.5));
        if (wanted && best >= 1.1 * base)
        {
            NB = bestNB;
            NT = bestNT;
        }
        busyLanes = utilisation(NB, NT);
    }

    // A streaming group (one phase, nothing in LDS) whose workgroups move very little is bound by the rate at
    // which workgroups start, not by memory: with 1 - 2 KB per workgroup a copy reaches 72 % of the HBM peak and
    // an outer product 64 %.  Such groups take more batch entries per workgroup, in several passes of its lanes,
    // until a workgroup moves 8 KB (copy 72 -> 79 %, outer product 64 -> 88 %, batched 8 x 8 transpose 70 -> 77 %,
    // batched dot product 71 -> 76 %).  From 3 KB per workgroup on the same change measured slower
    // (`A_e_i += B_e_i` 77 -> 75 %, three-operand product 78 -> 75 %), hence the threshold.
    lightWorkgroups = false;
    if (opt.force_nb <= 0 && opt.force_nt <= 0 && envInt("ACRO_HIP_NB") <= 0 && envInt("ACRO_HIP_NT") <= 0 && batch >= 0 &&
        envInt("ACRO_HIP_LIGHT") >= 0)
    {
        bool streaming = subs.back().phase == 0;
        // (a small invariant operand that every workgroup copies to LDS first does not change that, and more entries per
        // workgroup share the copy: a 64 x 5 operator, two entries per workgroup, 39 % of the HBM peak)
        for (const auto &st : stores) streaming = streaming && ((st.staged && envInt("ACRO_HIP_LIGHT_STAGED") >= 0) || (!st.wantLds && !st.staged));
        bool shared = false;   // outputs shared by lanes: their workgroups keep 128 lanes (batched dot product with
                               // 16 entries per workgroup: 76 % in 128 lanes, 66 % in 256)
        for (const auto &s : subs)
        {
            streaming = streaming && (!s.loopMode || s.splitLanes != 0) && s.matrixOp == 0 && has(s.out.idx, batch);
            shared = shared || s.splitLanes != 0;
        }
        double perEntry = 0.0;
        std::set<int> counted;
        for (const auto &s : subs)
        {
            for (const auto &v : s.in)
            {
                if (has(v.idx, batch) && counted.insert(v.uvar).second) perEntry += 8.0 * static_cast<double>(v.size) / static_cast<double>(E);
            }
            const double written = 8.0 * static_cast<double>(s.out.size) / static_cast<double>(E);
            if (s.op != '=' && !counted.count(s.out.uvar)) perEntry += written;  // the old value is read first
            if (counted.insert(s.out.uvar).second) perEntry += written;
        }
        // (four and more factors per item: up to 4 KB; "A_e_i = B_e_i C_e_i D_i F_e" in workgroups of 128 lanes with
        // 3 KB each: 62 % of the HBM peak, with 16 entries in 256 lanes 78 %)
        size_t factors = 0;
        for (const auto &s : subs) factors = std::max(factors, s.in.size());
        if (streaming && perEntry > 0.0 && NB * perEntry < (factors >= 4 ? 4096.0 : 2560.0))
        {
            long nb = NB;
            while (nb * perEntry < 8192.0 && nb * 2 <= E && nb < 256) nb *= 2;
            if (nb > NB)
            {
                NB = static_cast<int>(nb);
                if (static_cast<long>(NB) * maxLane >= 512 && !shared) NT = std::max(NT, 256);
                lightWorkgroups = true;
            }
        }
        // One entry of 129 - 256 items per workgroup, an item per lane ("A_e_i_j = B_e_i_j C_i_j" with 16 x 16, rows of
        // 256): two entries in two passes (copy 71 -> 79 % of the HBM peak, with a shared factor 62 -> 74 %, product of
        // two 66 -> 77 %; four entries 77 / 70 %).
        else if (streaming && !shared && perEntry > 0.0 && perEntry < 8192.0 && NB == 1 && E >= 2 && maxLane > 128 && maxLane <= NT &&
                 envInt("ACRO_HIP_LIGHT") < 2)
        {
            NB = 2;
            lightWorkgroups = true;
        }
    }

    // Products of tiny element matrices whose operands are copied to LDS first (3 x 3 to 7 x 7): some 500 outputs per
    // workgroup of 256 lanes, two passes of its lanes (3 x 3: 75 % of the HBM peak with 14 or 28 entries per workgroup,
    // 82 % with 56; 5 x 5: 72 / 77 / 72 % with 5, 20 and 40; 7 x 7: 69 / 77 / 72 % with 5, 10 and 20).
    if (opt.force_nb <= 0 && opt.force_nt <= 0 && envInt("ACRO_HIP_NB") <= 0 && envInt("ACRO_HIP_NT") <= 0 && batch >= 0)
    {
        const Sub &last = subs.back();
        bool anyStagedCopy = false;
        for (const auto &r : last.in) anyStagedCopy = anyStagedCopy || uvars[r.uvar].isStagedCopy;
        if (anyStagedCopy && last.tile.empty() && last.laneCount < 64 && !last.loopMode)
        {
            NB = static_cast<int>(std::min<long>(E, std::max<long>(NB, 512 / last.laneCount)));
            NT = 256;
        }
        // (matrices of 11 x 11 and 13 x 13, whose indices cannot be split into blocks: four passes, 69 -> 85 and 81 %)
        else if (anyStagedCopy && last.tile.empty() && last.laneCount < 200 && !last.loopMode)
        {
            NB = static_cast<int>(std::min<long>(E, std::max<long>(NB, 1024 / last.laneCount)));
            NT = 256;
        }
    }

    // Products first, row sums second ("A_e_i = B_e_i_j C_e_j" with rows of odd length): the second step has one lane per
    // row, so a workgroup takes enough entries for a wavefront of rows (15 x 15: 1 entry 48 %, 4 entries 62 % of the HBM
    // peak; 27 x 27: 59 -> 60 %), within 32 KB of LDS.
    if (opt.force_nb <= 0 && opt.force_nt <= 0 && envInt("ACRO_HIP_NB") <= 0 && envInt("ACRO_HIP_NT") <= 0 && batch >= 0 &&
        subs.size() == 2 && subs[0].flatItems && uvars[subs[0].out.uvar].isVirtual && !uvars[subs[0].out.uvar].isStagedCopy &&
        subs[1].laneCount < 64)
    {
        long nb = (64 + subs[1].laneCount - 1) / subs[1].laneCount;
        while (nb > NB && PlaceLds(static_cast<int>(nb)) * 8 > 32 * 1024) --nb;
        if (nb > NB && nb <= E)
        {
            NB = static_cast<int>(nb);
            NT = 256;
        }
    }

    // Everything that wants LDS gets it while the workgroup stays within the 64 KB a workgroup may declare
    // statically; otherwise shrink the batch, and finally leave the largest tiles in device memory.
    const int budgetDoubles = 64 * 1024 / 8;
    for (auto &st : stores) st.inLds = st.wantLds;
    // An operand staged in LDS is copied once per workgroup: the workgroup must serve enough batch entries for
    // that copy to stay small against what the entries themselves move (one entry per 256 doubles staged).
    if (opt.force_nb <= 0 && envInt("ACRO_HIP_NB") <= 0 && batch >= 0)
    {
        long staged = 0;
        for (const auto &st : stores) staged += (st.staged && st.inLds) ? uvars[st.members[0]].size : 0;
        const long wanted = std::min<long>(std::min<long>(E, 32), (staged + 255) / 256);
        if (wanted > NB)
        {
            NB = static_cast<int>(wanted);
            if (static_cast<long>(NB) * maxLane > 2L * NT) NT = 256;
        }
    }
    while (true)
    {
        ldsDoubles = PlaceLds(NB);
        if (ldsDoubles <= budgetDoubles) break;
        bool dropped = false;  // staged operands are the first to go back to device memory
        for (auto &st : stores)
        {
            if (st.staged && st.inLds && !dropped)
            {
                st.inLds = false;
                dropped = true;
            }
        }
        if (dropped) continue;
        if (NB > 1 && opt.force_nb <= 0)
        {
            NB /= 2;
            continue;
        }
        int biggest = -1;
        for (size_t si = 0; si < stores.size(); ++si)
        {
            if (stores[si].inLds && (biggest < 0 || stores[si].tileSize > stores[biggest].tileSize))
                biggest = static_cast<int>(si);
        }
        if (biggest < 0) break;
        stores[biggest].inLds = false;
    }

    // Stores to device memory that may be dropped: every view of the tensor is transient, and every read of it
    // inside the group (operands and old values of += / -=) is served from registers or from the LDS tile.
    const int K = static_cast<int>(subs.size());
    for (size_t si = 0; si < stores.size(); ++si)
    {
        Storage &st = stores[si];
        st.elide = false;
        if (!st.transient || !st.written) continue;
        bool ok = true, anyRead = false;
        for (int k = 0; k < K; ++k)
        {
            const Sub &s = subs[k];
            for (size_t v = 0; v < s.in.size(); ++v)
            {
                if (uvars[s.in[v].uvar].storage != static_cast<int>(si)) continue;
                anyRead = true;
                if (FromRegisters(k, static_cast<int>(v))) continue;
                if (!(st.inLds && readCovered[k][v])) ok = false;
            }
            if (uvars[s.out.uvar].storage == static_cast<int>(si) && s.op != '=' && !s.forwardedOld)
            {
                if (!(st.inLds && oldCovered[k])) ok = false;
            }
        }
        st.elide = ok && anyRead;
    }
    // Padding of every tile is opt-in (see PadLdsTiles); the copies of operands that StageReusedOperands makes are
    // padded always: their lanes read them along any dimension (32 x 32 matrices with the second factor transposed:
    // a 32-way bank conflict on every read, 10.5 % of the HBM peak unpadded).
    if (envInt("ACRO_HIP_LDS_PAD") > 0)
        PadLdsTiles(budgetDoubles, false);
    else
        PadLdsTiles(budgetDoubles, true);

    // A launch that writes several times what it reads streams better with fewer workgroups resident per CU
    // (fewer write streams interleave at the memory controllers): workgroups of 128 lanes become 256 lanes with
    // the upper half idle, which halves the residency.  Measured: p=2 mass assembly 37.2 -> 34.3 us, p=3 mass
    // apply with all intermediates stored 355 -> 335 us; the same change costs the read-dominated p=3 mass
    // apply with transient intermediates 8 % (86.4 -> 93.6 us), hence the condition.
    if (NT == 128 && !lightWorkgroups && opt.force_nt <= 0 && envInt("ACRO_HIP_NT") <= 0 && batch >= 0)
    {
        double stored = 0.0, loaded = 0.0;
        std::set<int> counted;
        for (int k = 0; k < K; ++k)
        {
            const Sub &s = subs[k];
            if (StoresToGlobal(k)) stored += static_cast<double>(s.out.size) / static_cast<double>(E);
            for (size_t v = 0; v < s.in.size(); ++v)
            {
                const Source src = SourceOf(k, static_cast<int>(v));
                if ((src == kFromGlobal || src == kFromConstant) && has(s.in[v].idx, batch) &&
                    counted.insert(s.in[v].uvar).second)
                    loaded += static_cast<double>(s.in[v].size) / static_cast<double>(E);
            }
        }
        if (stored >= 3.0 * loaded && stored > 0.0)
        {
            NT = 256;
            // Results that leave through their LDS tiles are written as one contiguous range per tensor and
            // workgroup.  Twice the batch entries in workgroups of twice the lanes keep as many entries in flight
            // per CU and make those ranges twice as long (p=3 mass apply with all intermediates stored, 4 entries
            // in 256 lanes -> 8 in 512: 336 -> 311 us; 8 in 256 lanes 332 us, 16 in 1 024 lanes 331 us).
            bool throughLds = false;
            for (int k = 0; k < K; ++k) throughLds = throughLds || CopiesOutFromLds(k);
            if (throughLds && NB >= envInt("ACRO_HIP_WRITE_BATCH_FROM", 1) && opt.force_nb <= 0 && envInt("ACRO_HIP_NB") <= 0 && 2L * NB <= E && envInt("ACRO_HIP_WRITE_BATCH") >= 0)
            {
                const int wider = PlaceLds(2 * NB);
                if (wider <= budgetDoubles / 2)
                {
                    NB *= 2;
                    NT = 512;
                    ldsDoubles = wider;
                }
                else
                {
                    ldsDoubles = PlaceLds(NB);
                }
            }
        }
    }

    // The tighter placement is taken when it lets one more workgroup live on a compute unit (160 KB of LDS in
    // granules of 1 280 bytes, 32 wavefronts) and fewer than 16 wavefronts live there now; otherwise the tiles stay
    // where they are.  Mass apply at p = 8, one element per workgroup of 128 lanes: 7 -> 10 workgroups per unit,
    // 58.2 -> 60.1 % of the HBM peak; diffusion apply at p = 7 with 9 points per direction: 3 -> 4, 69.9 -> 71.5 %.
    // With 28 wavefronts resident already (mass apply at p = 4 and 5) more of them measured 0.5 points slower.
    if (ldsDoubles > 0 && envInt("ACRO_HIP_LDS_BOTH_ENDS") >= 0)
    {
        auto resident = [&](long doubles) {
            const long bytes = (std::max<long>(1, doubles) * 8 + 1279) / 1280 * 1280;
            return std::min<long>(160L * 1024 / bytes, 32 / std::max(1, NT / 64));
        };
        std::vector<int> before;
        for (const auto &st : stores) before.push_back(st.ldsOffset);
        const int tighter = PlaceLdsFromBothEnds(NB);
        if (tighter > 0 && tighter < ldsDoubles && resident(tighter) > resident(ldsDoubles) &&
            resident(ldsDoubles) * std::max(1, NT / 64) < 16)
            ldsDoubles = tighter;
        else
            for (size_t si = 0; si < stores.size(); ++si) stores[si].ldsOffset = before[si];
    }
}

// A kernel on its own whose tensors all have the batch index as their fastest dimension ("A_i_e = B_i_e C_i_e",
// structure-of-arrays layouts): with the work items numbered entry by entry, neighbouring lanes are a whole row of the
// batch apart (24 % of the HBM peak for that product).  The items are numbered with the entry fastest instead, 64 or
// more entries per workgroup, so that a wavefront reads and writes 64 consecutive entries of one row.
auto Generator::EntriesAreFastest() const -> bool
{
    if (envInt("ACRO_HIP_ENTRIES_FASTEST") < 0 || subs.size() != 1 || batch < 0 || E < 4096) return false;
    if (opt.force_nb > 0 || opt.force_nt > 0 || envInt("ACRO_HIP_NB") > 0 || envInt("ACRO_HIP_NT") > 0) return false;
    const Sub &s = subs[0];
    if (s.matrixOp != 0) return false;
    auto entryLast = [&](const VarRef &r) { return !r.repeated && !r.idx.empty() && r.idx.back() == batch; };
    if (!entryLast(s.out)) return false;
    for (const auto &r : s.in)
    {
        if (has(r.idx, batch) && !entryLast(r)) return false;
    }
    return true;
}

auto Generator::ChooseEntriesFastest() -> void
{
    entriesFastest = false;
    if (!EntriesAreFastest() || ldsDoubles > 0) return;
    const Sub &s = subs[0];
    if (s.splitLanes != 0 || s.loopMode || s.laneCount > 1024) return;
    NB = s.laneCount >= 4 ? 64 : (s.laneCount >= 2 ? 128 : 256);
    NT = 256;
    batchUniform = false;
    entriesFastest = true;
}

// ----------------------------------------------------------------------------- LDS bank conflicts
// LDS has 64 banks of 4 bytes; a wavefront's 8-byte accesses are served 32 lanes at a time, and lanes of such a
// group that hit the same bank at different addresses serialise.  All addresses are known here (lane index
// decomposition, tile strides), so the cost of every LDS access instruction can be counted and the tile strides
// padded until the count stops improving.  The count models 8-byte accesses only (the compiler merges adjacent
// ones into 16-byte accesses).  Padding is opt-in (ACRO_HIP_LDS_PAD=1): it changed nothing measurable for the
// p=3 mass apply, and on the p=7 diffusion chain a few hundred bytes of padding cost a resident workgroup (LDS is
// handed out in granules) and 20 % of the speed until the acceptance test counted in granules.

// Serialisation cycles of one access instruction whose lane l of the chain's item w reads `base(w)` doubles.
auto Generator::ConflictCycles(const std::vector<long> &addr) -> long
{
    long cycles = 0;
    for (size_t g = 0; g < addr.size(); g += 32)
    {
        // distinct addresses per bank (a double covers two consecutive 4-byte banks: bank pair = addr mod 32)
        std::map<long, std::set<long>> perBank;
        for (size_t l = g; l < std::min(addr.size(), g + 32); ++l) perBank[((addr[l] % 32) + 32) % 32].insert(addr[l]);
        size_t worst = 1;
        for (const auto &b : perBank) worst = std::max(worst, b.second.size());
        cycles += static_cast<long>(worst);
    }
    return cycles;
}

// Lane part of the LDS address of an occurrence for every work item of its kernel.
auto Generator::LaneAddresses(const Sub &s, const VarRef &r, int nb) const -> std::vector<long>
{
    const Storage &st = StoreOf(r.uvar);
    const long items = static_cast<long>(nb) * s.laneCount;
    std::vector<long> addr(items);
    for (long w = 0; w < items; ++w)
    {
        const long b = w / s.laneCount;
        long rest = w % s.laneCount;
        std::vector<int> value(nidx, 0);
        for (int j = static_cast<int>(s.lane.size()) - 1; j >= 0; --j)
        {
            value[s.lane[j]] = static_cast<int>(rest % extent[s.lane[j]]);
            rest /= extent[s.lane[j]];
        }
        long a = b * st.tileSize;
        for (size_t d = 0; d < r.idx.size(); ++d)
        {
            if (r.idx[d] != batch && has(s.lane, r.idx[d])) a += static_cast<long>(value[r.idx[d]]) * LdsStride(r.uvar, d);
        }
        addr[w] = a;
    }
    return addr;
}

auto Generator::LdsCostOfStorage(int si, int nb) const -> long
{
    long cost = 0;
    for (int k = 0; k < static_cast<int>(subs.size()); ++k)
    {
        const Sub &s = subs[k];
        if (s.loopMode) continue;
        for (size_t v = 0; v < s.in.size(); ++v)
        {
            if (uvars[s.in[v].uvar].storage != si || SourceOf(k, static_cast<int>(v)) != kFromLds) continue;
            std::set<int> seen;
            long ninstr = 1;
            for (int id : s.in[v].idx)
            {
                if ((has(s.tile, id) || has(s.contr, id)) && seen.insert(id).second) ninstr *= extent[id];
            }
            cost += ninstr * ConflictCycles(LaneAddresses(s, s.in[v], nb));
        }
        if (uvars[s.out.uvar].storage == si && (NeedsLdsCopy(k) || (s.op != '=' && !s.forwardedOld && OldValueInLds(k))))
            cost += s.tileCount * ConflictCycles(LaneAddresses(s, s.out, nb));
    }
    return cost;
}

auto Generator::SetLdsStrides(Storage &st, const std::vector<int> &pad, int padEntry) const -> void
{
    long run = 1;
    st.ldsStride.assign(st.dims.size(), 0);
    int p = 0;
    for (int d = static_cast<int>(st.dims.size()) - 1; d >= 0; --d)
    {
        if (d == st.batchDim) continue;
        st.ldsStride[d] = static_cast<int>(run);
        run = run * st.dims[d] + pad[p++];
    }
    st.tileSize = static_cast<int>(run + padEntry);
}

auto Generator::PadLdsTiles(int budgetDoubles, bool stagedCopiesOnly) -> void
{
    // Padding must not cost a resident workgroup: a CU has 160 KB of LDS, handed out in granules of 1 280 bytes
    // (the p=7 diffusion chain at 53 440 bytes fits three times, at 54 080 bytes only twice).
    auto resident = [](long doubles) {
        const long bytes = (std::max<long>(1, doubles) * 8 + 1279) / 1280 * 1280;
        return 160L * 1024 / bytes;
    };
    const long residentBefore = resident(PlaceLds(NB));
    for (size_t si = 0; si < stores.size(); ++si)
    {
        Storage &st = stores[si];
        if (!st.inLds || st.staged) continue;
        if (stagedCopiesOnly && !(st.members.size() == 1 && uvars[st.members[0]].isStagedCopy)) continue;
        const int ndim = static_cast<int>(st.dims.size()) - 1;
        // Rows of odd length in the copy of an operand get one double more, whatever the count below says: pairs of
        // values along a row are then 16 bytes aligned and read with one instruction (25 x 25 matrix products
        // 42 -> 50 % of the HBM peak, 27 x 27: 40 -> 57 %).
        std::vector<int> natural(ndim, 0);
        if (ndim >= 2 && st.dims.back() % 2 == 1 && st.dims.back() >= 17 && st.members.size() == 1 && uvars[st.members[0]].isStagedCopy)
            natural[0] = 1;
        std::vector<int> pad = natural, bestPad = natural;
        int bestEntry = 0;
        SetLdsStrides(st, pad, 0);
        long best = LdsCostOfStorage(static_cast<int>(si), NB);
        const long unpadded = best;
        // coordinate descent: one stride at a time, innermost first, two sweeps
        for (int sweep = 0; sweep < 2 && best > 0; ++sweep)
        {
            for (int p = 0; p <= ndim; ++p)
            {
                const int limit = p == ndim ? 16 : 8;
                for (int cand = 0; cand <= limit; ++cand)
                {
                    if (p == 0 && natural[0] == 1 && cand % 2 == 0) continue;  // rows stay even
                    std::vector<int> trial = bestPad;
                    int trialEntry = bestEntry;
                    if (p == ndim)
                        trialEntry = cand;
                    else
                        trial[p] = cand;
                    SetLdsStrides(st, trial, trialEntry);
                    const long c = LdsCostOfStorage(static_cast<int>(si), NB);
                    if (c < best)
                    {
                        best = c;
                        bestPad = trial;
                        bestEntry = trialEntry;
                    }
                }
            }
        }
        SetLdsStrides(st, bestPad, bestEntry);
        const int total = PlaceLds(NB);
        if (total > budgetDoubles || best >= unpadded || (envInt("ACRO_HIP_LDS_PAD") < 2 && resident(total) < residentBefore))
        {
            SetLdsStrides(st, natural, 0);  // no room or no gain: natural layout
            if (PlaceLds(NB) > budgetDoubles) SetLdsStrides(st, std::vector<int>(ndim, 0), 0);
        }
    }
    ldsDoubles = PlaceLds(NB);
}

}  // namespace codegen
}  // namespace acro
