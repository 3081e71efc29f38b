// Kernel code generator, the operator schedules (a dense operator applied to every entry, on the FP64 matrix cores).
#include "hip_codegen_impl.hpp"

namespace acro
{
namespace codegen
{

auto Generator::FoldPointwiseKernels() const -> void
{
    if (opKernelsReady) return;
    opKernelsReady = true;
    opKernels.clear();
    for (size_t k = 0; k < subs.size(); ++k)
    {
        const Sub &p = subs[k];
        bool folded = false;
        if (!opKernels.empty() && p.contr.empty() && p.op == '=' && p.matrixOp == 0 && !p.out.repeated && envInt("ACRO_HIP_OPERATOR_FOLD") >= 0)
        {
            Sub &m = opKernels.back();
            const int u = m.out.uvar;
            int reads = 0;
            bool sameShape = true;
            for (const auto &v : p.in)
            {
                if (uvars[v.uvar].storage != uvars[u].storage) continue;
                ++reads;
                sameShape = sameShape && v.uvar == u && v.idx == m.out.idx && !v.repeated;
            }
            bool readLater = false;
            for (size_t j = k + 1; j < subs.size(); ++j)
            {
                for (const auto &v : subs[j].in) readLater = readLater || uvars[v.uvar].storage == uvars[u].storage;
                readLater = readLater || uvars[subs[j].out.uvar].storage == uvars[u].storage;
            }
            if (reads == 1 && sameShape && !readLater && m.op == '=' && !m.contr.empty() && p.out.idx == m.out.idx &&
                stores[uvars[u].storage].transient && uvars[p.out.uvar].storage != uvars[u].storage)
            {
                for (const auto &v : p.in)
                {
                    if (v.uvar != u) m.in.push_back(v);
                }
                m.out = p.out;
                m.text += " ; " + p.text;
                folded = true;
            }
        }
        if (!folded) opKernels.push_back(p);
    }
}

auto Generator::NumOpKernels() const -> int
{
    FoldPointwiseKernels();
    return static_cast<int>(opKernels.size());
}

auto Generator::OpKernel(int k) const -> const Sub &
{
    FoldPointwiseKernels();
    return opKernels[k];
}

// `k`: the kernel of the group; `alone`: it is the whole group (inputs are then never written in the launch).
auto Generator::OperatorPattern(OperatorShape &o, int k, bool alone) const -> bool
{
    if ((alone && NumOpKernels() != 1) || batch < 0 || !opt.noalias || NumGatherSlots() > 0 || envInt("ACRO_HIP_OPERATOR") < 0 || opt.no_matrix_cores) return false;
    const Sub &s = OpKernel(k);
    if (s.matrixOp != 0 || s.in.size() < 2 || s.contr.empty() || s.out.repeated) return false;
    // the operator: the one operand without the batch index that carries contracted and free indices;
    // the vectors: the first operand with the batch index that carries every contracted index
    for (const auto &v : s.in)
    {
        bool contracted = false, free = false, all = true;
        for (int id : v.idx) (has(s.contr, id) ? contracted : free) = true;
        for (int id : s.contr) all = all && has(v.idx, id);
        if (!has(v.idx, batch) && contracted && free)
        {
            if (o.op) return false;
            o.op = &v;
        }
        else if (has(v.idx, batch) && all && !o.x)
            o.x = &v;
    }
    if (!o.op || !o.x) return false;
    for (const auto &v : s.in)
    {
        if (v.repeated || v.uvar == s.out.uvar || uvars[v.uvar].storage == uvars[s.out.uvar].storage) return false;
        if (alone && !IsPureInput(v.uvar)) return false;
    }
    // out = (e..., I...), X = (e..., J...), B = (I..., J...) or (J..., I...): the leading indices that the result
    // and X share, the batch index first, number the entries
    if (s.out.idx.empty()) return false;
    std::vector<int> lead, rows, cols;
    size_t sharedLeading = 0;
    while (sharedLeading < s.out.idx.size() && sharedLeading < o.x->idx.size() && s.out.idx[sharedLeading] == o.x->idx[sharedLeading] &&
           !has(o.op->idx, s.out.idx[sharedLeading]))
        ++sharedLeading;
    // (the batch index anywhere among them: "A_i_e_j = B_i_e_k C_k_j" has the entries (i, e))
    if (has(std::vector<int>(s.out.idx.begin(), s.out.idx.begin() + sharedLeading), batch))
    {
        const size_t shared = sharedLeading;
        lead.assign(s.out.idx.begin(), s.out.idx.begin() + shared);
        rows.assign(s.out.idx.begin() + shared, s.out.idx.end());
        cols.assign(o.x->idx.begin() + shared, o.x->idx.end());
        // component indices: what the result and the vectors share behind the operator's indices
        while (rows.size() > 1 && cols.size() > 1 && rows.back() == cols.back() && !has(o.op->idx, rows.back()) &&
               !has(s.contr, rows.back()))
        {
            o.comp *= extent[rows.back()];
            rows.pop_back();
            cols.pop_back();
        }
        // Component indices between the result's row indices ("J_e_q_m_n = X_e_i_m G_q_i_n": Jacobians with the
        // component m in front of the derivative index n): the vectors carry them last as before, and the results of
        // a trip are put into memory order as they are collected in LDS.
        std::vector<int> between;
        for (int id : rows)
        {
            if (!has(o.op->idx, id)) between.push_back(id);
        }
        if (!between.empty())
        {
            if (o.comp > 1 || !alone || between.size() >= cols.size() || envInt("ACRO_HIP_OPERATOR_ANY_ORDER") < 0) return false;
            if (!std::equal(between.begin(), between.end(), cols.end() - between.size())) return false;
            for (int id : between)
            {
                if (has(s.contr, id) || std::count(rows.begin(), rows.end(), id) != 1) return false;
            }
            // per output dimension behind the entries' (fastest first): does it number rows or components, what to
            // divide that number by, its extent and its stride in the result
            long rowDiv = 1, compDiv = 1;
            for (size_t d = rows.size(); d-- > 0;)
            {
                const bool isComp = has(between, rows[d]);
                OperatorShape::Term t;
                t.div = isComp ? compDiv : rowDiv;
                t.ext = extent[rows[d]];
                t.stride = s.out.stride[shared + d];
                (isComp ? o.outCompTerms : o.outRowTerms).push_back(t);
                (isComp ? compDiv : rowDiv) *= extent[rows[d]];
            }
            // (the components in the vectors' order: the same as in the result, or the numbering would differ)
            std::vector<int> inResultOrder;
            for (int id : rows)
            {
                if (has(between, id)) inResultOrder.push_back(id);
            }
            if (inResultOrder != between) return false;
            o.outMixed = true;
            o.comp = compDiv;
            std::vector<int> only;
            for (int id : rows)
            {
                if (!has(between, id)) only.push_back(id);
            }
            rows = only;
            cols.resize(cols.size() - between.size());
        }
    }
    else
    {
        // or the trailing ones, the entries being the fastest dimension of the result and of X
        size_t shared = 0;
        const size_t no = s.out.idx.size(), nx = o.x->idx.size();
        while (shared < no && shared < nx && s.out.idx[no - 1 - shared] == o.x->idx[nx - 1 - shared] &&
               !has(o.op->idx, s.out.idx[no - 1 - shared]))
            ++shared;
        lead.assign(s.out.idx.end() - shared, s.out.idx.end());
        rows.assign(s.out.idx.begin(), s.out.idx.end() - shared);
        cols.assign(o.x->idx.begin(), o.x->idx.end() - shared);
        o.trailing = true;
        if (!has(lead, batch)) return false;
    }
    if (rows.empty() || cols.empty()) return false;
    std::vector<int> plain = rows, swapped = cols;
    plain.insert(plain.end(), cols.begin(), cols.end());
    swapped.insert(swapped.end(), rows.begin(), rows.end());
    if (o.op->idx != plain && o.op->idx != swapped)
    {
        // Any other order of the same indices ("J_e_q_n_m = G_q_i_n X_e_i_m": row indices q, n around the column
        // index i): the operator's copy in LDS is filled through the strides of its dimensions.  Matrix cores only.
        std::vector<int> sorted = o.op->idx, all = plain;
        std::sort(sorted.begin(), sorted.end());
        std::sort(all.begin(), all.end());
        if (sorted != all || o.op->repeated || envInt("ACRO_HIP_OPERATOR_ANY_ORDER") < 0) return false;
        o.mixed = true;
        long rowDiv = 1;
        for (size_t d = rows.size(); d-- > 0;)
        {
            for (size_t q = 0; q < o.op->idx.size(); ++q)
            {
                if (o.op->idx[q] == rows[d]) o.rowTerms.push_back({rowDiv, static_cast<long>(extent[rows[d]]), o.op->stride[q]});
            }
            rowDiv *= extent[rows[d]];
        }
        long colDiv = 1;
        for (size_t d = cols.size(); d-- > 0;)
        {
            for (size_t q = 0; q < o.op->idx.size(); ++q)
            {
                if (o.op->idx[q] == cols[d]) o.colTerms.push_back({colDiv, static_cast<long>(extent[cols[d]]), o.op->stride[q]});
            }
            colDiv *= extent[cols[d]];
        }
    }
    o.transposed = !o.mixed && o.op->idx != plain;
    for (int id : cols)
    {
        if (!has(s.contr, id)) return false;
    }
    if (cols.size() != s.contr.size()) return false;
    o.rows = product(rows, extent);
    o.cols = product(cols, extent);
    o.entries = product(lead, extent) * o.comp;
    if (o.rows > 1024 || o.rows * o.cols > 4096)
    {
        // Too large for LDS as a whole (the gradient at every point of an element, 192 x 64; 375 x 125): blocks of
        // rows that fit, each applied by a launch of its own to all entries, on the matrix cores.  The vectors are
        // read once per block, from the last-level cache where they fit (generic schedule, a row per lane with the
        // operator read from device memory by every workgroup: 2.4 % of the HBM peak).
        const long paddedCols = (o.cols + 7) / 8 * 8;
        o.blockRows = 8192 / paddedCols / 16 * 16;
        if (!alone || o.cols > 256 || o.rows > 8192 || o.blockRows < 16 || o.trailing || envInt("ACRO_HIP_OPERATOR_BLOCKS") < 0 ||
            envInt("ACRO_HIP_OPERATOR_MFMA") < 0)
            return false;
    }
    if (o.outMixed)
    {
        if (o.comp > 16 || s.in.size() != 2 || envInt("ACRO_HIP_OPERATOR_BLOCKS") < 0 || envInt("ACRO_HIP_OPERATOR_MFMA") < 0 ||
            envInt("ACRO_HIP_OPERATOR_COMPONENTS") != 0)
            return false;
    }
    // With components a lane holds rows / 4 results for each of them: at most 16 blocks of 16 rows in all, more rows
    // in blocks of rows as above.
    if (o.comp > 1 && !o.trailing && alone && envInt("ACRO_HIP_OPERATOR_BLOCKS") >= 0 && envInt("ACRO_HIP_OPERATOR_MFMA") >= 0 && o.comp <= 16)
    {
        // (components between the row indices have no other schedule to fall back on: half as many registers again)
        const long most = 16 * ((o.outMixed ? 24 : 16) / o.comp);
        if (ComponentsTogether(o) && (o.blockRows > most || (o.blockRows == 0 && o.rows > most)))
        {
            // (a small operator that only its many components push into blocks of rows, 20 x 9 with nine components: two
            // launches, 26 us against 10 us on the generic schedule)
            if (o.rows * o.cols < 1024 && !o.outMixed) return false;
            o.blockRows = most;
        }
    }
    // With components: vectors in 8-byte loads, no pointwise factors, and only where the generic schedule (an
    // entry and a row per lane) runs out of scalar registers for the operator or of coalescing for its stores
    // (64 x 64 with three components: 7 % of the HBM peak).
    if (o.comp > 1 && (s.in.size() != 2 || !alone || envInt("ACRO_HIP_OPERATOR_COMPONENTS") < 0)) return false;
    o.cores = envInt("ACRO_HIP_OPERATOR_MFMA") >= 0;
    // 16-byte loads: along the vectors, or along the entries where those are the fastest dimension
    o.pairs = (o.trailing ? o.entries % 2 == 0 && uvars[s.out.uvar].viewOffset % 2 == 0 : o.cols % 2 == 0) &&
              uvars[o.x->uvar].viewOffset % 2 == 0 && o.comp == 1;
    for (const auto &v : s.in)
    {
        if (&v == o.op || &v == o.x) continue;
        const bool even = uvars[v.uvar].viewOffset % 2 == 0;
        if (v.idx == lead)
        {
            o.perEntry.push_back(&v);
            if (o.trailing) o.pairs = o.pairs && even;
        }
        else if (v.idx == s.out.idx)
        {
            o.perOutput.push_back(&v);
            if (o.trailing) o.pairs = o.pairs && even;
        }
        else if (v.idx == rows) o.perRow.push_back(&v);
        else if (v.idx == cols) o.perColumn.push_back(&v);
        else if (v.idx == o.x->idx)
        {
            o.perElement.push_back(&v);
            o.pairs = o.pairs && even;
        }
        else return false;
    }
    if (!o.cores) return o.rows >= 16 && o.cols >= 16 && !o.transposed && !o.mixed && !o.trailing && s.in.size() == 2 && o.comp == 1;  // (its lanes walk the operator's rows)
    // A lane holds cols / 4 vector elements and rows / 4 results; the padded operator must fit the 64 KB of LDS
    // that a workgroup may declare.
    if (o.blockRows > 0) return true;
    if (o.rows > 256 || o.cols > 256 || ((o.rows + 15) / 16 * 16) * ((o.cols + 7) / 8 * 8) > 8192) return false;
    if (o.trailing)
    {
        // Entries fastest: the generic schedule (one entry per lane, operator in scalar registers) streams whole
        // lines already; it falls behind as the operator grows (generic -> matrix cores: 8 x 8 86 -> 85 %,
        // 16 x 16 82 -> 84 %, 27 x 27 64 -> 78 %, 32 x 32 72 -> 80 %, 64 x 64 3 -> 65 %).  Two entries per lane
        // cost a large operator its registers (64 x 64: 72 us against 52 us with one entry per lane).
        if (o.rows * o.cols >= 2048) o.pairs = false;
        return o.rows * o.cols >= 512;
    }
    // Small operators: the generic schedule (operator in scalar registers, an entry or an output per lane) reads
    // and writes short pieces per lane and reaches 40 - 65 % of the HBM peak; 16 entries per wavefront on the
    // matrix cores reach 70 - 88 % as long as the entries' vectors come in 16-byte loads (even length) and five
    // or more rows fill the stores, or the vectors are long.  Measured wins: 8 x 4 53 -> 73 %, 16 x 4 43 -> 84 %,
    // 8 x 8 61 -> 85 %, 10 x 10 52 -> 81 %, 8 x 16 62 -> 85 %, 3 x 27 41 -> 73 %; losses, hence excluded:
    // 4 x 4 65 -> 49 %, 4 x 8 82 -> 77 %, 7 x 9 62 -> 57 %, 27 x 3 36 -> 28 %; 20 x 5 a tie.
    // (odd lengths: 9 x 9 47 -> 59 %, 25 x 25 45 -> 68 %, 27 x 27 46 -> 66 %; 5 x 5 63 -> 58 %)
    if (o.comp > 1) return o.rows * o.cols >= envInt("ACRO_HIP_OPERATOR_COMPONENTS_MIN", 256);
    // Two to four rows applied to vectors of 16 values and more (a gradient at a point, "G_e_d = D_d_i X_e_i"): the generic
    // schedule has a lane per result read the whole vector (from HBM: 3 x 32 30 %, 4 x 64 25 %, 2 x 64 43 %, 3 x 128 27 % of
    // the HBM peak); on the matrix cores 73 / 72 / 71 / 67 %, and no worse at 16 columns (2 / 3 / 4 x 16: 56 / 71 / 75 ->
    // 72 / 75 / 75 %).
    // Measured again from HBM with the generic schedule as it is now (results of long runs per lane leave through an LDS
    // tile, light workgroups take more entries): below 16 rows and 16 columns it is ahead of or level with the matrix
    // cores, whose 16 x 8 blocks such operators fill in small part (here / generic, % of the HBM peak: 5 x 4 51 / 73,
    // 8 x 4 61 / 74, 12 x 4 66 / 77, 6 x 6 64 / 75, 10 x 6 69 / 73, 5 x 8 69 / 73, 8 x 8 71 / 71, 5 x 12 65 / 74, 12 x 12
    // 71 / 70; with a factor per entry 8 x 8 61 / 73).  From 16 rows on the matrix cores stay ahead (32 x 4 81 / 69,
    // 32 x 8 81 / 68, 56 x 8 75 / 42), and so they do from 16 columns on (5 x 32 74 / 57, 6 x 64 70 / 15).
    // (a kernel on its own: inside a group the schedule is what joins two operators into one launch)
    if (alone && o.pairs && o.cols < 16 && o.rows < 16 && envInt("ACRO_HIP_OPERATOR_SMALL") >= 0) return false;
    const long fewRowsFrom = envInt("ACRO_HIP_OPERATOR_FEW_ROWS", 16);
    if (o.pairs && o.rows >= 2 && o.rows < 5 && fewRowsFrom > 0 && o.cols >= fewRowsFrom) return true;
    return o.pairs ? (o.rows >= 5 && o.cols >= 4) : (o.cols >= 16 || (o.cols >= 9 && o.rows >= 8));
}

// A group of several kernels each of which is a large dense operator applied to every entry ("U = B X D" followed
// by "Y = Bt U": a dense element operator applied and applied back) runs as one matrix-core launch per kernel,
// in order on the stream, with the intermediates in device memory.  The fused chain schedule keeps the
// intermediates on chip but gives a lane one entry and one row, which for large operators is bound by LDS reads:
// 64 x 64, 2^18 entries: 400 us fused against 134 us for the two launches; 27 x 27: 241 against 143 us; small
// operators stay fused (8 x 8 with a transient intermediate: 156 against 227 us; 12 x 10: 124 against 165 us).
auto Generator::UseOperatorSequence() const -> bool
{
    if (NumOpKernels() < 2 || envInt("ACRO_HIP_OPERATOR_SEQUENCE") < 0) return false;
    for (int k = 0; k < NumOpKernels(); ++k)
    {
        OperatorShape o;
        if (!OperatorPattern(o, k, false) || !o.cores || o.rows * o.cols < 512 || o.blockRows > 0) return false;
    }
    return true;
}

// Two operator-shaped kernels of which the second is applied to the first one's result: one kernel, the
// intermediate handed over through LDS (and stored as well unless it is transient).
auto Generator::OperatorPair(OperatorShape &first, OperatorShape &second) const -> bool
{
    if (NumOpKernels() != 2 || envInt("ACRO_HIP_OPERATOR_PAIR") < 0) return false;
    if (!OperatorPattern(first, 0, false) || !OperatorPattern(second, 1, false)) return false;
    if (!first.cores || !second.cores || first.trailing || second.trailing || first.comp > 1 || second.comp > 1) return false;
    if (first.blockRows > 0 || second.blockRows > 0) return false;
    const Sub &k0 = OpKernel(0), &k1 = OpKernel(1);
    if (k0.op != '=' || second.x->uvar != k0.out.uvar || second.x->idx != k0.out.idx) return false;
    if (uvars[k1.out.uvar].storage == uvars[k0.out.uvar].storage) return false;
    for (const auto &v : k1.in)
    {
        if (&v != second.x && uvars[v.uvar].storage == uvars[k0.out.uvar].storage) return false;
    }
    if (first.entries != second.entries || first.rows != second.cols) return false;
    // (2^19 - 2^22 entries, generic fused chain -> this kernel: 8 x 8 156 -> 142 us, 12 x 10 124 -> 93 us, 16 x 16 137 -> 61 us,
    // 20 x 12 125 -> 64 us, 24 x 20 277 -> 169 us; against two launches: 27 x 27 143 -> 74 us, 32 x 27 112 -> 62 us,
    // 64 x 27 190 -> 92 us)
    if (first.rows * first.cols < 64 || second.rows * second.cols < 64) return false;
    const long n1 = ((first.rows + 15) / 16 * 16) * (first.pairs ? (first.cols + 7) / 8 * 8 : (first.cols + 3) / 4 * 4);
    const long n2 = ((second.rows + 15) / 16 * 16) * ((second.cols + 3) / 4 * 4);
    return (n1 + n2 + 64 * (first.rows + 1)) * 8 <= 64 * 1024;
}

// Index of the operator's entry (row, j) in its own memory: rows by columns, columns by rows, or any order of its
// dimensions (then `row` and `j` are taken apart into the indices they number).
// Head of the loop in which the 256 lanes of a workgroup fill `count` doubles of LDS (the body follows, then the closing
// brace).  A counted loop that the compiler unrolls: all loads of a lane are in flight together.  Written as
// "for (f = threadIdx.x; f < count; f += 256)" it stayed a loop of one load and one wait per turn, 16 round trips to
// L2 for a 64 x 64 operator before a workgroup's first trip.
static void FillLoopHead(std::ostream &out, long count)
{
    const long turns = (count + 255) / 256;
    out << "#pragma unroll\n    for (int turn = 0; turn < " << turns << "; ++turn)\n    {\n";
    out << "        const int f = threadIdx.x + 256 * turn;\n";
    if (count % 256 != 0) out << "        if (f >= " << count << ") continue;\n";
}

auto Generator::OperatorEntry(const OperatorShape &shape, const std::string &row, const std::string &j, long allRows) const -> std::string
{
    if (!shape.mixed) return shape.transposed ? j + " * " + str(allRows) + " + " + row : row + " * " + str(shape.cols) + " + " + j;
    std::string expr;
    auto add = [&](const std::string &flat, const std::vector<OperatorShape::Term> &terms) {
        for (const auto &t : terms)
        {
            std::string v = t.div == 1 ? flat : "(" + flat + " / " + str(t.div) + ")";
            expr += (expr.empty() ? "" : " + ") + ("(" + v + " % " + str(t.ext) + ")") + " * " + str(t.stride);
        }
    };
    add(row, shape.rowTerms);
    add(j, shape.colTerms);
    return expr;
}

auto Generator::UseOperatorSchedule() const -> bool
{
    OperatorShape o, o2;
    return OperatorPattern(o) || OperatorPair(o, o2) || UseOperatorSequence();
}

auto Generator::EmitOperator(HipKernelPlan &plan) -> void
{
    {
        OperatorShape first, second;
        if (OperatorPair(first, second))
        {
            opSub = 0;
            EmitOperatorMatrixCores(plan, first, &second, 1);
            return;
        }
    }
    if (NumOpKernels() > 1)
    {
        opSequence = true;
        std::string schedule;
        int lds = 0;
        for (int k = 0; k < NumOpKernels(); ++k)
        {
            opSub = k;
            OperatorShape shape;
            OperatorPattern(shape, opSub, false);
            if (shape.trailing)
                EmitOperatorEntriesFastest(plan, shape);
            else
                EmitOperatorMatrixCores(plan, shape);
            schedule += plan.schedule;
            lds = std::max(lds, plan.lds_bytes);
        }
        plan.schedule = schedule;
        plan.lds_bytes = lds;
        plan.module_name = plan.launches.front().function_name;
        return;
    }
    const Sub &s = OpKernel(0);
    OperatorShape shape;
    OperatorPattern(shape);
    if (shape.blockRows > 0)
    {
        std::string schedule;
        int lds = 0;
        for (long r0 = 0; r0 < shape.rows; r0 += shape.blockRows, ++opBlock)
        {
            OperatorShape block = shape;
            block.allRows = shape.rows;
            block.rowOffset = r0;
            block.rows = std::min(shape.blockRows, shape.rows - r0);
            if (shape.comp > 1 && ComponentsTogether(shape))
                EmitOperatorComponents(plan, block);
            else
                EmitOperatorMatrixCores(plan, block);
            schedule += plan.schedule;
            lds = std::max(lds, plan.lds_bytes);
        }
        opBlock = 0;
        plan.schedule = schedule;
        plan.lds_bytes = lds;
        plan.module_name = plan.launches.front().function_name;
        return;
    }
    const VarRef *opr = shape.op, *x = shape.x;
    const long nJ = shape.cols, nI = shape.rows;
    const long E = shape.entries;        // entries of this schedule: all leading indices together
    if (shape.cores)
    {
        if (shape.trailing)
            EmitOperatorEntriesFastest(plan, shape);
        else if (shape.comp > 1 && ComponentsTogether(shape))
            EmitOperatorComponents(plan, shape);
        else
            EmitOperatorMatrixCores(plan, shape);
        return;
    }
    const int R = kOperatorEntriesPerLane;
    const long LI = (nI + 63) / 64 * 64;             // lanes per group of R entries: whole wavefronts
    // 512 lanes: the operator's copy in LDS allows four workgroups per CU, and the scalar loads of X come straight
    // from device memory, so the wavefronts in flight are what hides their latency (64 x 64: 104 us with 256
    // lanes, 87 us with 512, 93 us with 1 024).
    const int NTo = static_cast<int>(std::max<long>(512, LI));
    const long rowStride = nJ % 2 == 0 ? nJ + 1 : nJ;  // odd: the lanes' rows start in different LDS banks
    // Entries per workgroup: enough for the copy of B to stay small against what the entries move.
    // (64 x 64: 143 us with 16 entries per workgroup, 104 us with 64, the same with 128.)
    long groupsPerBlock = std::max<long>(1, (nI * nJ / 64 + R - 1) / R);
    groupsPerBlock = std::max<long>(groupsPerBlock, NTo / LI);
    const long NBo = groupsPerBlock * R;
    const long blocks = (E + NBo - 1) / NBo;
    for (const auto &st : stores)
    {
        long entries = 1;
        for (int d : st.dims) entries *= d;
        if (entries >= (1L << 31) - 1) wide = true;
    }

    const std::string dimName = mk.GetDimensionedNameString();
    char hex[32];
    std::snprintf(hex, sizeof(hex), "%016llx",
                  static_cast<unsigned long long>(hashString(dimName + "/operator/" + (Positional() ? "p" : "u"))));
    plan.module_name = std::string("acro_op_") + hex;
    std::ostringstream sched;
    sched << "operator schedule: " << nI << " x " << nJ << " operator in LDS (row stride " << rowStride << "), " << NBo
          << " entries per workgroup of " << NTo << " lanes, a lane keeps its row for " << R << " entries\n  [0] " << s.text << "\n";
    plan.schedule = sched.str();

    out << "// Generated by the acrotensor HIP code generator for gfx950.\n";
    {
        std::istringstream lines(plan.schedule);
        std::string l;
        while (std::getline(lines, l)) out << "// " << l << "\n";
    }
    const std::string B = PtrName(opr->uvar), X = PtrName(x->uvar), A = PtrName(s.out.uvar);
    const char *assign = s.op == '=' ? " = " : (s.op == '+' ? " += " : " -= ");
    out << "typedef const __attribute__((address_space(4))) double *acro_scalar_ptr;\n";
    out << "\nextern \"C\" __global__ __launch_bounds__(" << NTo << ") void " << plan.module_name << "(" << ParamList() << ")\n{\n";
    out << "    __shared__ double rows[" << nI * rowStride << "];\n";
    out << "    const int tid = threadIdx.x;\n";
    out << "    for (int i = tid; i < " << nI * nJ << "; i += " << NTo << ") rows[(i / " << nJ << ") * " << rowStride << " + i % " << nJ
        << "] = " << B << "[" << Lit(uvars[opr->uvar].viewOffset) << " + i];\n";
    out << "    __syncthreads();\n";
    out << "    const long e0 = (long)blockIdx.x * " << NBo << ";\n";
    out << "    for (int w = tid; w < " << groupsPerBlock * LI << "; w += " << NTo << ")\n    {\n";
    out << "        const int g = __builtin_amdgcn_readfirstlane(w / " << LI << ");  // whole wavefronts share the entries\n";
    out << "        const int i = w - g * " << LI << ";\n";
    out << "        const long e = e0 + g * " << R << ";\n";
    out << "        if (i >= " << nI << " || e >= " << E << ") continue;\n";
    out << "        const double *row = rows + i * " << rowStride << ";\n";
    out << "        const acro_scalar_ptr x = (acro_scalar_ptr)(" << X << " + " << Lit(uvars[x->uvar].viewOffset) << " + e * " << nJ
        << ");  // uniform: scalar loads\n";
    out << "        double *a = " << A << " + " << Lit(uvars[s.out.uvar].viewOffset) << " + e * " << nI << " + i;\n";
    out << "        if (e + " << R << " <= " << E << ")\n        {\n";
    for (int r = 0; r < R; ++r) out << "            double s" << r << " = 0.0;\n";
    // Eight terms per trip: the entry's operand words of one trip arrive in one scalar load per entry, and two
    // trips' worth in flight hide the scalar cache's latency (measured: 119 / 87 / 79 / 78 us at 2 / 4 / 8 / 16).
    out << "#pragma unroll 8\n";
    out << "            for (int j = 0; j < " << nJ << "; ++j)\n            {\n                const double b = row[j];\n";
    for (int r = 0; r < R; ++r) out << "                s" << r << " += b * x[" << r * nJ << " + j];\n";
    out << "            }\n";
    for (int r = 0; r < R; ++r) out << "            a[" << r * nI << "]" << assign << "s" << r << ";\n";
    out << "        }\n        else\n        {\n";
    out << "            for (int r = 0; e + r < " << E << "; ++r)\n            {\n                double sum = 0.0;\n";
    out << "                for (int j = 0; j < " << nJ << "; ++j) sum += row[j] * x[r * " << nJ << " + j];\n";
    out << "                a[r * " << nI << "]" << assign << "sum;\n            }\n        }\n    }\n}\n";

    plan.source = out.str();
    plan.nb = static_cast<int>(NBo);
    plan.lds_bytes = static_cast<int>(nI * rowStride * 8);
    FillParams(plan, false);
    HipLaunch launch;
    launch.function_name = plan.module_name;
    launch.grid = static_cast<unsigned>(blocks);
    launch.block = static_cast<unsigned>(NTo);
    for (int si = 0; si < NumParamStores(); ++si) launch.params.push_back(si);
    plan.launches.push_back(launch);
}

// The same on the FP64 matrix cores: a wavefront takes 16 entries at a time and forms their nI outputs with
// v_mfma_f64_16x16x4 (16 entries x 16 outputs x 4 terms per instruction).  The entries' vectors are the
// instruction's first operand, read with ordinary 16-byte vector loads (lane = entry + 16 * term group); the
// operator sits in LDS in the order the second operand wants it, one conflict-free 8-byte read per lane and
// instruction; a lane holds outputs (entry 4r + lane / 16, output lane % 16) in register r, so one store
// instruction writes four runs of 128 bytes.  The order of the terms inside a step is free as long as both
// operands agree: term group g of step s stands for j = 8 (s / 2) + 2 g + s % 2, which makes the entry's two
// doubles of a 16-byte load the operands of two successive steps.  MI355X's vector and matrix FP64 peaks are the
// same; what the matrix cores save is operand delivery: no scalar loads and 1/16 of the LDS reads.
// 64 x 64 on 2^18 entries: 47 - 51 us against 79 us with scalar loads (512 workgroups; 58 us with 1 024, 76 us
// with 2 048; loading the next 16 entries ahead of the arithmetic made no difference).
// With `next` (and its kernel `nextSub`) the result of this operator never leaves the chip: it is scaled, written
// to a per-wavefront piece of LDS in the result layout (entry 4r + lane / 16, output lane % 16), read back in the
// operand layout (entry lane % 16, term group lane / 16) and multiplied by the second operator.
auto Generator::EmitOperatorMatrixCores(HipKernelPlan &plan, const OperatorShape &shape, const OperatorShape *next, int nextSub) -> void
{
    const Sub &s = OpKernel(opSub);
    const VarRef &opr = *shape.op, &x = *shape.x;
    const long nI = shape.rows, nJ = shape.cols, E = shape.entries;
    // (a block of rows of a larger operator: rows row0 .. row0 + nI of nAll)
    const long nAll = shape.allRows > 0 ? shape.allRows : nI, row0 = shape.rowOffset;
    const bool first = opSub == 0 && opBlock == 0;
    // Sizes that the instruction's 16 x 4 blocks do not divide: the operator's copy in LDS is padded with zero
    // rows and columns, the entries' vectors read as zero past their end, outputs past the last row are not
    // stored.  Pairs of doubles (16-byte loads) need an even row length and an even first element.
    const bool pairs = shape.pairs;
    // (Vectors of odd length come in 8-byte loads, 32-byte pieces per entry.  Reading the 16 vectors of a trip as
    // one contiguous range into a per-wavefront piece of LDS first measured slower: 17 x 17 70 -> 58 %,
    // 33 x 33 63 -> 41 %, 9 x 9 59 -> 39 %; only 27 x 27 gained, 66 -> 70 %.)
    const long nIp = (nI + 15) / 16 * 16, nJp = pairs ? (nJ + 7) / 8 * 8 : (nJ + 3) / 4 * 4;
    const long tilesN = nIp / 16, steps = nJp / 4;
    // Rows that the instruction's 16-row blocks do not divide: a lane's stores would be single doubles in runs of 128
    // bytes that start anywhere in a line (81 x 8: 31 % of the HBM peak, 80 x 8: 73 %).  The 16 entries of a trip lie
    // next to each other in memory, so the wavefront collects their results in LDS in memory order and writes them
    // out as one contiguous range.
    // (all 16 entries at once where LDS allows, else 8 or 4 at a time)
    int stageRounds = 0;
    if (!next && shape.allRows == 0 && shape.comp == 1 && nI % 16 != 0 && envInt("ACRO_HIP_OPERATOR_STAGE_OUT") >= 0)
    {
        for (int rounds : {1, 2, 4})
        {
            if (stageRounds == 0 && (nIp * nJp + 64 / rounds * nI) * 8 <= 64 * 1024) stageRounds = rounds;
        }
    }
    const bool viaStage = stageRounds > 0;
    const long steps2 = (nI + 3) / 4;                 // the second operator contracts over this one's rows
    const long midStride = nI % 2 == 0 ? nI + 1 : nI; // odd: the lanes' rows of the hand-over buffer start in different banks
    const long tiles = (E + 15) / 16;
    const bool ragged = E % 16 != 0;
    // Equal work per CU matters more than the number of wavefronts: 256 CUs, a whole number of workgroups each
    // (640 workgroups: 10 - 15 % slower than 512 or 768 at every size).  How many is a matter of bytes in flight: a
    // wavefront requests 128 x columns bytes per trip, and a CU needs some 20 KB of loads outstanding to keep its
    // share of the memory system busy.  Measured on tensors that exceed the memory-side cache, % of the HBM peak with
    // 256 / 512 / 768 / 1 024 workgroups: 8 x 8 - / 56 / 70 / 73, 10 x 10 - / 57 / 70 / 75, 12 x 12 - / 66 / 75 / 73,
    // 8 x 16 - / 70 / 74 / 72, 17 x 17 43 / 65 / 74 / 73, 19 x 19 - / 71 / 75 / 72, 21 x 21 - / 69 / 73 / 68,
    // 40 x 12 - / 66 / 71 / 67, 27 x 27 55 / 74 / 71 / 67, 32 x 32 66 / 74 / 72 / 72, 48 x 48 66 / 71 / 67 / 67,
    // 64 x 64 on 2^18 entries 67 / 63 / - / 60, on 2^20 74 / 67 / - / 68, 128 x 32 78 / 72 / - / 74.
    // (An operator above 32 KB: one workgroup per CU, since every workgroup reads all of it.  192 x 64 on 2^15 entries:
    // 34.6 -> 26.9 us; 375 x 125 on 2^17: 410 -> 320 us; 1 024 workgroups: 558 us.  Results that leave through the
    // LDS stage keep two: 60 x 60 59 against 50 %.)
    long most = 512;
    if (nIp * nJp > 4096 || (nIp * nJp == 4096 && nIp >= 32 && !viaStage)) most = 256;
    else if (nJ <= 10) most = 1024;
    else if (nJ <= 24) most = 768;
    if (envInt("ACRO_HIP_OPERATOR_GROUPS") > 0) most = envInt("ACRO_HIP_OPERATOR_GROUPS");
    const long blocks = std::max<long>(1, std::min<long>(most, (tiles + 3) / 4));
    for (const auto &st : stores)
    {
        long entries = 1;
        for (int d : st.dims) entries *= d;
        if (entries >= (1L << 31) - 1) wide = true;
    }
    const std::string dimName = mk.GetDimensionedNameString();
    char hex[32];
    std::snprintf(hex, sizeof(hex), "%016llx",
                  static_cast<unsigned long long>(hashString(dimName + "/operator-mfma/" + str(opSub) + (shape.allRows > 0 ? "@" + str(row0) : std::string()) + "/" + (Positional() ? "p" : "u") + (pairs ? "2" : "1") + (next ? "+" : "") + (shape.comp > 1 ? "c" + str(shape.comp) : ""))));
    plan.module_name = std::string("acro_op_") + hex;
    std::ostringstream sched;
    sched << "operator schedule on the FP64 matrix cores: ";
    if (shape.allRows > 0) sched << "rows " << row0 << " - " << row0 + nI - 1 << " of the " << nAll << " x " << nJ << (shape.transposed ? " operator (stored transposed)" : (shape.mixed ? " operator (dimensions in another order)" : " operator"));
    else sched << nI << " x " << nJ << (shape.transposed ? " operator (stored transposed)" : (shape.mixed ? " operator (dimensions in another order)" : " operator"));
    sched << " in LDS in operand order";
    if (nIp != nI || nJp != nJ) sched << " (padded to " << nIp << " x " << nJp << ")";
    if (shape.comp > 1) sched << ", " << shape.comp << " components per vector element";
    if (viaStage) sched << ", results written out through LDS";
    sched << ", " << E << " entries, 16 per wavefront and trip, "
          << tilesN * steps << " v_mfma_f64_16x16x4 per trip, " << blocks << " workgroups of 256 lanes\n  [" << opSub << "] " << s.text << "\n";
    if (next)
        sched << "  [" << nextSub << "] " << OpKernel(nextSub).text << " : " << next->rows << " x " << next->cols << (next->transposed ? " operator (stored transposed)" : " operator")
              << " applied to the first result on chip (handed over through " << 16 * midStride * 8 << " bytes of LDS per wavefront)\n";
    plan.schedule = sched.str();

    if (first) out << "// Generated by the acrotensor HIP code generator for gfx950.\n";
    {
        std::istringstream lines(plan.schedule);
        std::string l;
        while (std::getline(lines, l)) out << "// " << l << "\n";
    }
    const std::string B = PtrName(opr.uvar), X = PtrName(x.uvar), A = PtrName(s.out.uvar);
    const bool stream = s.op == '=' && envInt("ACRO_HIP_NT_STORE") >= 0;
    // term group g (lane / 16) of step s stands for this j
    const std::string termOf = pairs ? "8 * (step >> 1) + 2 * (l >> 4) + (step & 1)" : "4 * step + (l >> 4)";
    out << (first ? "" : "\n") << "typedef double acro_double4 __attribute__((ext_vector_type(4)));\n";
    // Two doubles moved by one 16-byte instruction.  The type only promises the 8-byte alignment that every
    // operand has (a caller's device buffer, a slice at an odd offset of it); the hardware takes such
    // addresses for accesses to device memory.
    out << "typedef double acro_pair __attribute__((ext_vector_type(2), aligned(8)));\n";
    out << "\nextern \"C\" __global__ __launch_bounds__(256) void " << plan.module_name << "(" << ParamList() << ")\n{\n";
    out << "    __shared__ double frag[" << nIp * nJp << "];\n";
    FillLoopHead(out, nIp * nJp);
    out << "        const int l = f & 63, step = (f >> 6) % " << steps << ", t = (f >> 6) / " << steps << ";\n";
    out << "        const int row = 16 * t + (l & 15), j = " << termOf << ";\n";
    const std::string rowHere = row0 > 0 ? "(row + " + str(row0) + ")" : std::string("row");
    const std::string element = B + "[" + Lit(uvars[opr.uvar].viewOffset) + " + " + OperatorEntry(shape, rowHere, "j", nAll) + "]";
    if (nIp != nI || nJp != nJ)
        out << "        frag[f] = row < " << nI << " && j < " << nJ << " ? " << element << " : 0.0;\n    }\n";
    else
        out << "        frag[f] = " << element << ";\n    }\n";
    if (viaStage) out << "    __shared__ double stage[" << 64 / stageRounds * nI << "];\n";
    if (next)
    {
        // the second operator: its columns are the first one's rows, terms in natural order
        const long rows2P = (next->rows + 15) / 16 * 16;
        out << "    __shared__ double frag2[" << rows2P * steps2 * 4 << "];\n";
        out << "    __shared__ double stage[" << 4 * 16 * midStride << "];\n";
        FillLoopHead(out, rows2P * steps2 * 4);
        out << "        const int l = f & 63, step = (f >> 6) % " << steps2 << ", t = (f >> 6) / " << steps2 << ";\n";
        out << "        const int row = 16 * t + (l & 15), j = 4 * step + (l >> 4);\n";
        out << "        frag2[f] = row < " << next->rows << " && j < " << nI << " ? " << PtrName(next->op->uvar) << "[" << Lit(uvars[next->op->uvar].viewOffset)
            << (next->transposed ? " + j * " + str(next->rows) + " + row]" : " + row * " + str(nI) + " + j]") << " : 0.0;\n    }\n";
    }
    out << "    __syncthreads();\n";
    out << "    const int lane = threadIdx.x & 63, g = lane >> 4, c = lane & 15;\n";
    // (A contiguous range of trips per workgroup instead of this stride: the same or up to 8 % slower.)
    out << "    const long waves = (long)gridDim.x * 4;\n";
    out << "    for (long tile = (long)blockIdx.x * 4 + (threadIdx.x >> 6); tile < " << tiles << "; tile += waves)\n    {\n";
    // (a kernel that the compiler can only fit into the registers with spills is compiled again with this macro:
    // the operator's values are then read from LDS on every trip instead of being kept in registers across trips)
    out << "#ifdef ACRO_KEEP_OPERATOR_IN_LDS\n        __asm__ volatile(\"\" ::: \"memory\");\n#endif\n";
    if (ragged)
        out << "        const long ex = tile * 16 + c < " << E << " ? tile * 16 + c : " << E - 1 << ";  // past the end: any valid entry, never stored\n";
    else
        out << "        const long ex = tile * 16 + c;\n";
    if (pairs)
    {
        out << "        const double *x = " << X << " + " << Lit(uvars[x.uvar].viewOffset) << " + ex * " << nJ << " + 2 * g;\n";
        out << "        double2 xv[" << nJp / 8 << "];\n";
        out << "#pragma unroll\n";
        out << "        for (int q = 0; q < " << nJp / 8 << "; ++q) xv[q] = ";
        if (nJp != nJ) out << "8 * q + 2 * g >= " << nJ << " ? double2{0.0, 0.0} : ";
        out << "[&] { const acro_pair t = *reinterpret_cast<const acro_pair *>(x + 8 * q); return double2{t.x, t.y}; }();\n";
        for (const VarRef *w : shape.perElement)
        {
            out << "#pragma unroll\n";
            out << "        for (int q = 0; q < " << nJp / 8 << "; ++q)\n        {\n";
            if (nJp != nJ) out << "            if (8 * q + 2 * g >= " << nJ << ") continue;\n";
            out << "            const acro_pair f = *reinterpret_cast<const acro_pair *>(" << PtrName(w->uvar) << " + " << Lit(uvars[w->uvar].viewOffset)
                << " + ex * " << nJ << " + 2 * g + 8 * q);\n            xv[q].x *= f.x;\n            xv[q].y *= f.y;\n        }\n";
        }
        for (const VarRef *w : shape.perColumn)
        {
            out << "#pragma unroll\n";
            out << "        for (int q = 0; q < " << nJp / 8 << "; ++q)\n        {\n";
            if (nJp != nJ) out << "            if (8 * q + 2 * g >= " << nJ << ") continue;\n";
            out << "            const double *f = " << PtrName(w->uvar) << " + " << Lit(uvars[w->uvar].viewOffset)
                << " + 2 * g + 8 * q;\n            xv[q].x *= f[0];\n            xv[q].y *= f[1];\n        }\n";
        }
    }
    else
    {
        const long C = shape.comp;
        if (C > 1)
            out << "        const double *x = " << X << " + " << Lit(uvars[x.uvar].viewOffset) << " + (ex / " << C << ") * " << nJ * C
                << " + ex % " << C << " + g * " << C << ";\n";
        else
            out << "        const double *x = " << X << " + " << Lit(uvars[x.uvar].viewOffset) << " + ex * " << nJ << " + g;\n";
        out << "        double xv[" << steps << "];\n";
        out << "#pragma unroll\n";
        out << "        for (int q = 0; q < " << steps << "; ++q) xv[q] = ";
        if (nJp != nJ) out << "4 * q + g >= " << nJ << " ? 0.0 : ";
        out << "x[" << 4 * C << " * q];\n";
        for (const VarRef *w : shape.perElement)
        {
            out << "#pragma unroll\n";
            out << "        for (int q = 0; q < " << steps << "; ++q) ";
            if (nJp != nJ) out << "if (4 * q + g < " << nJ << ") ";
            out << "xv[q] *= " << PtrName(w->uvar) << "[" << Lit(uvars[w->uvar].viewOffset) << " + ex * " << nJ << " + g + 4 * q];\n";
        }
        for (const VarRef *w : shape.perColumn)
        {
            out << "#pragma unroll\n";
            out << "        for (int q = 0; q < " << steps << "; ++q) ";
            if (nJp != nJ) out << "if (4 * q + g < " << nJ << ") ";
            out << "xv[q] *= " << PtrName(w->uvar) << "[" << Lit(uvars[w->uvar].viewOffset) << " + g + 4 * q];\n";
        }
    }
    out << "        acro_double4 acc[" << tilesN << "];\n";
    out << "#pragma unroll\n";
    out << "        for (int t = 0; t < " << tilesN << "; ++t) acc[t] = acro_double4{0.0, 0.0, 0.0, 0.0};\n";
    out << "#pragma unroll\n";
    out << "        for (int step = 0; step < " << steps << "; ++step)\n        {\n";
    if (pairs)
        out << "            const double xs = (step & 1) ? xv[step >> 1].y : xv[step >> 1].x;\n";
    else
        out << "            const double xs = xv[step];\n";
    out << "#pragma unroll\n";
    out << "            for (int t = 0; t < " << tilesN << "; ++t)\n";
    out << "                acc[t] = __builtin_amdgcn_mfma_f64_16x16x4f64(xs, frag[(t * " << steps << " + step) * 64 + lane], acc[t], 0, 0, 0);\n";
    out << "        }\n";
    // Stores of one operator's results (or, with toLds, their hand-over to the second operator).
    auto emitResults = [&](const Sub &ks, const OperatorShape &sh, long rows, const std::string &accName, bool toLds) {
        const long rowsP = (rows + 15) / 16 * 16;
        const bool streams = ks.op == '=' && envInt("ACRO_HIP_NT_STORE") >= 0;
        const long C = sh.comp;
        // (a block of rows: the entries' results lie `stride` apart and start at row `off`)
        const long stride = sh.allRows > 0 ? sh.allRows : rows, off = sh.rowOffset;
        if (viaStage)
        {
            const int perRound = 4 / stageRounds;   // result registers (entries g + 4 r) per round
            out << "        double *mid = stage + (threadIdx.x >> 6) * " << 4 * perRound * rows << ";\n";
            for (int h = 0; h < stageRounds; ++h)
            {
                out << "#pragma unroll\n";
                out << "        for (int r = " << h * perRound << "; r < " << (h + 1) * perRound << "; ++r)\n        {\n";
                std::string staged = accName + "[t][r]";
                const bool scaledHere = !sh.perEntry.empty() || !sh.perOutput.empty() || !sh.perRow.empty();
                if (scaledHere)
                    out << "            const long en = " << (ragged ? "tile * 16 + g + 4 * r < " + str(E) + " ? tile * 16 + g + 4 * r : " + str(E - 1) : std::string("tile * 16 + g + 4 * r")) << ";\n";
                if (!sh.perEntry.empty())
                {
                    out << "            const double se = ";
                    for (size_t i = 0; i < sh.perEntry.size(); ++i)
                        out << (i ? " * " : "") << PtrName(sh.perEntry[i]->uvar) << "[" << Lit(uvars[sh.perEntry[i]->uvar].viewOffset) << " + en]";
                    out << ";\n";
                    staged += " * se";
                }
                for (const VarRef *w : sh.perOutput)
                    staged += " * " + PtrName(w->uvar) + "[" + Lit(uvars[w->uvar].viewOffset) + " + en * " + str(rows) + " + 16 * t + c]";
                for (const VarRef *w : sh.perRow)
                    staged += " * " + PtrName(w->uvar) + "[" + Lit(uvars[w->uvar].viewOffset) + " + 16 * t + c]";
                out << "#pragma unroll\n";
                out << "            for (int t = 0; t < " << rowsP / 16 << "; ++t)\n";
                out << "                if (16 * t + c < " << rows << ") mid[(4 * " << (h ? "(r - " + str(static_cast<long>(h * perRound)) + ")" : std::string("r")) << " + g) * " << rows << " + 16 * t + c] = " << staged << ";\n";
                out << "        }\n";
                out << "        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, \"wavefront\");\n        __builtin_amdgcn_wave_barrier();\n";
                out << "        {\n";
                const long firstEntry = 4L * h * perRound, entries = 4L * perRound;
                out << "            double *a = " << PtrName(ks.out.uvar) << " + " << Lit(uvars[ks.out.uvar].viewOffset) << " + (tile * 16 + " << firstEntry << ") * " << rows << ";\n";
                if (ragged)
                    out << "            const long left = " << E << " - tile * 16 - " << firstEntry << ";\n"
                        << "            const int count = (int)(left < 0 ? 0 : (left < " << entries << " ? left : " << entries << ")) * " << rows << ";\n";
                else
                    out << "            const int count = " << entries * rows << ";\n";
                out << "            for (int i = lane; i < count; i += 64)\n";
                if (streams)
                    out << "                __builtin_nontemporal_store(mid[i], a + i);\n";
                else
                    out << "                a[i]" << (ks.op == '=' ? " = " : (ks.op == '+' ? " += " : " -= ")) << "mid[i];\n";
                out << "        }\n";
                out << "        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, \"wavefront\");\n        __builtin_amdgcn_wave_barrier();\n";
            }
            return;
        }
        if (!toLds && C == 1)
            out << "        double *a = " << PtrName(ks.out.uvar) << " + " << Lit(uvars[ks.out.uvar].viewOffset) << " + (tile * 16 + g) * " << stride << (off ? " + " + str(off) : std::string()) << " + c;\n";
        out << "#pragma unroll\n";
        out << "        for (int r = 0; r < 4; ++r)\n        {\n";
        if (ragged) out << "            if (tile * 16 + g + 4 * r >= " << E << ") continue;\n";
        if (!toLds && C > 1)
        {
            // entry (e, k): its outputs lie C doubles apart
            out << "            const long en_ = tile * 16 + g + 4 * r;\n";
            out << "            double *a = " << PtrName(ks.out.uvar) << " + " << Lit(uvars[ks.out.uvar].viewOffset) << " + (en_ / " << C << ") * "
                << stride * C << (off ? " + " + str(off * C) : std::string()) << " + en_ % " << C << " + c * " << C << ";\n";
        }
        // the result's pointwise factors
        std::string value = accName + "[t][r]";
        const bool scaled = !sh.perEntry.empty() || !sh.perOutput.empty() || !sh.perRow.empty();
        if (scaled) out << "            const long en = tile * 16 + g + 4 * r;\n";
        if (!sh.perEntry.empty())
        {
            out << "            const double se = ";
            for (size_t i = 0; i < sh.perEntry.size(); ++i)
                out << (i ? " * " : "") << PtrName(sh.perEntry[i]->uvar) << "[" << Lit(uvars[sh.perEntry[i]->uvar].viewOffset) << " + en]";
            out << ";\n";
            value += " * se";
        }
        for (const VarRef *w : sh.perOutput)
            value += " * " + PtrName(w->uvar) + "[" + Lit(uvars[w->uvar].viewOffset) + " + en * " + str(stride) + (off ? " + " + str(off) : std::string()) + " + 16 * t + c]";
        for (const VarRef *w : sh.perRow)
            value += " * " + PtrName(w->uvar) + "[" + Lit(uvars[w->uvar].viewOffset) + (off ? " + " + str(off) : std::string()) + " + 16 * t + c]";
        out << "#pragma unroll\n";
        out << "            for (int t = 0; t < " << rowsP / 16 << "; ++t)\n";
        std::string guard = rowsP != rows ? "if (16 * t + c < " + str(rows) + ") " : "";
        if (toLds)
            out << "                " << guard << "mid[(4 * r + g) * " << midStride << " + 16 * t + c] = " << value << ";\n";
        else if (C > 1)
            out << "                " << guard << "a[" << 16 * C << " * t]" << (ks.op == '=' ? " = " : (ks.op == '+' ? " += " : " -= ")) << value << ";\n";
        else if (streams)
            out << "                " << guard << "__builtin_nontemporal_store(" << value << ", a + 4 * r * " << stride << " + 16 * t);\n";
        else
            out << "                " << guard << "a[4 * r * " << stride << " + 16 * t]" << (ks.op == '=' ? " = " : (ks.op == '+' ? " += " : " -= ")) << value << ";\n";
        out << "        }\n";
    };
    (void)A;
    (void)stream;
    if (!next)
        emitResults(s, shape, nI, "acc", false);
    else
    {
        const long rows2 = next->rows, rows2P = (rows2 + 15) / 16 * 16;
        out << "        double *mid = stage + (threadIdx.x >> 6) * " << 16 * midStride << ";\n";
        out << "        {\n";
        emitResults(s, shape, nI, "acc", true);
        out << "        }\n";
        if (!stores[uvars[s.out.uvar].storage].transient)
        {
            // the first result is wanted in device memory as well
            out << "        {\n";
            emitResults(s, shape, nI, "acc", false);
            out << "        }\n";
        }
        // a wavefront's LDS accesses complete in program order: no barrier, only the compiler kept from reordering
        out << "        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, \"wavefront\");\n        __builtin_amdgcn_wave_barrier();\n";
        out << "        acro_double4 acc2[" << rows2P / 16 << "];\n";
        out << "#pragma unroll\n";
        out << "        for (int t = 0; t < " << rows2P / 16 << "; ++t) acc2[t] = acro_double4{0.0, 0.0, 0.0, 0.0};\n";
        out << "#pragma unroll\n";
        out << "        for (int step = 0; step < " << steps2 << "; ++step)\n        {\n";
        out << "            const double us = ";
        if (steps2 * 4 != nI) out << "4 * step + g >= " << nI << " ? 0.0 : ";
        out << "mid[c * " << midStride << " + 4 * step + g]";
        // the second kernel's factors on its operand side: per element of the intermediate, or per column
        const std::string inRange = steps2 * 4 != nI ? "(4 * step + g < " + str(nI) + " ? " : "";
        const std::string otherwise = steps2 * 4 != nI ? " : 0.0)" : "";
        for (const VarRef *w : next->perElement)
            out << " * " << inRange << PtrName(w->uvar) << "[" << Lit(uvars[w->uvar].viewOffset) << " + ex * " << nI << " + 4 * step + g]" << otherwise;
        for (const VarRef *w : next->perColumn)
            out << " * " << inRange << PtrName(w->uvar) << "[" << Lit(uvars[w->uvar].viewOffset) << " + 4 * step + g]" << otherwise;
        out << ";\n";
        out << "#pragma unroll\n";
        out << "            for (int t = 0; t < " << rows2P / 16 << "; ++t)\n";
        out << "                acc2[t] = __builtin_amdgcn_mfma_f64_16x16x4f64(us, frag2[(t * " << steps2 << " + step) * 64 + lane], acc2[t], 0, 0, 0);\n";
        out << "        }\n";
        out << "        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, \"wavefront\");\n        __builtin_amdgcn_wave_barrier();\n";
        emitResults(OpKernel(nextSub), *next, rows2, "acc2", false);
    }
    out << "    }\n}\n";


    plan.source = out.str();
    plan.nb = 64;
    plan.lds_bytes = static_cast<int>((nIp * nJp + (next ? (next->rows + 15) / 16 * 16 * steps2 * 4 + 64 * midStride : 0) + (viaStage ? 64 / stageRounds * nI : 0)) * 8);
    FillParams(plan, false);
    HipLaunch launch;
    launch.function_name = plan.module_name;
    launch.grid = static_cast<unsigned>(blocks);
    launch.block = 256;
    for (int si = 0; si < NumParamStores(); ++si) launch.params.push_back(si);
    plan.launches.push_back(launch);
}

// Vectors and results with component indices behind the operator's ("V_e_q_c = B_q_i X_e_i_c", a vector field
// interpolated component by component).  A wavefront takes 16 entries (all their components) per trip: a lane loads the
// C components of its vector elements, which lie next to each other, every block of the operator read from LDS serves C
// instructions, and the results of a trip, 16 entries x rows x C doubles that lie next to each other in memory, are
// collected in LDS in memory order and written out as one range (all 16 entries at once where LDS allows, else 8 or 4
// at a time, else by the lanes that hold them).  Treating (entry, component) pairs as the entries instead, as this
// schedule first did, reads and writes single doubles C apart: 27 x 27 x 3 62 %, 64 x 27 x 3 55 % of the HBM peak.
// Measured against the entries (entry, component): 16 x 16 x 3 68 -> 72 %, 27 x 27 x 3 62 -> 68 %, 125 x 64 x 3 (two blocks
// of rows) 23 -> 34 %; 64 x 64 x 3 61 -> 59 % and 216 x 125 x 3 21 -> 15 %, which keep the entries (entry, component).
auto Generator::ComponentsTogether(const OperatorShape &o) const -> bool
{
    if (o.comp <= 1 || o.comp > 16 || o.trailing || envInt("ACRO_HIP_OPERATOR_COMPONENTS") >= 2) return false;
    if (o.outMixed) return true;
    const long padded = ((o.rows + 15) / 16 * 16) * ((o.cols + 3) / 4 * 4);
    // (on tensors that exceed the memory-side cache, entries (entry, component) against the components together:
    // 64 x 27 x 3 58 -> 64 %, 48 x 48 x 2 66 -> 66 % (re-launched on the same tensors 66 -> 74 %), 64 x 64 x 3 67 -> 58 %;
    // non-temporal stores of the single doubles C apart: slower everywhere, 27 x 27 x 3 62 -> 56 %)
    return padded <= 2304 || (o.rows * o.cols > 4096 && o.cols <= 64);
}

auto Generator::EmitOperatorComponents(HipKernelPlan &plan, const OperatorShape &shape) -> void
{
    const Sub &s = OpKernel(opSub);
    const VarRef &opr = *shape.op, &x = *shape.x;
    const long nI = shape.rows, nJ = shape.cols, C = shape.comp, NE = shape.entries / shape.comp;
    const long nAll = shape.allRows > 0 ? shape.allRows : nI, row0 = shape.rowOffset;
    const bool first = opSub == 0 && opBlock == 0;
    const long nIp = (nI + 15) / 16 * 16, nJp = (nJ + 3) / 4 * 4;
    const long tilesN = nIp / 16, steps = nJp / 4;
    const long tiles = (NE + 15) / 16;
    const bool ragged = NE % 16 != 0;
    int stageRounds = 0;
    if (shape.allRows == 0 && envInt("ACRO_HIP_OPERATOR_STAGE_OUT") >= 0)
    {
        for (int rounds : {1, 2, 4})
        {
            if (stageRounds == 0 && (nIp * nJp + 64 / rounds * nI * C) * 8 <= 64 * 1024) stageRounds = rounds;
        }
    }
    const long most = nIp * nJp > 4096 ? 256 : 512;
    const long blocks = std::max<long>(1, std::min<long>(most, (tiles + 3) / 4));
    for (const auto &st : stores)
    {
        long entries = 1;
        for (int d : st.dims) entries *= d;
        if (entries >= (1L << 31) - 1) wide = true;
    }
    const std::string dimName = mk.GetDimensionedNameString();
    char hex[32];
    std::snprintf(hex, sizeof(hex), "%016llx",
                  static_cast<unsigned long long>(hashString(dimName + "/operator-mfma-components/" + str(opSub) + (shape.allRows > 0 ? "@" + str(row0) : std::string()) + "/" +
                                                             (Positional() ? "p" : "u") + "c" + str(C))));
    plan.module_name = std::string("acro_op_") + hex;
    std::ostringstream sched;
    sched << "operator schedule on the FP64 matrix cores: ";
    if (shape.allRows > 0) sched << "rows " << row0 << " - " << row0 + nI - 1 << " of the " << nAll << " x " << nJ << (shape.transposed ? " operator (stored transposed)" : (shape.mixed ? " operator (dimensions in another order)" : " operator"));
    else sched << nI << " x " << nJ << (shape.transposed ? " operator (stored transposed)" : (shape.mixed ? " operator (dimensions in another order)" : " operator"));
    sched << " in LDS in operand order";
    if (nIp != nI || nJp != nJ) sched << " (padded to " << nIp << " x " << nJp << ")";
    sched << ", " << C << " components per vector element";
    if (stageRounds > 0) sched << ", results written out through LDS";
    sched << ", " << NE << " entries, 16 per wavefront and trip, " << tilesN * steps * C << " v_mfma_f64_16x16x4 per trip, " << blocks
          << " workgroups of 256 lanes\n  [" << opSub << "] " << s.text << "\n";
    plan.schedule = sched.str();
    if (first) out << "// Generated by the acrotensor HIP code generator for gfx950.\n";
    {
        std::istringstream lines(plan.schedule);
        std::string l;
        while (std::getline(lines, l)) out << "// " << l << "\n";
    }
    const std::string B = PtrName(opr.uvar), X = PtrName(x.uvar), A = PtrName(s.out.uvar);
    const bool streams = s.op == '=' && envInt("ACRO_HIP_NT_STORE") >= 0;
    out << (first ? "" : "\n") << "typedef double acro_double4 __attribute__((ext_vector_type(4)));\n";
    out << "\nextern \"C\" __global__ __launch_bounds__(256) void " << plan.module_name << "(" << ParamList() << ")\n{\n";
    out << "    __shared__ double frag[" << nIp * nJp << "];\n";
    FillLoopHead(out, nIp * nJp);
    out << "        const int l = f & 63, step = (f >> 6) % " << steps << ", t = (f >> 6) / " << steps << ";\n";
    out << "        const int row = 16 * t + (l & 15), j = 4 * step + (l >> 4);\n";
    const std::string rowHere = row0 > 0 ? "(row + " + str(row0) + ")" : std::string("row");
    const std::string element = B + "[" + Lit(uvars[opr.uvar].viewOffset) + " + " + OperatorEntry(shape, rowHere, "j", nAll) + "]";
    if (nIp != nI || nJp != nJ)
        out << "        frag[f] = row < " << nI << " && j < " << nJ << " ? " << element << " : 0.0;\n    }\n";
    else
        out << "        frag[f] = " << element << ";\n    }\n";
    const int perRound = stageRounds > 0 ? 4 / stageRounds : 0;   // result registers (entries g + 4 r) per round
    if (stageRounds > 0) out << "    __shared__ double stage[" << 4 * 4 * perRound * nI * C << "];\n";
    out << "    __syncthreads();\n";
    out << "    const int lane = threadIdx.x & 63, g = lane >> 4, c = lane & 15;\n";
    out << "    const long waves = (long)gridDim.x * 4;\n";
    out << "    for (long tile = (long)blockIdx.x * 4 + (threadIdx.x >> 6); tile < " << tiles << "; tile += waves)\n    {\n";
    // (a kernel that the compiler can only fit into the registers with spills is compiled again with this macro:
    // the operator's values are then read from LDS on every trip instead of being kept in registers across trips)
    out << "#ifdef ACRO_KEEP_OPERATOR_IN_LDS\n        __asm__ volatile(\"\" ::: \"memory\");\n#endif\n";
    if (ragged)
        out << "        const long ex = tile * 16 + c < " << NE << " ? tile * 16 + c : " << NE - 1 << ";  // past the end: any valid entry, never stored\n";
    else
        out << "        const long ex = tile * 16 + c;\n";
    out << "        const double *x = " << X << " + " << Lit(uvars[x.uvar].viewOffset) << " + ex * " << nJ * C << " + g * " << C << ";\n";
    out << "        double xv[" << C << "][" << steps << "];\n";
    out << "#pragma unroll\n        for (int q = 0; q < " << steps << "; ++q)\n";
    out << "#pragma unroll\n            for (int k = 0; k < " << C << "; ++k) xv[k][q] = ";
    if (nJp != nJ) out << "4 * q + g >= " << nJ << " ? 0.0 : ";
    out << "x[" << 4 * C << " * q + k];\n";
    out << "        acro_double4 acc[" << C << "][" << tilesN << "];\n";
    out << "#pragma unroll\n        for (int k = 0; k < " << C << "; ++k)\n";
    out << "#pragma unroll\n            for (int t = 0; t < " << tilesN << "; ++t) acc[k][t] = acro_double4{0.0, 0.0, 0.0, 0.0};\n";
    out << "#pragma unroll\n        for (int step = 0; step < " << steps << "; ++step)\n";
    out << "#pragma unroll\n            for (int t = 0; t < " << tilesN << "; ++t)\n            {\n";
    out << "                const double b = frag[(t * " << steps << " + step) * 64 + lane];\n";
    out << "#pragma unroll\n                for (int k = 0; k < " << C << "; ++k) acc[k][t] = __builtin_amdgcn_mfma_f64_16x16x4f64(xv[k][step], b, acc[k][t], 0, 0, 0);\n";
    out << "            }\n";
    // register r of a lane holds entry 4 r + g of the trip and row 16 t + c
    const long rowsC = nI * C, strideC = nAll * C;
    const std::string rowGuard = nIp != nI ? "if (16 * t + c < " + str(nI) + ") " : std::string();
    // components between the result's row indices: where row `row` and component k of an entry lie
    auto mixedOffset = [&](const std::string &row) {
        std::string at;
        auto add = [&](const std::string &flat, const std::vector<OperatorShape::Term> &terms) {
            for (const auto &term : terms)
            {
                const std::string v = term.div == 1 ? flat : "(" + flat + " / " + str(term.div) + ")";
                at += (at.empty() ? "" : " + ") + ("(" + v + " % " + str(term.ext) + ")") + " * " + str(term.stride);
            }
        };
        add(row, shape.outRowTerms);
        add("k", shape.outCompTerms);
        return at;
    };
    if (stageRounds > 0)
    {
        out << "        double *mid = stage + (threadIdx.x >> 6) * " << 4 * perRound * rowsC << ";\n";
        for (int h = 0; h < stageRounds; ++h)
        {
            out << "#pragma unroll\n        for (int r = " << h * perRound << "; r < " << (h + 1) * perRound << "; ++r)\n";
            out << "#pragma unroll\n            for (int t = 0; t < " << tilesN << "; ++t)\n";
            out << "#pragma unroll\n                for (int k = 0; k < " << C << "; ++k)\n";
            const std::string inEntry = shape.outMixed ? mixedOffset("(16 * t + c)") : "(16 * t + c) * " + str(C) + " + k";
            out << "                    " << rowGuard << "mid[(4 * " << (h ? "(r - " + str(static_cast<long>(h * perRound)) + ")" : std::string("r")) << " + g) * " << rowsC
                << " + " << inEntry << "] = acc[k][t][r];\n";
            out << "        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, \"wavefront\");\n        __builtin_amdgcn_wave_barrier();\n";
            out << "        {\n";
            const long firstEntry = 4L * h * perRound, entries = 4L * perRound;
            out << "            double *a = " << A << " + " << Lit(uvars[s.out.uvar].viewOffset) << " + (tile * 16 + " << firstEntry << ") * " << rowsC << ";\n";
            if (ragged)
                out << "            const long left = " << NE << " - tile * 16 - " << firstEntry << ";\n"
                    << "            const int count = (int)(left < 0 ? 0 : (left < " << entries << " ? left : " << entries << ")) * " << rowsC << ";\n";
            else
                out << "            const int count = " << entries * rowsC << ";\n";
            out << "            for (int i = lane; i < count; i += 64)\n";
            if (streams)
                out << "                __builtin_nontemporal_store(mid[i], a + i);\n";
            else
                out << "                a[i]" << (s.op == '=' ? " = " : (s.op == '+' ? " += " : " -= ")) << "mid[i];\n";
            out << "        }\n";
            out << "        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, \"wavefront\");\n        __builtin_amdgcn_wave_barrier();\n";
        }
    }
    else
    {
        out << "#pragma unroll\n        for (int r = 0; r < 4; ++r)\n        {\n";
        if (ragged) out << "            if (tile * 16 + g + 4 * r >= " << NE << ") continue;\n";
        out << "            double *a = " << A << " + " << Lit(uvars[s.out.uvar].viewOffset) << " + (tile * 16 + g + 4 * r) * " << strideC;
        if (!shape.outMixed) out << " + " << row0 * C << " + c * " << C;
        out << ";\n";
        out << "#pragma unroll\n            for (int t = 0; t < " << tilesN << "; ++t)\n";
        out << "#pragma unroll\n                for (int k = 0; k < " << C << "; ++k)\n";
        const std::string where = shape.outMixed ? mixedOffset("(16 * t + c" + (row0 > 0 ? " + " + str(row0) : std::string()) + ")") : str(16 * C) + " * t + k";
        out << "                    " << rowGuard << "a[" << where << "]" << (s.op == '=' ? " = " : (s.op == '+' ? " += " : " -= ")) << "acc[k][t][r];\n";
        out << "        }\n";
    }
    out << "    }\n}\n";

    plan.source = out.str();
    plan.nb = 64;
    plan.lds_bytes = static_cast<int>((nIp * nJp + (stageRounds > 0 ? 4 * 4 * perRound * rowsC : 0)) * 8);
    FillParams(plan, false);
    HipLaunch launch;
    launch.function_name = plan.module_name;
    launch.grid = static_cast<unsigned>(blocks);
    launch.block = 256;
    for (int si = 0; si < NumParamStores(); ++si) launch.params.push_back(si);
    plan.launches.push_back(launch);
}

// The same with the entries as the fastest dimension ("A_i_e = B_i_j X_j_e"): the roles of the instruction's operands
// are exchanged.  The operator is the first operand (16 rows x 4 terms per instruction, from LDS in operand order),
// the entries' vectors the second: lane = entry + 16 * term group reads X[j][e], 16 consecutive entries per term, and
// result register r of a lane holds row 4r + lane / 16 of its entry, so loads and stores run along the entries.
// With an even number of entries a wavefront takes 32 entries per trip: a lane loads two neighbouring entries in
// 16 bytes, which feed two accumulator sets (even and odd entries), and stores its two results together.
auto Generator::EmitOperatorEntriesFastest(HipKernelPlan &plan, const OperatorShape &shape) -> void
{
    const Sub &s = OpKernel(opSub);
    const VarRef &opr = *shape.op, &x = *shape.x;
    const long nI = shape.rows, nJ = shape.cols, E = shape.entries;
    const bool pairs = shape.pairs;
    const int per = pairs ? 32 : 16;
    const long nIp = (nI + 15) / 16 * 16, nJp = (nJ + 3) / 4 * 4;
    const long tilesM = nIp / 16, steps = nJp / 4;
    const long trips = (E + per - 1) / per;
    const bool ragged = E % per != 0;
    const long blocks = std::max<long>(1, std::min<long>(512, (trips + 3) / 4));
    for (const auto &st : stores)
    {
        long entries = 1;
        for (int d : st.dims) entries *= d;
        if (entries >= (1L << 31) - 1) wide = true;
    }
    const std::string dimName = mk.GetDimensionedNameString();
    char hex[32];
    std::snprintf(hex, sizeof(hex), "%016llx",
                  static_cast<unsigned long long>(hashString(dimName + "/operator-mfma-t/" + str(opSub) + "/" + (Positional() ? "p" : "u") + (pairs ? "2" : "1"))));
    plan.module_name = std::string("acro_op_") + hex;
    std::ostringstream sched;
    sched << "operator schedule on the FP64 matrix cores, entries fastest: " << nI << " x " << nJ
          << (shape.transposed ? " operator (stored transposed)" : (shape.mixed ? " operator (dimensions in another order)" : " operator")) << " in LDS in operand order";
    if (nIp != nI || nJp != nJ) sched << " (padded to " << nIp << " x " << nJp << ")";
    sched << ", " << E << " entries, " << per << " per wavefront and trip, " << tilesM * steps * (pairs ? 2 : 1)
          << " v_mfma_f64_16x16x4 per trip, " << blocks << " workgroups of 256 lanes\n  [" << opSub << "] " << s.text << "\n";
    plan.schedule = sched.str();

    if (opSub == 0) out << "// Generated by the acrotensor HIP code generator for gfx950.\n";
    {
        std::istringstream lines(plan.schedule);
        std::string l;
        while (std::getline(lines, l)) out << "// " << l << "\n";
    }
    const std::string B = PtrName(opr.uvar), X = PtrName(x.uvar), A = PtrName(s.out.uvar);
    const bool stream = s.op == '=' && envInt("ACRO_HIP_NT_STORE") >= 0;
    const std::string vt = pairs ? "acro_double2" : "double";
    auto offsetOf = [&](const VarRef &v) { return Lit(uvars[v.uvar].viewOffset); };
    out << (opSub == 0 ? "" : "\n") << "typedef double acro_double4 __attribute__((ext_vector_type(4)));\n";
    // only the 8-byte alignment that every operand has is promised (see acro_pair in the other operator kernel)
    out << "typedef double acro_double2 __attribute__((ext_vector_type(2), aligned(8)));\n";
    out << "\nextern \"C\" __global__ __launch_bounds__(256) void " << plan.module_name << "(" << ParamList() << ")\n{\n";
    out << "    __shared__ double frag[" << nIp * nJp << "];\n";
    FillLoopHead(out, nIp * nJp);
    out << "        const int l = f & 63, step = (f >> 6) % " << steps << ", t = (f >> 6) / " << steps << ";\n";
    out << "        const int row = 16 * t + (l & 15), j = 4 * step + (l >> 4);\n";
    const std::string element = B + "[" + offsetOf(opr) + " + " + OperatorEntry(shape, "row", "j", nI) + "]";
    if (nIp != nI || nJp != nJ)
        out << "        frag[f] = row < " << nI << " && j < " << nJ << " ? " << element << " : 0.0;\n    }\n";
    else
        out << "        frag[f] = " << element << ";\n    }\n";
    out << "    __syncthreads();\n";
    out << "    const int lane = threadIdx.x & 63, g = lane >> 4, c = lane & 15;\n";
    out << "    const long waves = (long)gridDim.x * 4;\n";
    out << "    for (long trip = (long)blockIdx.x * 4 + (threadIdx.x >> 6); trip < " << trips << "; trip += waves)\n    {\n";
    // (a kernel that the compiler can only fit into the registers with spills is compiled again with this macro:
    // the operator's values are then read from LDS on every trip instead of being kept in registers across trips)
    out << "#ifdef ACRO_KEEP_OPERATOR_IN_LDS\n        __asm__ volatile(\"\" ::: \"memory\");\n#endif\n";
    out << "        const long e = trip * " << per << " + " << (pairs ? "2 * c" : "c") << ";\n";
    if (ragged)
        out << "        const long ex = e < " << E << " ? e : " << E - (pairs ? 2 : 1) << ";  // past the end: any valid entry, never stored\n";
    else
        out << "        const long ex = e;\n";
    out << "        " << vt << " xv[" << steps << "];\n";
    out << "#pragma unroll\n";
    out << "        for (int step = 0; step < " << steps << "; ++step)\n        {\n";
    out << "            const int j = 4 * step + g;\n";
    if (nJp != nJ) out << "            if (j >= " << nJ << ") { xv[step] = " << (pairs ? "acro_double2{0.0, 0.0}" : "0.0") << "; continue; }\n";
    out << "            xv[step] = *reinterpret_cast<const " << vt << " *>(" << X << " + " << offsetOf(x) << " + j * " << E << " + ex);\n";
    for (const VarRef *w : shape.perElement)
        out << "            xv[step] *= *reinterpret_cast<const " << vt << " *>(" << PtrName(w->uvar) << " + " << offsetOf(*w) << " + j * " << E << " + ex);\n";
    for (const VarRef *w : shape.perColumn)
        out << "            xv[step] *= " << PtrName(w->uvar) << "[" << offsetOf(*w) << " + j];\n";
    out << "        }\n";
    out << "        acro_double4 acc0[" << tilesM << "]" << (pairs ? ", acc1[" + str(tilesM) + "]" : "") << ";\n";
    out << "#pragma unroll\n";
    out << "        for (int t = 0; t < " << tilesM << "; ++t) acc0[t] = " << (pairs ? "acc1[t] = " : "") << "acro_double4{0.0, 0.0, 0.0, 0.0};\n";
    out << "#pragma unroll\n";
    out << "        for (int step = 0; step < " << steps << "; ++step)\n        {\n";
    out << "#pragma unroll\n";
    out << "            for (int t = 0; t < " << tilesM << "; ++t)\n            {\n";
    out << "                const double b = frag[(t * " << steps << " + step) * 64 + lane];\n";
    if (pairs)
    {
        out << "                acc0[t] = __builtin_amdgcn_mfma_f64_16x16x4f64(b, xv[step].x, acc0[t], 0, 0, 0);\n";
        out << "                acc1[t] = __builtin_amdgcn_mfma_f64_16x16x4f64(b, xv[step].y, acc1[t], 0, 0, 0);\n";
    }
    else
        out << "                acc0[t] = __builtin_amdgcn_mfma_f64_16x16x4f64(b, xv[step], acc0[t], 0, 0, 0);\n";
    out << "            }\n        }\n";
    if (ragged) out << "        if (e >= " << E << ") continue;\n";
    if (!shape.perEntry.empty())
    {
        out << "        const " << vt << " se = ";
        for (size_t i = 0; i < shape.perEntry.size(); ++i)
            out << (i ? " * " : "") << "*reinterpret_cast<const " << vt << " *>(" << PtrName(shape.perEntry[i]->uvar) << " + " << offsetOf(*shape.perEntry[i]) << " + e)";
        out << ";\n";
    }
    out << "#pragma unroll\n";
    out << "        for (int t = 0; t < " << tilesM << "; ++t)\n";
    out << "#pragma unroll\n";
    out << "            for (int r = 0; r < 4; ++r)\n            {\n";
    out << "                const int i = 16 * t + 4 * r + g;\n";
    if (nIp != nI) out << "                if (i >= " << nI << ") continue;\n";
    out << "                " << vt << " v = " << (pairs ? "acro_double2{acc0[t][r], acc1[t][r]}" : "acc0[t][r]") << ";\n";
    if (!shape.perEntry.empty()) out << "                v *= se;\n";
    for (const VarRef *w : shape.perOutput)
        out << "                v *= *reinterpret_cast<const " << vt << " *>(" << PtrName(w->uvar) << " + " << offsetOf(*w) << " + i * " << E << " + e);\n";
    for (const VarRef *w : shape.perRow)
        out << "                v *= " << PtrName(w->uvar) << "[" << offsetOf(*w) << " + i];\n";
    out << "                " << vt << " *a = reinterpret_cast<" << vt << " *>(" << A << " + " << offsetOf(s.out) << " + i * " << E << " + e);\n";
    if (stream)
        out << "                __builtin_nontemporal_store(v, a);\n";
    else
        out << "                *a " << (s.op == '=' ? "= " : (s.op == '+' ? "+= " : "-= ")) << "v;\n";
    out << "            }\n    }\n}\n";

    plan.source = out.str();
    plan.nb = 64;
    plan.lds_bytes = static_cast<int>(nIp * nJp * 8);
    FillParams(plan, false);
    HipLaunch launch;
    launch.function_name = plan.module_name;
    launch.grid = static_cast<unsigned>(blocks);
    launch.block = 256;
    for (int si = 0; si < NumParamStores(); ++si) launch.params.push_back(si);
    plan.launches.push_back(launch);
}

}  // namespace codegen
}  // namespace acro
