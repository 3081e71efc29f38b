// Generator: DimensionedMultiKernel -> HIP C++ source (see hip_codegen.hpp for the schedule in words).
// The reference's generator (exec/CudaExecutor.cpp:111-702) maps one CUDA thread to one output entry and loops
// over the contraction reading shared memory twice per multiply-add; this one maps a lane to a pencil of outputs,
// keeps operands in registers / SGPRs and batches several elements per workgroup.
#include "hip_codegen_impl.hpp"

namespace acro
{
namespace codegen
{

auto Generator::Run() -> HipKernelPlan
{
    HipKernelPlan plan;
    BuildModel();
    std::string why;
    if (!CheckFusable(why))
    {
        plan.fusable = false;
        plan.why_not = why;
        return plan;
    }
    plan.fusable = true;
    if (UseGramSchedule())
    {
        EmitGram(plan);
        return plan;
    }
    if (UseReductionSchedule())
    {
        EmitReduction(plan);
        return plan;
    }
    if (UseTransposeSchedule())
    {
        EmitTranspose(plan);
        return plan;
    }
    if (UseProductSchedule())
    {
        EmitProduct(plan);
        return plan;
    }
    if (UseTiledProductSchedule())
    {
        // A shared factor of 4 097 to 8 192 entries with at most 96 columns still does better as an operator in LDS in
        // blocks of rows, where that schedule takes the kernel (tensors that exceed the memory-side cache, % of the HBM
        // peak, tiled product -> operator: 125 x 64 39.5 -> 45.5, 128 x 64 47 -> 51, 96 x 48 56 -> 65, 80 x 60 49.5 -> 56,
        // 72 x 72 41 -> 47.5; but 64 x 125 43 -> 41, 125 x 125 28 -> 20.5, 216 x 64 33 -> 34, 100 x 100 26.5 -> 24).
        TiledProductShape p;
        TiledProductPattern(subs[0], p);
        const long mid = envInt("ACRO_HIP_TILED_PRODUCT_OPERATOR_MID", 8192);
        if (!p.batched && std::min(p.M, p.N) * p.K <= mid && p.K <= 96 && UseOperatorSchedule())
        {
            EmitOperator(plan);
            return plan;
        }
        EmitTiledProduct(plan);
        return plan;
    }
    if (UseOperatorSchedule())
    {
        EmitOperator(plan);
        return plan;
    }
    ChooseTiles();
    PlanFusion();
    ChooseBatching();
    if (NB == 1 && batch >= 0 && opt.noalias)
    {
        // One batch entry per workgroup makes the batch index uniform across the workgroup: operands that
        // depend on it but on no lane index can then be read with scalar loads too.  Plan again under that
        // assumption and keep the result if it still puts one entry in a workgroup.
        batchUniform = true;
        for (auto &s : subs)
        {
            s.fusedWithPrev = false;
            s.forwardedIn.clear();
            s.forwardedOld = false;
            s.loopMode = false;
        }
        const double busyBefore = busyLanes;
        ChooseTiles();
        PlanFusion();
        ChooseBatching();
        // Scalar operands take their indices out of the lanes; a plan that leaves the wavefronts much emptier than
        // before costs more in issue slots than the scalar loads save (T1_e_q_j_k = B_q_i X_e_i_j_k with X scalar
        // has 6 busy lanes instead of 25: p=4 diffusion apply at 44.8 % of the HBM peak against 72.3 %).
        if (NB != 1 || busyLanes < 0.8 * busyBefore)
        {
            batchUniform = false;
            for (auto &s : subs)
            {
                s.fusedWithPrev = false;
                s.forwardedIn.clear();
                s.forwardedOld = false;
                s.loopMode = false;
            }
            ChooseTiles();
            PlanFusion();
            ChooseBatching();
        }
    }
    if (factorised)
    {
        for (const auto &st : stores)
        {
            // every read of a partial result must be served from registers or from its LDS tile
            if (uvars[st.members[0]].isVirtual && !st.elide) factorisationAbandoned = true;
        }
        if (factorisationAbandoned)
        {
            plan.fusable = false;
            plan.why_not = "intermediates of the factorised kernel do not fit on chip";
            return plan;
        }
    }
    if (UseReductionFallback())
    {
        EmitReduction(plan);
        return plan;
    }
    ChooseEntriesFastest();
    Emit(plan);
    return plan;
}

auto Generator::FirstOccurrence(int u) const -> std::pair<int, int>
{
    return Positional() ? std::make_pair(0, u - 1) : mk.GetFirstKiVariForUVari(u);
}

}  // namespace codegen

namespace
{

// Every launch of a module that contains a matrix-core instruction is named for the spill check at compile time.
HipKernelPlan withSpillGuard(HipKernelPlan plan)
{
    if (!plan.fusable || plan.source.find("__builtin_amdgcn_mfma") == std::string::npos) return plan;
    for (const HipLaunch &launch : plan.launches)
    {
        bool known = false;
        for (const std::string &name : plan.matrix_core_functions) known = known || name == launch.function_name;
        if (!known) plan.matrix_core_functions.push_back(launch.function_name);
    }
    if (plan.source.find("#ifdef ACRO_KEEP_OPERATOR_IN_LDS") != std::string::npos)
        plan.register_relief_macro = "ACRO_KEEP_OPERATOR_IN_LDS";
    return plan;
}

}  // namespace

HipKernelPlan GenerateHipKernel(const DimensionedMultiKernel &mk, const HipCodegenOptions &options)
{
    // Partial results of a reordered kernel may take up to 48 KB of LDS per batch entry; when the tiles that are
    // live together do not fit in a workgroup's 64 KB, plan again with tiles of half that size (any two fit), and
    // finally evaluate the kernel as written.
    for (long maxTile : {6144L, 3072L})
    {
        codegen::Generator g(mk, options, maxTile);
        HipKernelPlan plan = g.Run();
        if (!g.factorisationAbandoned) return withSpillGuard(std::move(plan));
    }
    codegen::Generator g(mk, options, 0);
    return withSpillGuard(g.Run());
}

}  // namespace acro
