// fp32 storage on the fp32 MFMA: launchers for one padded (DI, DJ) pair.
#include "cott_mfma_launch.inc"
#include "cott_mfma_f32.h"
#include "cott_split.h"

namespace cott {
namespace {

// Padded head dims 64 x 64: the products run on the bf16 matrix cores from split operands (cott_split.h).
template <int DI, int DJ>
hipError_t run_causal_split(const SetArgs &a) {
    using TL = Tiling<DI, DJ>;
    constexpr int PF = 2;
    const ProblemSetF ps = make_set<float, DI, DJ>(a);
    if (a.G > 1) {
        if (ps.nact > 0) {
            ProfScope prof(K_GROUP_STATE, a.stream);
            group_state_split_kernel<DI, DJ, PF><<<dim3(grid_for(a.BH, ps.nact * a.sub, a.G - 1, a.xcds)), dim3(kThreads), 0, a.stream>>>(
                ps, a.BH, a.N, a.nchunks, a.cpg, a.G, a.G - 1);
        }
        const int bps = (TL::STATE_FLOATS / 4 + kThreads - 1) / kThreads;
        ProfScope prof(K_STATE_PREFIX, a.stream);
        state_prefix_kernel<float><<<dim3((unsigned)(a.BH * ps.count * bps)), dim3(kThreads), 0, a.stream>>>(
            ps, a.BH, a.G, a.sub, a.G - 1, TL::STATE_FLOATS, 0);
    }
    ProfScope prof(a.scan_prof_id, a.stream);
    split_scan_kernel<DI, DJ, PF><<<dim3(grid_for(a.BH, a.count, a.G, a.xcds)), dim3(512), 0, a.stream>>>(
        ps, a.BH, a.N, a.nchunks, a.cpg, a.G);
    return hipGetLastError();
}

template <int DI, int DJ>
hipError_t run_causal_f32(const SetArgs &a) {
    if constexpr (DI == 64 && DJ == 64) {
        static const int split = exp_env("COTT_F32_SPLIT", 1);
        if (split) return run_causal_split<DI, DJ>(a);
    }
    using TL = TilingF32<DI, DJ>;
    const ProblemSetF32 ps = make_set<float, DI, DJ>(a);
    if (a.G > 1) {
        {
            ProfScope prof(K_GROUP_STATE, a.stream);
            group_state_f32_kernel<DI, DJ><<<dim3(grid_for(a.BH, a.count, a.G, a.xcds)), dim3(kThreads), 0, a.stream>>>(
                ps, a.BH, a.N, a.nchunks, a.cpg, a.G, a.G - 1);
        }
        const int bps = (TL::STATE_FLOATS / 4 + kThreads - 1) / kThreads;
        ProfScope prof(K_STATE_PREFIX, a.stream);
        state_prefix_kernel<float><<<dim3((unsigned)(a.BH * a.count * bps)), dim3(kThreads), 0, a.stream>>>(
            ps, a.BH, a.G, 1, a.G - 1, TL::STATE_FLOATS, 0);
    }
    ProfScope prof(a.scan_prof_id, a.stream);
    scan_f32_kernel<DI, DJ, false><<<dim3(grid_for(a.BH, a.count, a.G, a.xcds)), dim3(kThreads), 0, a.stream>>>(
        ps, a.BH, a.N, a.nchunks, a.cpg, a.G);
    return hipGetLastError();
}

// Non-causal: per-group sums of B^T C, their total, then out = A S.  Always through the workspace.
template <int DI, int DJ>
hipError_t run_noncausal_f32(const SetArgs &a) {
    using TL = TilingF32<DI, DJ>;
    const ProblemSetF32 ps = make_set<float, DI, DJ>(a);
    {
        ProfScope prof(K_GROUP_STATE, a.stream);
        group_state_f32_kernel<DI, DJ><<<dim3(grid_for(a.BH, a.count, a.G, a.xcds)), dim3(kThreads), 0, a.stream>>>(
            ps, a.BH, a.N, a.nchunks, a.cpg, a.G, a.G);
    }
    if (a.G > 1) {
        const int bps = (TL::STATE_FLOATS / 4 + kThreads - 1) / kThreads;
        ProfScope prof(K_STATE_PREFIX, a.stream);
        state_prefix_kernel<float><<<dim3((unsigned)(a.BH * a.count * bps)), dim3(kThreads), 0, a.stream>>>(
            ps, a.BH, a.G, 1, a.G, TL::STATE_FLOATS, 1);
    }
    ProfScope prof(K_APPLY, a.stream);
    scan_f32_kernel<DI, DJ, true><<<dim3(grid_for(a.BH, a.count, a.G, a.xcds)), dim3(kThreads), 0, a.stream>>>(
        ps, a.BH, a.N, a.nchunks, a.cpg, a.G);
    return hipGetLastError();
}

template <bool CAUSAL>
hipError_t dispatch_f32(const SetArgs &a) {
    if (a.count < 1 || a.count > kMaxProblems) return hipErrorInvalidValue;
    const int pi = mfma_pad(a.op[0].di), pj = mfma_pad(a.op[0].dj);
    for (int i = 1; i < a.count; ++i)
        if (mfma_pad(a.op[i].di) != pi || mfma_pad(a.op[i].dj) != pj) return hipErrorInvalidValue;
#define COTT_CASE(DI, DJ) \
    if (pi == DI && pj == DJ) return CAUSAL ? run_causal_f32<DI, DJ>(a) : run_noncausal_f32<DI, DJ>(a);
    COTT_CASE(32, 32) COTT_CASE(32, 64) COTT_CASE(32, 128)
    COTT_CASE(64, 32) COTT_CASE(64, 64) COTT_CASE(64, 128)
    COTT_CASE(128, 32) COTT_CASE(128, 64) COTT_CASE(128, 128)
#undef COTT_CASE
    return hipErrorInvalidValue;
}

}  // namespace

hipError_t launch_causal_mfma_f32(const SetArgs &a) { return dispatch_f32<true>(a); }
hipError_t launch_noncausal_mfma_f32(const SetArgs &a) { return dispatch_f32<false>(a); }

}  // namespace cott
