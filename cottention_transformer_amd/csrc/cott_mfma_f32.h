// Chunked-scan kernels for fp32 storage on the fp32 MFMA (v_mfma_f32_16x16x4_f32): same recurrence
// and the same launch structure (problem sets, sequence groups, register-native state slots) as
// the 16-bit kernels, with every product and the state carried in fp32.
//
// v_mfma_f32_16x16x4_f32: D(16x16) += A(16x4) B(4x16); lane l (m = l%16, g = l/16) supplies A[m][g]
// and B[g][m] and holds D[4g..4g+3][m].  The contraction index of a product may be enumerated in
// any order as long as both operands use the same one, which is used twice below:
//   * a row-major LDS tile X[row][i] gives, with ONE 16-byte read per lane at X[16b+m][16it+4g..+3],
//     the operands of four MFMAs contracting i = 16it+4g+r (r = 0..3);
//   * with that order the state accumulators S[i=16it+4g+r][j=16jt+m] ARE the B operands of A S.
#pragma once
#include "cott_mfma.h"

namespace cott {

typedef ProblemT<float> ProblemF32;
typedef ProblemSetT<float> ProblemSetF32;

template <int DI, int DJ>
struct TilingF32 {
    static_assert(DI % 32 == 0 && DJ % 32 == 0, "padded head dims are multiples of 32");
    static constexpr int CH = (DI + DJ > 128) ? 32 : 64;  // positions per step (LDS budget)
    static constexpr int SUB = kChunk / CH;               // steps per 64-position chunk
    static constexpr int NB = CH / 16;                    // 16-position blocks per step
    // Row strides in dwords.  8 (mod 32): the 16-byte row reads (lane m -> row, g -> 4 dwords) and the
    // column reads (lane g -> row, m -> dword) both spread evenly over the 32 banks.
    static constexpr int AS = DI + 8;   // A and B tiles [CH][DI]
    static constexpr int CS = DJ + 8;   // C tile [CH][DJ]
    static constexpr int PS = CH + 4;   // masked scores [CH][CH] (4 mod 32 for its 16-byte row reads + dword writes)
    static constexpr int NIT = DI / 16, NJT = DJ / 16;
    static constexpr int JPW = (NJT + 3) / 4;             // column tiles per wavefront: jt = w + 4*js
    static constexpr int NTRI = NB * (NB + 1) / 2;        // score tiles on or below the diagonal
    static constexpr int STATE_FLOATS = DI * DJ;
    static constexpr int VA = CH * DI / 4 / kThreads;     // 16-byte vectors per thread, A or B tile
    static constexpr int VC = CH * DJ / 4 / kThreads;     // ... C tile
    static_assert(VA >= 1 && VC >= 1, "tiles divide over the workgroup");
};

// Per-wavefront registers: the state columns it owns and the C operands of the current step.
template <int DI, int DJ>
struct StateF32 {
    f32x4 v[TilingF32<DI, DJ>::JPW][TilingF32<DI, DJ>::NIT];
};
template <int DI, int DJ>
struct CFragsF32 {
    float v[TilingF32<DI, DJ>::JPW][TilingF32<DI, DJ>::NB][4];
};

__device__ __forceinline__ f32x4 mfma_f32(float a, float b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ void buf_store4(rsrc_t r, uint32_t byte_off, float v) {
    __builtin_amdgcn_raw_buffer_store_b32(bitcast<uint32_t>(v), r, (int)byte_off, 0, 0);
}

// [CH][D] fp32 tile, global -> registers (rows past the end of the head read as zero).
template <int CH, int D>
__device__ __forceinline__ void load_tile_f32(u32x4 *r, rsrc_t rs, int row0, int ld, int tid) {
#pragma unroll
    for (int u = 0; u < CH * D / 4 / kThreads; ++u) {
        const int v = tid + kThreads * u;
        r[u] = buf_load16(rs, (uint32_t)((row0 + v / (D / 4)) * ld + (v % (D / 4)) * 4) * 4u);
    }
}
// registers -> LDS tile with row stride STRIDE dwords; columns past the runtime width d become zero.
template <int CH, int D, int STRIDE>
__device__ __forceinline__ void store_tile_f32(float *tile, const u32x4 *r, int d, int tid) {
#pragma unroll
    for (int u = 0; u < CH * D / 4 / kThreads; ++u) {
        const int v = tid + kThreads * u;
        const int col = (v % (D / 4)) * 4;
        *reinterpret_cast<u32x4 *>(tile + (v / (D / 4)) * STRIDE + col) = (col < d) ? r[u] : u32x4{0u, 0u, 0u, 0u};
    }
}

// Wavefront w owns the state columns jt = w + 4*js and keeps S.v[js][it] = S[16it+4g+r][16jt+m] in
// accumulators.  cf.v[js][tb][r] = C[16tb+4r+g][16jt+m] are the C operands of both the score product
// and the state update (contraction index t = 16tb+4r+g: lanes g walk consecutive rows).
template <int DI, int DJ>
__device__ __forceinline__ void load_c_frags(CFragsF32<DI, DJ> &cf, const float *sC, int w, int g, int m) {
    using TL = TilingF32<DI, DJ>;
#pragma unroll
    for (int js = 0; js < TL::JPW; ++js) {
        const int jt = w + 4 * js;
        if (jt < TL::NJT) {
#pragma unroll
            for (int tb = 0; tb < TL::NB; ++tb)
#pragma unroll
                for (int r = 0; r < 4; ++r) cf.v[js][tb][r] = sC[(16 * tb + 4 * r + g) * TL::CS + 16 * jt + m];
        }
    }
}

// S.v[js][it] += B^T C over the CH positions of the step.
template <int DI, int DJ>
__device__ __forceinline__ void state_update_f32(StateF32<DI, DJ> &S, const CFragsF32<DI, DJ> &cf, const float *sB,
                                                 int w, int g, int m) {
    using TL = TilingF32<DI, DJ>;
#pragma unroll
    for (int tb = 0; tb < TL::NB; ++tb)
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int it = 0; it < TL::NIT; ++it) {
                const float b = sB[(16 * tb + 4 * r + g) * TL::AS + 16 * it + m];
#pragma unroll
                for (int js = 0; js < TL::JPW; ++js)
                    if (w + 4 * js < TL::NJT) S.v[js][it] = mfma_f32(b, cf.v[js][tb][r], S.v[js][it]);
            }
}

// State slot order (float4 units): ((w + 4*js) * NIT + it) * 64 + lane.
template <int DI, int DJ>
__device__ __forceinline__ void read_state_f32(StateF32<DI, DJ> &S, const float *slot, int w, int l) {
    using TL = TilingF32<DI, DJ>;
    const f32x4 *p = reinterpret_cast<const f32x4 *>(slot);
#pragma unroll
    for (int js = 0; js < TL::JPW; ++js)
        if (w + 4 * js < TL::NJT) {
#pragma unroll
            for (int it = 0; it < TL::NIT; ++it) S.v[js][it] = p[((w + 4 * js) * TL::NIT + it) * 64 + l];
        }
}
template <int DI, int DJ>
__device__ __forceinline__ void write_state_f32(const StateF32<DI, DJ> &S, float *slot, int w, int l) {
    using TL = TilingF32<DI, DJ>;
    f32x4 *p = reinterpret_cast<f32x4 *>(slot);
#pragma unroll
    for (int js = 0; js < TL::JPW; ++js)
        if (w + 4 * js < TL::NJT) {
#pragma unroll
            for (int it = 0; it < TL::NIT; ++it) p[((w + 4 * js) * TL::NIT + it) * 64 + l] = S.v[js][it];
        }
}

// Sum of B^T C over each group of chunks (scan order), into slot (bh*G + grp).
template <int DI, int DJ>
__global__ __launch_bounds__(kThreads) void group_state_f32_kernel(ProblemSetF32 set, int BH, int N, int nchunks,
                                                                   int cpg, int G, int ngroups) {
    using TL = TilingF32<DI, DJ>;
    constexpr int CH = TL::CH;
    __shared__ __attribute__((aligned(16))) float sB[CH * TL::AS];
    __shared__ __attribute__((aligned(16))) float sC[CH * TL::CS];
    const int tid = threadIdx.x, l = tid & 63, g = l >> 4, m = l & 15;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const WorkItem wi = decode_workgroup(set.count, BH, set.xcds);  // the (head, group) -> XCD map of the scan
    if (wi.grp >= ngroups) return;
    const ProblemF32 &pr = set.p[wi.prob];
    const int di = pr.di, dj = pr.dj, ldc = pr.ldc, reversed = pr.reversed;
    const rsrc_t rB = make_rsrc(pr.B + (size_t)wi.bh * N * di, (uint32_t)N * di * 4u);
    const rsrc_t rC = make_rsrc(pr.C + (size_t)wi.bh * N * ldc, ((uint32_t)(N - 1) * ldc + dj) * 4u);
    const int nsteps = nchunks * TL::SUB;
    const int p0 = wi.grp * cpg * TL::SUB;
    const int p1 = min((wi.grp + 1) * cpg, nchunks) * TL::SUB;

    StateF32<DI, DJ> S;
#pragma unroll
    for (int js = 0; js < TL::JPW; ++js)
#pragma unroll
        for (int it = 0; it < TL::NIT; ++it) S.v[js][it] = f32x4{0.f, 0.f, 0.f, 0.f};
    u32x4 rb[TL::VA], rc[TL::VC];
    auto load_step = [&](int p) {
        const int pc = min(p, p1 - 1);
        const int row0 = (reversed ? nsteps - 1 - pc : pc) * CH;
        load_tile_f32<CH, DI>(rb, rB, row0, di, tid);
        load_tile_f32<CH, DJ>(rc, rC, row0, ldc, tid);
    };
    load_step(p0);
    for (int p = p0; p < p1; ++p) {
        store_tile_f32<CH, DI, TL::AS>(sB, rb, di, tid);
        store_tile_f32<CH, DJ, TL::CS>(sC, rc, dj, tid);
        __syncthreads();
        load_step(p + 1);
        CFragsF32<DI, DJ> cf;
        load_c_frags<DI, DJ>(cf, sC, w, g, m);
        state_update_f32<DI, DJ>(S, cf, sB, w, g, m);
        __syncthreads();
    }
    write_state_f32<DI, DJ>(S, pr.gstate + ((size_t)wi.bh * G + wi.grp) * TL::STATE_FLOATS, w, l);
}

// The recurrence for one group of one head of one problem.  APPLY = true: out = A S only, with S
// the total of slot 0 of the head (second pass of the non-causal form).
//
// Per step of CH positions: (1) the score tiles on or below the diagonal, P^T = B_tb A_rb^T, are
// shared out over the four wavefronts, masked, and written to LDS with their 4x4 position blocks
// transposed, so that a 16-byte row read returns the contraction order of the C fragments;
// (2) each wavefront forms out[:, its columns] = P C + A S for every position block and stores it;
// (3) it then adds B^T C to its state columns.
template <int DI, int DJ, bool APPLY>
__global__ __launch_bounds__(kThreads) void scan_f32_kernel(ProblemSetF32 set, int BH, int N, int nchunks, int cpg,
                                                            int G) {
    using TL = TilingF32<DI, DJ>;
    constexpr int CH = TL::CH, NB = TL::NB;
    __shared__ __attribute__((aligned(16))) float sA[CH * TL::AS];
    __shared__ __attribute__((aligned(16))) float sB[APPLY ? 4 : CH * TL::AS];
    __shared__ __attribute__((aligned(16))) float sC[APPLY ? 4 : CH * TL::CS];
    __shared__ __attribute__((aligned(16))) float sP[APPLY ? 4 : CH * TL::PS];
    const int tid = threadIdx.x, l = tid & 63, g = l >> 4, m = l & 15;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const WorkItem wi = decode_workgroup(set.count, BH, set.xcds);
    if (wi.grp >= G) return;
    const ProblemF32 &pr = set.p[wi.prob];
    const int di = pr.di, dj = pr.dj, ldc = pr.ldc, reversed = APPLY ? 0 : pr.reversed;
    const rsrc_t rA = make_rsrc(pr.A + (size_t)wi.bh * N * di, (uint32_t)N * di * 4u);
    const rsrc_t rB = make_rsrc(pr.B + (size_t)wi.bh * N * di, (uint32_t)N * di * 4u);
    const rsrc_t rC = make_rsrc(pr.C + (size_t)wi.bh * N * ldc, ((uint32_t)(N - 1) * ldc + dj) * 4u);
    const rsrc_t rO = make_rsrc(pr.O + (size_t)wi.bh * N * ldc, ((uint32_t)(N - 1) * ldc + dj) * 4u);
    const int nsteps = nchunks * TL::SUB;
    const int p0 = wi.grp * cpg * TL::SUB;
    const int p1 = min((wi.grp + 1) * cpg, nchunks) * TL::SUB;

    StateF32<DI, DJ> S;
#pragma unroll
    for (int js = 0; js < TL::JPW; ++js)
#pragma unroll
        for (int it = 0; it < TL::NIT; ++it) S.v[js][it] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (APPLY)
        read_state_f32<DI, DJ>(S, pr.gstate + (size_t)wi.bh * G * TL::STATE_FLOATS, w, l);
    else if (pr.gstate != nullptr)
        read_state_f32<DI, DJ>(S, pr.gstate + ((size_t)wi.bh * G + wi.grp) * TL::STATE_FLOATS, w, l);
    if (!APPLY && pr.sin != nullptr) {
        const float *si = pr.sin + (size_t)wi.bh * di * pr.lds;
#pragma unroll
        for (int js = 0; js < TL::JPW; ++js)
            if (w + 4 * js < TL::NJT) {
                const int j = 16 * (w + 4 * js) + m;
#pragma unroll
                for (int it = 0; it < TL::NIT; ++it)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int i = 16 * it + 4 * g + r;
                        if (i < di && j < dj) S.v[js][it][r] += si[(size_t)i * pr.lds + j];
                    }
            }
    }

    u32x4 ra[TL::VA], rb[APPLY ? 1 : TL::VA], rc[APPLY ? 1 : TL::VC];
    auto load_step = [&](int p) {
        const int pc = min(p, p1 - 1);
        const int row0 = (reversed ? nsteps - 1 - pc : pc) * CH;
        load_tile_f32<CH, DI>(ra, rA, row0, di, tid);
        if (!APPLY) {
            load_tile_f32<CH, DI>(rb, rB, row0, di, tid);
            load_tile_f32<CH, DJ>(rc, rC, row0, ldc, tid);
        }
    };
    load_step(p0);
    for (int p = p0; p < p1; ++p) {
        const int row0 = (reversed ? nsteps - 1 - p : p) * CH;
        store_tile_f32<CH, DI, TL::AS>(sA, ra, di, tid);
        if (!APPLY) {
            store_tile_f32<CH, DI, TL::AS>(sB, rb, di, tid);
            store_tile_f32<CH, DJ, TL::CS>(sC, rc, dj, tid);
        }
        __syncthreads();
        load_step(p + 1);

        CFragsF32<DI, DJ> cf;
        if (!APPLY) {
            // (1) score tiles: canonical pair (x, y), y <= x; mirrored when the scan runs backwards
#pragma unroll
            for (int idx = 0; idx < TL::NTRI; ++idx) {
                if ((idx & 3) != w) continue;
                int x = 0;
                while ((x + 1) * (x + 2) / 2 <= idx) ++x;
                const int y = idx - x * (x + 1) / 2;
                const int rbk = reversed ? NB - 1 - x : x;  // position block (rows of P)
                const int tb = reversed ? NB - 1 - y : y;   // key block (columns of P)
                f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int it = 0; it < TL::NIT; ++it) {
                    const f32x4 bf = *reinterpret_cast<const f32x4 *>(sB + (16 * tb + m) * TL::AS + 16 * it + 4 * g);
                    const f32x4 af = *reinterpret_cast<const f32x4 *>(sA + (16 * rbk + m) * TL::AS + 16 * it + 4 * g);
#pragma unroll
                    for (int r = 0; r < 4; ++r) acc = mfma_f32(bf[r], af[r], acc);
                }
                // acc[r] = P[position 16*rbk + m][key 16*tb + 4g + r]
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const bool keep = (x != y) || (reversed ? (4 * g + r >= m) : (4 * g + r <= m));
                    sP[(16 * rbk + m) * TL::PS + 16 * tb + 4 * r + g] = keep ? acc[r] : 0.f;
                }
            }
            load_c_frags<DI, DJ>(cf, sC, w, g, m);
            __syncthreads();
        }
        // (2) outputs
#pragma unroll
        for (int rbk = 0; rbk < NB; ++rbk) {
            f32x4 o[TL::JPW];
#pragma unroll
            for (int js = 0; js < TL::JPW; ++js) o[js] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int it = 0; it < TL::NIT; ++it) {
                const f32x4 af = *reinterpret_cast<const f32x4 *>(sA + (16 * rbk + m) * TL::AS + 16 * it + 4 * g);
#pragma unroll
                for (int js = 0; js < TL::JPW; ++js)
                    if (w + 4 * js < TL::NJT) {
#pragma unroll
                        for (int r = 0; r < 4; ++r) o[js] = mfma_f32(af[r], S.v[js][it][r], o[js]);
                    }
            }
            if (!APPLY) {
#pragma unroll
                for (int tb = 0; tb < NB; ++tb) {
                    if (reversed ? (tb < rbk) : (tb > rbk)) continue;
                    const f32x4 pf = *reinterpret_cast<const f32x4 *>(sP + (16 * rbk + m) * TL::PS + 16 * tb + 4 * g);
#pragma unroll
                    for (int js = 0; js < TL::JPW; ++js)
                        if (w + 4 * js < TL::NJT) {
#pragma unroll
                            for (int r = 0; r < 4; ++r) o[js] = mfma_f32(pf[r], cf.v[js][tb][r], o[js]);
                        }
                }
            }
#pragma unroll
            for (int js = 0; js < TL::JPW; ++js) {
                const int col = 16 * (w + 4 * js) + m;
                if (w + 4 * js < TL::NJT) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int row = row0 + 16 * rbk + 4 * g + r;
                        buf_store4(rO, (col < dj) ? (uint32_t)(row * ldc + col) * 4u : kOobOffset, o[js][r]);
                    }
                }
            }
        }
        // (3) state
        if (!APPLY) state_update_f32<DI, DJ>(S, cf, sB, w, g, m);
        __syncthreads();
    }
    if (!APPLY && pr.sout != nullptr && wi.grp == G - 1) {
        float *so = pr.sout + (size_t)wi.bh * di * pr.lds;
#pragma unroll
        for (int js = 0; js < TL::JPW; ++js)
            if (w + 4 * js < TL::NJT) {
                const int j = 16 * (w + 4 * js) + m;
#pragma unroll
                for (int it = 0; it < TL::NIT; ++it)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int i = 16 * it + 4 * g + r;
                        if (i < di && j < dj) so[(size_t)i * pr.lds + j] = S.v[js][it][r];
                    }
            }
    }
}

}  // namespace cott
