// Chunked-scan kernels for 16-bit storage types (bf16 / fp16) on gfx950 MFMA.
//
// Generic op (per batch*head):  out[s,j] = sum_i A[s,i] * sum_{s' <= s (>= s if reversed)} B[s',i] C[s',j]
// restructured over chunks of 64 positions (scan order p, state S[i][j] carried in fp32):
//     out_c = ((A_c B_c^T) o mask) C_c + A_c S_c ;   S_{c+1} = S_c + B_c^T C_c
// The sequence of one head is cut into G groups of consecutive chunks so that B*H*G workgroups
// fill the chip: group_state_kernel sums B^T C over each group, state_prefix_kernel turns the
// per-group sums into exclusive prefixes, scan_kernel runs the chunk recurrence seeded with its
// group's prefix.  The same three kernels serve the forward pass and, with permuted operands,
// every gradient (dQ = G(dO,V,K), dK = G(V,dO,Q,rev), dV = G(K,Q,dO,rev)).
#pragma once
#include "cott_common.h"

namespace cott {

constexpr int kChunk = 64;     // positions per chunk
constexpr int kThreads = 256;  // 4 wavefronts per workgroup

template <int DI, int DJ>
struct Tiling {
    static_assert(DI % 32 == 0 && DJ % 32 == 0, "padded head dims are multiples of 32");
    static constexpr int BS = DI + 8;            // LDS row stride (elements) of a [64][DI] tile
    static constexpr int CS = DJ + 8;            // ... of a [64][DJ] tile
    static constexpr int SS = DI + 8;            // ... of the transposed 16-bit state [DJ][DI]
    static constexpr int NIT = DI / 16;          // 16-wide tiles along i
    static constexpr int NJT = DJ / 16;          // 16-wide tiles along j
    static constexpr int TPW = NIT * NJT / 4;    // fp32 state tiles owned by one wavefront
    static constexpr int KS = DI / 32;           // MFMA k-steps over i
    static constexpr int STATE_FLOATS = DI * DJ;
};

// [64][D] tile, global -> registers.  Thread t owns 16-byte vectors t, t+256, ...; rows past N
// and columns past the runtime width d read as zero, so padded positions add nothing to a state.
template <int D>
__device__ __forceinline__ void load_tile(u32x4 (&r)[D / 32], const u16 *head, int row0, int N, int d, int tid) {
#pragma unroll
    for (int u = 0; u < D / 32; ++u) {
        const int v = tid + kThreads * u;
        const int row = row0 + v / (D / 8);
        const int col = (v % (D / 8)) * 8;
        r[u] = ld_global16(head + (size_t)row * d + col, row < N && col < d);
    }
}

template <int D>
__device__ __forceinline__ void store_tile(u16 *tile, const u32x4 (&r)[D / 32], int tid) {
#pragma unroll
    for (int u = 0; u < D / 32; ++u) {
        const int v = tid + kThreads * u;
        *reinterpret_cast<u32x4 *>(tile + (v / (D / 8)) * (D + 8) + (v % (D / 8)) * 8) = r[u];
    }
}

// S[i][j] += sum_{tok<64} B[tok][i] * C[tok][j] for the tiles this wavefront owns
// (tile index t = w*TPW + u -> (t / NJT, t % NJT)).  Both operands are column fragments of the
// row-major LDS tiles, fetched with transposing reads.
template <class TR, int DI, int DJ>
__device__ __forceinline__ void state_update(f32x4 *S, const u16 *sB, const u16 *sC,
                                             int w, int g, int m) {
    using TL = Tiling<DI, DJ>;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
        const int k0 = 32 * kb + 8 * g;
        u32x4 a;
#pragma unroll
        for (int u = 0; u < TL::TPW; ++u) {
            const int t = w * TL::TPW + u;
            const int it = t / TL::NJT, jt = t % TL::NJT;
            if (u % TL::NJT == 0) a = cat(lds_col4(sB, TL::BS, k0, 16 * it, m), lds_col4(sB, TL::BS, k0 + 4, 16 * it, m));
            const u32x4 b = cat(lds_col4(sC, TL::CS, k0, 16 * jt, m), lds_col4(sC, TL::CS, k0 + 4, 16 * jt, m));
            S[u] = TR::mfma(a, b, S[u]);
        }
    }
}

// Sum of B^T C over each group of chunks, written in register-native order:
// float4 index (w*TPW + u)*64 + lane of slot (bh*G + grp).
template <class TR, int DI, int DJ>
__global__ __launch_bounds__(kThreads) void group_state_kernel(const u16 *__restrict__ B, const u16 *__restrict__ C,
                                                               float *__restrict__ gstate, int N, int di, int dj,
                                                               int nchunks, int cpg, int G, int ngroups,
                                                               int reversed) {
    using TL = Tiling<DI, DJ>;
    __shared__ __attribute__((aligned(16))) u16 sB[kChunk * TL::BS];
    __shared__ __attribute__((aligned(16))) u16 sC[kChunk * TL::CS];
    const int tid = threadIdx.x, w = tid >> 6, l = tid & 63, g = l >> 4, m = l & 15;
    const int grp = blockIdx.x % ngroups, bh = blockIdx.x / ngroups;  // G slots per head, `ngroups` launched
    B += (size_t)bh * N * di;
    C += (size_t)bh * N * dj;
    const int p0 = grp * cpg;
    const int p1 = min(p0 + cpg, nchunks);

    f32x4 S[TL::TPW];
#pragma unroll
    for (int u = 0; u < TL::TPW; ++u) S[u] = f32x4{0.f, 0.f, 0.f, 0.f};

    u32x4 rb[DI / 32], rc[DJ / 32];
    {
        const int c = reversed ? nchunks - 1 - p0 : p0;
        load_tile<DI>(rb, B, c * kChunk, N, di, tid);
        load_tile<DJ>(rc, C, c * kChunk, N, dj, tid);
    }
    for (int p = p0; p < p1; ++p) {
        __syncthreads();
        store_tile<DI>(sB, rb, tid);
        store_tile<DJ>(sC, rc, tid);
        __syncthreads();
        if (p + 1 < p1) {
            const int c = reversed ? nchunks - 2 - p : p + 1;
            load_tile<DI>(rb, B, c * kChunk, N, di, tid);
            load_tile<DJ>(rc, C, c * kChunk, N, dj, tid);
        }
        state_update<TR, DI, DJ>(S, sB, sC, w, g, m);
    }
    f32x4 *out = reinterpret_cast<f32x4 *>(gstate + ((size_t)bh * G + grp) * TL::STATE_FLOATS);
#pragma unroll
    for (int u = 0; u < TL::TPW; ++u) out[(w * TL::TPW + u) * 64 + l] = S[u];
}

// Over the G slots of one head, element-wise: mode 0 -> exclusive prefix in place (slot g gets the
// sum of slots < g; only the first `ncomputed` slots hold data), mode 1 -> total into slot 0.
static __global__ __launch_bounds__(kThreads) void state_prefix_kernel(float *__restrict__ gstate, int G, int ncomputed,
                                                                int state_floats, int mode) {
    const int sf4 = state_floats / 4;
    const int blocks_per_head = (sf4 + kThreads - 1) / kThreads;
    const int bh = blockIdx.x / blocks_per_head;
    const int e = (blockIdx.x % blocks_per_head) * kThreads + threadIdx.x;
    if (e >= sf4) return;
    f32x4 *p = reinterpret_cast<f32x4 *>(gstate + (size_t)bh * G * state_floats) + e;
    f32x4 run = {0.f, 0.f, 0.f, 0.f};
    for (int s = 0; s < G; ++s) {
        f32x4 t = {0.f, 0.f, 0.f, 0.f};
        if (s < ncomputed) t = p[(size_t)s * sf4];
        if (mode == 0) p[(size_t)s * sf4] = run;
        run += t;
    }
    if (mode == 1) p[0] = run;
}

// The chunk recurrence for one group of one head.  CAUSAL=false is the non-causal apply pass:
// out = A * S_total with the state taken from slot 0 and never updated.
//
// Work split (4 wavefronts, chunk of 64): wavefront w owns output positions 16w..16w+15 of the
// chunk.  It forms P^T = B_c A_w^T tile by tile (so the accumulator layout IS the operand layout
// of the next product -- the masked scores never leave registers), then
// out_w^T = C_c^T P^T + S^T A_w^T, stored as 8-byte row segments.
template <class TR, int DI, int DJ, bool CAUSAL>
__global__ __launch_bounds__(kThreads) void scan_kernel(const u16 *__restrict__ A, const u16 *__restrict__ B,
                                                        const u16 *__restrict__ C, u16 *__restrict__ O,
                                                        const float *__restrict__ gstate, int N, int di, int dj,
                                                        int nchunks, int cpg, int G, int reversed) {
    using TL = Tiling<DI, DJ>;
    __shared__ __attribute__((aligned(16))) u16 sB[CAUSAL ? kChunk * TL::BS : 8];
    __shared__ __attribute__((aligned(16))) u16 sC[CAUSAL ? kChunk * TL::CS : 8];
    __shared__ __attribute__((aligned(16))) u16 sS[DJ * TL::SS];
    const int tid = threadIdx.x, w = tid >> 6, l = tid & 63, g = l >> 4, m = l & 15;
    const int grp = blockIdx.x % G, bh = blockIdx.x / G;
    A += (size_t)bh * N * di;
    B += (size_t)bh * N * di;
    C += (size_t)bh * N * dj;
    O += (size_t)bh * N * dj;
    const int p0 = grp * cpg;
    const int p1 = min(p0 + cpg, nchunks);

    f32x4 S[TL::TPW];
#pragma unroll
    for (int u = 0; u < TL::TPW; ++u) S[u] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (gstate != nullptr) {
        const f32x4 *gs =
            reinterpret_cast<const f32x4 *>(gstate + ((size_t)bh * G + (CAUSAL ? grp : 0)) * TL::STATE_FLOATS);
#pragma unroll
        for (int u = 0; u < TL::TPW; ++u) S[u] = gs[(w * TL::TPW + u) * 64 + l];
    }

    u32x4 rb[DI / 32], rc[DJ / 32], qn[TL::KS], qc[TL::KS];
    auto load_chunk = [&](int p) {
        const int row0 = (reversed ? nchunks - 1 - p : p) * kChunk;
        if (CAUSAL) {
            load_tile<DI>(rb, B, row0, N, di, tid);
            load_tile<DJ>(rc, C, row0, N, dj, tid);
        }
        const int row = row0 + 16 * w + m;
#pragma unroll
        for (int ks = 0; ks < TL::KS; ++ks) {
            const int col = 32 * ks + 8 * g;
            qn[ks] = ld_global16(A + (size_t)row * di + col, row < N && col < di);
        }
    };
    load_chunk(p0);

    for (int p = p0; p < p1; ++p) {
        const int row0 = (reversed ? nchunks - 1 - p : p) * kChunk;
        __syncthreads();  // every wavefront is done reading the previous chunk's tiles
        if (CAUSAL) {
            store_tile<DI>(sB, rb, tid);
            store_tile<DJ>(sC, rc, tid);
        }
        if (CAUSAL || p == p0) {
            // 16-bit copy of the state BEFORE this chunk, transposed to [j][i] for the A_w S product
#pragma unroll
            for (int u = 0; u < TL::TPW; ++u) {
                const int t = w * TL::TPW + u;
                const int it = t / TL::NJT, jt = t % TL::NJT;
                u32x2 pk = {TR::pack2(S[u][0], S[u][1]), TR::pack2(S[u][2], S[u][3])};
                *reinterpret_cast<u32x2 *>(sS + (16 * jt + m) * TL::SS + 16 * it + 4 * g) = pk;
            }
        }
#pragma unroll
        for (int ks = 0; ks < TL::KS; ++ks) qc[ks] = qn[ks];
        __syncthreads();
        if (p + 1 < p1) load_chunk(p + 1);  // prefetch: lands while this chunk is computed

        // masked scores, transposed: pk[jt] = P^T[16jt+4g .. +3][16w+m]
        u32x2 pk[4];
        if (CAUSAL) {
#pragma unroll
            for (int jt = 0; jt < 4; ++jt) {
                pk[jt] = u32x2{0u, 0u};
                const bool active = reversed ? (jt >= w) : (jt <= w);
                if (active) {
                    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int ks = 0; ks < TL::KS; ++ks) {
                        const u32x4 a = *reinterpret_cast<const u32x4 *>(sB + (16 * jt + m) * TL::BS + 32 * ks + 8 * g);
                        acc = TR::mfma(a, qc[ks], acc);
                    }
                    if (jt == w) {
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            const bool keep = reversed ? (4 * g + r >= m) : (4 * g + r <= m);
                            acc[r] = keep ? acc[r] : 0.f;
                        }
                    }
                    pk[jt] = u32x2{TR::pack2(acc[0], acc[1]), TR::pack2(acc[2], acc[3])};
                }
            }
        }

        const int orow = row0 + 16 * w + m;
#pragma unroll
        for (int jt = 0; jt < TL::NJT; ++jt) {
            f32x4 o = {0.f, 0.f, 0.f, 0.f};
            if (CAUSAL) {
#pragma unroll
                for (int kb = 0; kb < 2; ++kb) {
                    const bool active = reversed ? (2 * kb + 1 >= w) : (2 * kb <= w);
                    if (active) {
                        const u32x4 a = cat(lds_col4(sC, TL::CS, 32 * kb + 4 * g, 16 * jt, m),
                                            lds_col4(sC, TL::CS, 32 * kb + 16 + 4 * g, 16 * jt, m));
                        o = TR::mfma(a, cat(pk[2 * kb], pk[2 * kb + 1]), o);
                    }
                }
            }
#pragma unroll
            for (int ks = 0; ks < TL::KS; ++ks) {
                const u32x4 a = *reinterpret_cast<const u32x4 *>(sS + (16 * jt + m) * TL::SS + 32 * ks + 8 * g);
                o = TR::mfma(a, qc[ks], o);
            }
            const int col = 16 * jt + 4 * g;
            if (orow < N && col < dj) {
                u32x2 v = {TR::pack2(o[0], o[1]), TR::pack2(o[2], o[3])};
                *reinterpret_cast<u32x2 *>(O + (size_t)orow * dj + col) = v;
            }
        }
        if (CAUSAL) state_update<TR, DI, DJ>(S, sB, sC, w, g, m);
    }
}

}  // namespace cott
