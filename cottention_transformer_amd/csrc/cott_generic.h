// Plain-FMA kernels for every storage type (fp32, fp64, and 16-bit types whose head dims fall
// outside the MFMA kernels' range), plus the bandwidth-bound decode step.
#pragma once
#include "cott_common.h"

namespace cott {

struct StF32 {
    typedef float elem;
    typedef float acc;
    __device__ static __forceinline__ acc load(const elem *p) { return *p; }
    __device__ static __forceinline__ void store(elem *p, acc v) { *p = v; }
};
struct StF64 {
    typedef double elem;
    typedef double acc;
    __device__ static __forceinline__ acc load(const elem *p) { return *p; }
    __device__ static __forceinline__ void store(elem *p, acc v) { *p = v; }
};
struct StBf16 {
    typedef u16 elem;
    typedef float acc;
    __device__ static __forceinline__ acc load(const elem *p) { return Bf16::to_float(*p); }
    __device__ static __forceinline__ void store(elem *p, acc v) { *p = Bf16::from_float(v); }
};
struct StFp16 {
    typedef u16 elem;
    typedef float acc;
    __device__ static __forceinline__ acc load(const elem *p) { return Fp16::to_float(*p); }
    __device__ static __forceinline__ void store(elem *p, acc v) { *p = Fp16::from_float(v); }
};

// Chunked scan with a [di][DJT] slice of the state in LDS; one workgroup per (j-slice, head)
// walks the whole sequence.  CH (chunk length) and DJT (slice width) are chosen by the host so
// that the dynamic LDS footprint fits.  CAUSAL=false: out = A (B^T C) in two passes.
template <class ST, bool CAUSAL>
__global__ __launch_bounds__(256) void generic_scan_kernel(const typename ST::elem *__restrict__ A,
                                                           const typename ST::elem *__restrict__ B,
                                                           const typename ST::elem *__restrict__ C,
                                                           typename ST::elem *__restrict__ O,
                                                           const typename ST::acc *__restrict__ sin,
                                                           typename ST::acc *__restrict__ sout, int N, int di, int dj,
                                                           int CH, int DJT, int nslices, int reversed) {
    typedef typename ST::acc acc_t;
    extern __shared__ __attribute__((aligned(32))) unsigned char smem_raw[];
    acc_t *sA = reinterpret_cast<acc_t *>(smem_raw);  // [CH][di+1]
    acc_t *sB = sA + CH * (di + 1);                   // [CH][di+1]
    acc_t *sC = sB + CH * (di + 1);                   // [CH][DJT]
    acc_t *sP = sC + CH * DJT;                        // [CH][CH+1]
    acc_t *sS = sP + CH * (CH + 1);                   // [di][DJT]
    const int tid = threadIdx.x;
    const int j0 = (blockIdx.x % nslices) * DJT, bh = blockIdx.x / nslices;
    A += (size_t)bh * N * di;
    B += (size_t)bh * N * di;
    C += (size_t)bh * N * dj;
    O += (size_t)bh * N * dj;
    const int nchunks = (N + CH - 1) / CH;
    const int lda = di + 1;

    // start state: zero, or the caller's [di][dj] row-major state of this head
    for (int x = tid; x < di * DJT; x += 256) {
        const int i = x / DJT, jj = x % DJT;
        sS[x] = (sin != nullptr && j0 + jj < dj) ? sin[((size_t)bh * di + i) * dj + j0 + jj] : (acc_t)0;
    }

    auto load_bc = [&](int row0) {
        for (int x = tid; x < CH * di; x += 256) {
            const int r = x / di, i = x % di;
            sB[r * lda + i] = (row0 + r < N) ? ST::load(B + (size_t)(row0 + r) * di + i) : (acc_t)0;
        }
        for (int x = tid; x < CH * DJT; x += 256) {
            const int r = x / DJT, jj = x % DJT;
            sC[x] = (row0 + r < N && j0 + jj < dj) ? ST::load(C + (size_t)(row0 + r) * dj + j0 + jj) : (acc_t)0;
        }
    };
    auto update_state = [&]() {
        for (int x = tid; x < di * DJT; x += 256) {
            const int i = x / DJT, jj = x % DJT;
            acc_t s = sS[x];
            for (int t = 0; t < CH; ++t) s += sB[t * lda + i] * sC[t * DJT + jj];
            sS[x] = s;
        }
    };

    if (!CAUSAL) {
        for (int c = 0; c < nchunks; ++c) {
            __syncthreads();
            load_bc(c * CH);
            __syncthreads();
            update_state();
        }
    }

    for (int p = 0; p < nchunks; ++p) {
        const int row0 = (reversed ? nchunks - 1 - p : p) * CH;
        __syncthreads();
        for (int x = tid; x < CH * di; x += 256) {
            const int r = x / di, i = x % di;
            sA[r * lda + i] = (row0 + r < N) ? ST::load(A + (size_t)(row0 + r) * di + i) : (acc_t)0;
        }
        if (CAUSAL) load_bc(row0);
        __syncthreads();
        if (CAUSAL) {
            for (int x = tid; x < CH * CH; x += 256) {
                const int r = x / CH, t = x % CH;
                acc_t s = (acc_t)0;
                if (reversed ? (t >= r) : (t <= r))
                    for (int i = 0; i < di; ++i) s += sA[r * lda + i] * sB[t * lda + i];
                sP[r * (CH + 1) + t] = s;
            }
            __syncthreads();
        }
        for (int x = tid; x < CH * DJT; x += 256) {
            const int r = x / DJT, jj = x % DJT;
            acc_t s = (acc_t)0;
            if (CAUSAL)
                for (int t = 0; t < CH; ++t) s += sP[r * (CH + 1) + t] * sC[t * DJT + jj];
            for (int i = 0; i < di; ++i) s += sA[r * lda + i] * sS[i * DJT + jj];
            if (row0 + r < N && j0 + jj < dj) ST::store(O + (size_t)(row0 + r) * dj + j0 + jj, s);
        }
        if (CAUSAL) {
            __syncthreads();
            update_state();
        }
    }
    if (sout != nullptr) {
        __syncthreads();
        for (int x = tid; x < di * DJT; x += 256) {
            const int i = x / DJT, jj = x % DJT;
            if (j0 + jj < dj) sout[((size_t)bh * di + i) * dj + j0 + jj] = sS[x];
        }
    }
}

// Decode step: one workgroup per (batch, head) streams its [dk][dv] state once.
//   S[i][j] += k[i] v[j] ;  o[j] = sum_i q[i] S[i][j]
// Thread t owns a 4-wide column strip (t % nvb) and every rg-th row starting at t / nvb.  Rows are
// processed 16 at a time; the state loads of a pass are issued before anything else (q and k are
// staged through LDS while they are in flight) and every load precedes the first store.
template <class ST, class SF /* state scalar: float or double */>
__global__ __launch_bounds__(256) void decode_kernel(SF *__restrict__ S, const typename ST::elem *__restrict__ q,
                                                     const typename ST::elem *__restrict__ k,
                                                     const typename ST::elem *__restrict__ v,
                                                     typename ST::elem *__restrict__ o, int dk, int dv) {
    typedef SF __attribute__((ext_vector_type(4))) sf4;
    constexpr int U = 16;
    extern __shared__ __attribute__((aligned(32))) unsigned char smem_raw[];
    SF *sq = reinterpret_cast<SF *>(smem_raw);  // [dk]
    SF *sk = sq + dk;                           // [dk]
    sf4 *sred = reinterpret_cast<sf4 *>(sk + dk);  // [256]
    const int tid = threadIdx.x, bh = blockIdx.x;
    S += (size_t)bh * dk * dv;
    q += (size_t)bh * dk;
    k += (size_t)bh * dk;
    v += (size_t)bh * dv;
    o += (size_t)bh * dv;
    const int nv = dv / 4;
    const int nvb = nv < 256 ? nv : 256;
    const int rg = 256 / nvb;
    const int mc = tid % nvb, mr = tid / nvb;
    bool staged = false;
    for (int c0 = 0; c0 < nv; c0 += nvb) {
        const int c4 = c0 + mc;
        const bool live = (mr < rg) && (c4 < nv);
        sf4 acc = {0, 0, 0, 0};
        sf4 vv = {0, 0, 0, 0};
        sf4 *col = reinterpret_cast<sf4 *>(S) + (live ? c4 : 0);
        for (int r0 = mr; r0 < dk || !staged; r0 += U * rg) {
            sf4 s[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int r = r0 + u * rg;
                if (live && r < dk) s[u] = col[(size_t)r * nv];
            }
            if (!staged) {  // first pass of the workgroup: q, k -> LDS while the state is in flight
                for (int i = tid; i < dk; i += 256) {
                    sq[i] = (SF)ST::load(q + i);
                    sk[i] = (SF)ST::load(k + i);
                }
                __syncthreads();
                staged = true;
            }
            if (live && r0 == mr) {
                vv.x = (SF)ST::load(v + 4 * c4);
                vv.y = (SF)ST::load(v + 4 * c4 + 1);
                vv.z = (SF)ST::load(v + 4 * c4 + 2);
                vv.w = (SF)ST::load(v + 4 * c4 + 3);
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int r = r0 + u * rg;
                if (live && r < dk) {
                    s[u] += sk[r] * vv;
                    col[(size_t)r * nv] = s[u];
                    acc += sq[r] * s[u];
                }
            }
        }
        __syncthreads();
        sred[tid] = acc;
        __syncthreads();
        if (mr == 0 && c4 < nv) {
            sf4 t = sred[mc];
            for (int r = 1; r < rg; ++r) t += sred[r * nvb + mc];
            ST::store(o + 4 * c4, (typename ST::acc)t.x);
            ST::store(o + 4 * c4 + 1, (typename ST::acc)t.y);
            ST::store(o + 4 * c4 + 2, (typename ST::acc)t.z);
            ST::store(o + 4 * c4 + 3, (typename ST::acc)t.w);
        }
    }
}

// Decode step, one WAVEFRONT per (batch, head): no workgroup barrier anywhere, so the four heads of
// a workgroup stream independently.  For dv/4 = nv in {8,16,32,64} columns of float4: lane l owns
// column l % nv and every (64/nv)-th row starting at l / nv; q and k are staged in a per-wavefront
// LDS slice while the first batch of state loads is in flight; the row groups are combined with
// lane-xor shuffles.  Plain (cacheable) loads and stores: a state that fits the last-level cache is
// then served from it on the next step.
// Optional preparation of the raw projections of the ONE new token inside the decode step (on = 1): GPT-J
// rotation of the first R columns of q and k by the table row `pos`, L2 normalisation of q and k, and
// v / max(cnt^sig[h], 1) -- what GPT_Trainer/GPTCosAttention.py:229-248,462-476 do with separate kernels before
// the recurrence of :264-267.  dk <= 256.
struct DecodePrep {
    const float *sig;  // (H) sigmoid(norm_const), or null: no value scaling
    const float *rot;  // (rows, R) table [sin | cos], or null: no rotation
    long long pos;     // table row, already clamped to the table
    float cnt, eps;    // number of tokens so far including this one; norm clamp
    int R, H, on;
};

// NT bit 0: non-temporal state loads, bit 1: non-temporal state stores (a state far larger than the last-level
// cache is not found there again by the next step).
template <class ST, class SF, bool PREP, int NT = 0>
__global__ __launch_bounds__(256) void decode_wave_kernel(SF *__restrict__ S, const typename ST::elem *__restrict__ q,
                                                          const typename ST::elem *__restrict__ k,
                                                          const typename ST::elem *__restrict__ v,
                                                          typename ST::elem *__restrict__ o, int BH, int dk, int dv,
                                                          DecodePrep prep) {
    typedef SF __attribute__((ext_vector_type(4))) sf4;
    constexpr int U = 16;
    extern __shared__ __attribute__((aligned(32))) unsigned char smem_raw[];
    const int lane = threadIdx.x & 63;
    const int wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int bh = blockIdx.x * 4 + wv;
    if (bh >= BH) return;
    SF *sq = reinterpret_cast<SF *>(smem_raw) + (size_t)wv * 2 * dk;  // this wavefront's [q | k]
    SF *sk = sq + dk;
    S += (size_t)bh * dk * dv;
    q += (size_t)bh * dk;
    k += (size_t)bh * dk;
    v += (size_t)bh * dv;
    o += (size_t)bh * dv;
    const int nv = dv / 4;       // 8, 16, 32 or 64
    const int rpw = 64 / nv;     // rows covered by one wavefront-wide load
    const int mc = lane % nv, mr = lane / nv;
    sf4 *col = reinterpret_cast<sf4 *>(S) + mc;
    sf4 acc = {0, 0, 0, 0};
    sf4 vv = {0, 0, 0, 0};
    bool staged = false;
    for (int r0 = mr; r0 < dk; r0 += U * rpw) {
        sf4 s[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int r = r0 + u * rpw;
            if (r < dk) s[u] = (NT & 1) ? __builtin_nontemporal_load(&col[(size_t)r * nv]) : col[(size_t)r * nv];
        }
        if (!staged) {
            if constexpr (PREP) {
                vv.x = (SF)ST::load(v + 4 * mc);
                vv.y = (SF)ST::load(v + 4 * mc + 1);
                vv.z = (SF)ST::load(v + 4 * mc + 2);
                vv.w = (SF)ST::load(v + 4 * mc + 3);
                // element i = lane + 64 t of q and k lives in lane `lane`; the pair partner of the rotation (i ^ 1) in
                // the neighbouring lane; every lane takes part in every shuffle
                SF xq[4], xk[4], ssq = 0, ssk = 0;
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const int i = lane + 64 * t;
                    xq[t] = i < dk ? (SF)ST::load(q + i) : (SF)0;
                    xk[t] = i < dk ? (SF)ST::load(k + i) : (SF)0;
                    const SF pq = __shfl_xor(xq[t], 1), pk = __shfl_xor(xk[t], 1);
                    if (prep.rot != nullptr && i < prep.R) {
                        const SF sn = (SF)prep.rot[prep.pos * prep.R + i / 2];
                        const SF cs = (SF)prep.rot[prep.pos * prep.R + prep.R / 2 + i / 2];
                        xq[t] = (i & 1) ? xq[t] * cs + pq * sn : xq[t] * cs - pq * sn;
                        xk[t] = (i & 1) ? xk[t] * cs + pk * sn : xk[t] * cs - pk * sn;
                    }
                    ssq += xq[t] * xq[t];
                    ssk += xk[t] * xk[t];
                }
                for (int off = 1; off < 64; off <<= 1) {
                    ssq += __shfl_xor(ssq, off);
                    ssk += __shfl_xor(ssk, off);
                }
                const SF nq = sqrt(ssq), nk = sqrt(ssk);
                const SF rq = (SF)1 / (nq > (SF)prep.eps ? nq : (SF)prep.eps), rk = (SF)1 / (nk > (SF)prep.eps ? nk : (SF)prep.eps);
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const int i = lane + 64 * t;
                    if (i < dk) {
                        sq[i] = xq[t] * rq;
                        sk[i] = xk[t] * rk;
                    }
                }
                if (prep.sig != nullptr) {
                    const SF p = prep.cnt > 0.f ? (SF)pow((SF)prep.cnt, (SF)prep.sig[bh % prep.H]) : (SF)0;
                    if (p > (SF)1) vv = vv * ((SF)1 / p);
                }
            } else {
                for (int i = lane; i < dk; i += 64) {
                    sq[i] = (SF)ST::load(q + i);
                    sk[i] = (SF)ST::load(k + i);
                }
                vv.x = (SF)ST::load(v + 4 * mc);
                vv.y = (SF)ST::load(v + 4 * mc + 1);
                vv.z = (SF)ST::load(v + 4 * mc + 2);
                vv.w = (SF)ST::load(v + 4 * mc + 3);
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            staged = true;
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int r = r0 + u * rpw;
            if (r < dk) {
                s[u] += sk[r] * vv;
                if (NT & 2)
                    __builtin_nontemporal_store(s[u], &col[(size_t)r * nv]);
                else
                    col[(size_t)r * nv] = s[u];
                acc += sq[r] * s[u];
            }
        }
    }
    for (int off = nv; off < 64; off <<= 1) {
        acc.x += __shfl_xor(acc.x, off);
        acc.y += __shfl_xor(acc.y, off);
        acc.z += __shfl_xor(acc.z, off);
        acc.w += __shfl_xor(acc.w, off);
    }
    if (mr == 0) {
        ST::store(o + 4 * mc, (typename ST::acc)acc.x);
        ST::store(o + 4 * mc + 1, (typename ST::acc)acc.y);
        ST::store(o + 4 * mc + 2, (typename ST::acc)acc.z);
        ST::store(o + 4 * mc + 3, (typename ST::acc)acc.w);
    }
}

}  // namespace cott
