// fp32 storage on the bf16 matrix cores: every fp32 operand is split into two bf16 numbers, x = hi + lo with
// hi = bf16(x) and lo = bf16(x - hi), and every product of the chunk recurrence is formed from three bf16 matrix
// instructions accumulating in fp32,
//     a b  ~  a_hi b_hi + a_hi b_lo + a_lo b_hi .
// hi + lo carries 16 of the 24 significant bits of x and the term left out, a_lo b_lo, is 2^-16 of the product: measured
// rel-L2 of o, dQ, dK, dV against fp64 is 6.3e-6, inside the 1e-4 bar of fp32 inputs (the fp32 matrix pipe gives
// 2e-7).  The price is three times the bf16 matrix work; the fp32 matrix pipe is sixteen times slower than the bf16
// one on this part and the kernels on it (cott_mfma_f32.h) are bound by it: at B8 H16 N2048 D64 forward + backward
// takes 430 us there and 243 us here (forward 73: group sums 26, prefix 6, scan 50; three gradients 146).
//
// Structure: that of colscan_kernel (cott_colscan.h) -- four compute wavefronts that each own a quarter of the
// state's columns in fp32 accumulators and produce those columns of the output, the masked scores formed once per
// workgroup and handed round through LDS, four loader wavefronts -- with these differences:
//   * the loaders read fp32 rows and write TWO 16-bit tiles per operand (hi and lo);
//   * the 16-bit operand copies of the state and of the masked scores are split the same way;
//   * the outputs leave as fp32 straight from the accumulators (16 bytes per lane and tile);
//   * one barrier per chunk: the (scores) x C product of a chunk is finished at the start of the next one, when every
//     wavefront's score tiles have passed the barrier anyway (a barrier in the middle of the chunk also stops the
//     loader wavefronts, whose conversion work is a fifth of the chunk here: gradients 164 -> 146 us).
// Where the time goes (counters at the shape above, gradient launch, 384 workgroups on 256 CUs): per workgroup and chunk
// 5300 cycles, of which the matrix pipe is busy 1344 on each SIMD, LDS 2030, vector-ALU issue about 2600 (the hi / lo
// conversions of loaders and compute wavefronts: 284 instructions per wavefront), waves waiting on counters a third
// of their time: one workgroup of eight wavefronts per CU (155 KiB of LDS) leaves no second wavefront to cover them.
// The state slots of the group-state pass use the layout of the 16-bit kernels, so state_prefix_kernel serves both.
// Padded head dims 64 x 64 (33 .. 64 columns); other widths stay on the fp32 matrix pipe.
#pragma once
#include "cott_colscan.h"

namespace cott {

typedef ProblemT<float> ProblemF;
typedef ProblemSetT<float> ProblemSetF;

// eight fp32 values (two 16-byte vectors) -> their bf16 hi parts and bf16 lo parts
__device__ __forceinline__ void split8(u32x4 a, u32x4 b, u32x4 &hi, u32x4 &lo) {
    const float x[8] = {bitcast<float>(a[0]), bitcast<float>(a[1]), bitcast<float>(a[2]), bitcast<float>(a[3]),
                        bitcast<float>(b[0]), bitcast<float>(b[1]), bitcast<float>(b[2]), bitcast<float>(b[3])};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const uint32_t h = Bf16::pack2(x[2 * e], x[2 * e + 1]);
        hi[e] = h;
        lo[e] = Bf16::pack2(x[2 * e] - bitcast<float>(h << 16), x[2 * e + 1] - bitcast<float>(h & 0xffff0000u));
    }
}
// four accumulator values -> two dwords of hi parts, two of lo parts
__device__ __forceinline__ void split4(f32x4 v, u32x2 &hi, u32x2 &lo) {
#pragma unroll
    for (int e = 0; e < 2; ++e) {
        const uint32_t h = Bf16::pack2(v[2 * e], v[2 * e + 1]);
        hi[e] = h;
        lo[e] = Bf16::pack2(v[2 * e] - bitcast<float>(h << 16), v[2 * e + 1] - bitcast<float>(h & 0xffff0000u));
    }
}
// Term t = 0, 1, 2 of a product: a_lo b_hi, a_hi b_lo, a_hi b_hi.  Callers with several independent accumulators run term
// 0 for all of them, then term 1, then term 2, so that a matrix instruction never follows the one it depends on.
__device__ __forceinline__ f32x4 mfma_term(int t, u32x4 ah, u32x4 al, u32x4 bh, u32x4 bl, f32x4 c) {
    return Bf16::mfma(t == 0 ? al : ah, t == 1 ? bl : bh, c);
}
// c + a b from the three leading terms of (a_hi + a_lo)(b_hi + b_lo)
__device__ __forceinline__ f32x4 mfma3(u32x4 ah, u32x4 al, u32x4 bh, u32x4 bl, f32x4 c) {
    c = Bf16::mfma(al, bh, c);
    c = Bf16::mfma(ah, bl, c);
    return Bf16::mfma(ah, bh, c);
}

// [64][D] fp32 tile, global -> registers: thread t of NT owns the 32-byte pieces t, t + NT, ... (eight columns of a row)
template <int D, int NT, bool STREAM>
__device__ __forceinline__ void load_tile_f(u32x4 (*r)[2], rsrc_t rs, int row0, int ld, int tid) {
#pragma unroll
    for (int u = 0; u < 8 * D / NT; ++u) {
        const int v = tid + NT * u;
        const uint32_t off = (uint32_t)((row0 + v / (D / 8)) * ld + (v % (D / 8)) * 8) * 4u;
        r[u][0] = buf_load16<STREAM>(rs, off);
        r[u][1] = buf_load16<STREAM>(rs, off + 16u);
    }
}
// registers -> the hi tile and the lo tile in LDS; columns past the runtime width d become zero
template <int D, int STRIDE, int NT>
__device__ __forceinline__ void store_tile_split(u16 *th, u16 *tl, const u32x4 (*r)[2], int d, int tid) {
#pragma unroll
    for (int u = 0; u < 8 * D / NT; ++u) {
        const int v = tid + NT * u;
        const int col = (v % (D / 8)) * 8;
        u32x4 hi = {0u, 0u, 0u, 0u}, lo = hi;
        if (col < d) split8(r[u][0], r[u][1], hi, lo);
        *reinterpret_cast<u32x4 *>(th + (v / (D / 8)) * STRIDE + col) = hi;
        *reinterpret_cast<u32x4 *>(tl + (v / (D / 8)) * STRIDE + col) = lo;
    }
}

// Sum of B^T C over each group of chunks of each head, in the slot layout of group_state_kernel (cott_mfma.h):
// float4 index (w * TPW + u) * 64 + lane of slot (bh * G + grp) * sub + piece.
template <int DI, int DJ, int PF>
__global__ __launch_bounds__(kThreads) void group_state_split_kernel(ProblemSetF set, int BH, int N, int nchunks, int cpg,
                                                                     int G, int ngroups) {
    using TL = Tiling<DI, DJ>;
    constexpr int SB = kChunk * TL::BS, SC = kChunk * TL::CS;
    __shared__ __attribute__((aligned(16))) u16 sBh[2 * SB];
    __shared__ __attribute__((aligned(16))) u16 sBl[2 * SB];
    __shared__ __attribute__((aligned(16))) u16 sCh[2 * SC];
    __shared__ __attribute__((aligned(16))) u16 sCl[2 * SC];
    const int tid = threadIdx.x, l = tid & 63, g = l >> 4, m = l & 15;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    // every group is cut into `sub` pieces, one workgroup and one slot each (slot (bh * G + grp) * sub + piece)
    const int sub = set.sub;
    const WorkItem wi = decode_workgroup(set.nact * sub, BH, set.xcds);
    if (wi.grp >= ngroups) return;
    const ProblemF &pr = set.p[set.act[wi.prob / sub]];
    const int piece = wi.prob % sub;
    const int di = pr.di, dj = pr.dj, ldb = pr.ldb, ldc = pr.ldc, reversed = pr.reversed;
    const rsrc_t rB = make_rsrc(pr.B + head_base(pr.bsB, pr.hsB, pr.H, wi.bh), ((uint32_t)(N - 1) * ldb + di) * 4u);
    const rsrc_t rC = make_rsrc(pr.C + head_base(pr.bsC, pr.hsC, pr.H, wi.bh), ((uint32_t)(N - 1) * ldc + dj) * 4u);
    const int cps = (cpg + sub - 1) / sub;  // chunks per piece
    const int p0 = wi.grp * cpg + piece * cps;
    const int p1 = min(p0 + cps, min((wi.grp + 1) * cpg, nchunks));
    f32x4 S[TL::TPW];
#pragma unroll
    for (int u = 0; u < TL::TPW; ++u) S[u] = f32x4{0.f, 0.f, 0.f, 0.f};
    f32x4 *slot = reinterpret_cast<f32x4 *>(pr.gstate + (((size_t)wi.bh * G + wi.grp) * sub + piece) * TL::STATE_FLOATS);
    if (p1 <= p0) {  // a piece past the end of its group: its slot is zero
#pragma unroll
        for (int u = 0; u < TL::TPW; ++u) slot[(w * TL::TPW + u) * 64 + l] = S[u];
        return;
    }
    u32x4 rb[PF][DI / 32][2], rc[PF][DJ / 32][2];
    auto load_chunk = [&](int s, int p) __attribute__((always_inline)) {
        const int pc = min(p, p1 - 1);
        const int row0 = (reversed ? nchunks - 1 - pc : pc) * kChunk;
        load_tile_f<DI, kThreads, false>(rb[s], rB, row0, ldb, tid);
        load_tile_f<DJ, kThreads, false>(rc[s], rC, row0, ldc, tid);
    };
    auto stage = [&](int s, int buf) __attribute__((always_inline)) {
        store_tile_split<DI, TL::BS, kThreads>(sBh + buf * SB, sBl + buf * SB, rb[s], di, tid);
        store_tile_split<DJ, TL::CS, kThreads>(sCh + buf * SC, sCl + buf * SC, rc[s], dj, tid);
    };
    // S[i][j] += sum over the 64 positions of B[tok][i] C[tok][j] for the tiles this wavefront owns (see state_update)
    auto update = [&](int buf) __attribute__((always_inline)) {
        constexpr int ROWS = (TL::TPW + TL::NJT - 1) / TL::NJT;
        constexpr int COLS = TL::TPW < TL::NJT ? TL::TPW : TL::NJT;
        const u16 *bh = sBh + buf * SB, *bl = sBl + buf * SB, *ch = sCh + buf * SC, *cl = sCl + buf * SC;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            const int k0 = 32 * kb + 8 * g;
            u32x4 ah[ROWS], al[ROWS], xh[COLS], xl[COLS];
#pragma unroll
            for (int r = 0; r < ROWS; ++r) {
                const int it = (w * TL::TPW + r * TL::NJT) / TL::NJT;
                ah[r] = cat(lds_col4(bh, TL::BS, k0, 16 * it, m), lds_col4(bh, TL::BS, k0 + 4, 16 * it, m));
                al[r] = cat(lds_col4(bl, TL::BS, k0, 16 * it, m), lds_col4(bl, TL::BS, k0 + 4, 16 * it, m));
            }
#pragma unroll
            for (int c = 0; c < COLS; ++c) {
                const int jt = (w * TL::TPW + c) % TL::NJT;
                xh[c] = cat(lds_col4(ch, TL::CS, k0, 16 * jt, m), lds_col4(ch, TL::CS, k0 + 4, 16 * jt, m));
                xl[c] = cat(lds_col4(cl, TL::CS, k0, 16 * jt, m), lds_col4(cl, TL::CS, k0 + 4, 16 * jt, m));
            }
#pragma unroll
            for (int u = 0; u < TL::TPW; ++u)
                S[u] = mfma3(ah[u / TL::NJT], al[u / TL::NJT], xh[u % COLS], xl[u % COLS], S[u]);
        }
    };
#pragma unroll
    for (int s = 0; s < PF; ++s) load_chunk(s, p0 + s);
    stage(0, 0);
    load_chunk(0, p0 + PF);
    __syncthreads();
    run_rounds<PF>(p0, p1, [&](int s, int p) __attribute__((always_inline)) {
        const int s1 = (s + 1) % PF;
        const int buf = (p - p0) & 1;
        stage(s1, buf ^ 1);
        load_chunk(s1, p + 1 + PF);
        update(buf);
        chunk_barrier();
    });
#pragma unroll
    for (int u = 0; u < TL::TPW; ++u) slot[(w * TL::TPW + u) * 64 + l] = S[u];
}

// Loader role: LT threads move the A, B and C tiles of fp32 rows global -> registers -> hi / lo tiles in LDS, PF
// chunks ahead.  One barrier per chunk.
template <int DI, int DJ, int PF, int LT>
__device__ __forceinline__ void split_loader_role(const float *A_head, const float *B_head, const float *C_head, int di, int dj,
                                                  int lda, int ldb, int ldc, const ScanRange &r, int tid, u16 *sA, u16 *sB,
                                                  u16 *sC) {
    using TL = Tiling<DI, DJ>;
    using CT = ColTiling<DI, DJ>;
    static_assert((8 * DI) % LT == 0 && (8 * DJ) % LT == 0, "tile pieces divide over the loader threads");
    const rsrc_t rA = make_rsrc(A_head, ((uint32_t)(r.N - 1) * lda + di) * 4u);
    const rsrc_t rB = make_rsrc(B_head, ((uint32_t)(r.N - 1) * ldb + di) * 4u);
    const rsrc_t rC = make_rsrc(C_head, ((uint32_t)(r.N - 1) * ldc + dj) * 4u);
    u32x4 ra[PF][8 * DI / LT][2], rb[PF][8 * DI / LT][2], rc[PF][8 * DJ / LT][2];
    auto load_chunk = [&](int s, int p) __attribute__((always_inline)) {
        const int pc = min(p, r.p1 - 1);
        const int row0 = (r.reversed ? r.nchunks - 1 - pc : pc) * kChunk;
        load_tile_f<DI, LT, false>(ra[s], rA, row0, lda, tid);
        load_tile_f<DI, LT, false>(rb[s], rB, row0, ldb, tid);
        load_tile_f<DJ, LT, false>(rc[s], rC, row0, ldc, tid);
    };
    // LDS: [hi | lo] x [2 buffers] per operand
    auto stage = [&](int s, int buf) __attribute__((always_inline)) {
        store_tile_split<DI, TL::BS, LT>(sA + buf * CT::SA, sA + (2 + buf) * CT::SA, ra[s], di, tid);
        store_tile_split<DI, TL::BS, LT>(sB + buf * CT::SA, sB + (2 + buf) * CT::SA, rb[s], di, tid);
        store_tile_split<DJ, TL::CS, LT>(sC + buf * CT::SC, sC + (2 + buf) * CT::SC, rc[s], dj, tid);
    };
#pragma unroll
    for (int s = 0; s < PF; ++s) load_chunk(s, r.p0 + s);
    stage(0, 0);
    load_chunk(0, r.p0 + PF);
    __syncthreads();
    run_rounds<PF>(r.p0, r.p1, [&](int s, int p) __attribute__((always_inline)) {
        const int s1 = (s + 1) % PF;
        const int buf = (p - r.p0) & 1;
        stage(s1, buf ^ 1);
        load_chunk(s1, p + 1 + PF);
        chunk_barrier();
    });
}

// Compute role: col_compute_role (cott_colscan.h) with split operands and fp32 outputs.  io: seed (group prefix),
// sin / sout; the transposed seeds and the states saved for a backward pass exist for 16-bit storage only.
template <int DI, int DJ, bool FUT>
__device__ __forceinline__ void split_compute_role(const ColStateIO &io, float *O_head, int ldo, int di, int dj,
                                                   const ScanRange &r, int w, int l, const u16 *sA, const u16 *sB,
                                                   const u16 *sC, u32x2 *sP) {
    using TL = Tiling<DI, DJ>;
    using CT = ColTiling<DI, DJ>;
    constexpr int KS = TL::KS, NIT = TL::NIT, NJW = CT::NJW;
    static_assert(NIT == 2 * KS && NIT % 4 == 0, "two row tiles per contraction step, row tiles in batches of four");
    const int g = l >> 4, m = l & 15;
    const bool mask_rev = r.mask_rev != 0;
    auto live = [&](int pb, int jt) __attribute__((always_inline)) { return FUT ? jt >= pb : jt <= pb; };
    const rsrc_t rO = make_rsrc(O_head, ((uint32_t)(r.N - 1) * ldo + dj) * 4u);
    int spb[3], sjt[3];  // the three score tiles of this wavefront (see col_compute_role)
    {
        const int fut_pb[12] = {0, 0, 0, 0, 1, 1, 1, 2, 2, 3, 3, 3}, fut_jt[12] = {0, 1, 2, 3, 1, 2, 3, 2, 3, 3, 3, 3};
        const int pst_pb[12] = {0, 1, 1, 2, 2, 2, 3, 3, 3, 3, 3, 3}, pst_jt[12] = {0, 0, 1, 0, 1, 2, 0, 1, 2, 3, 3, 3};
#pragma unroll
        for (int t = 0; t < 3; ++t) {
            int pbv = 0, jtv = 0;
#pragma unroll
            for (int e = 0; e < 12; ++e)
                if (e == 3 * w + t) {
                    pbv = FUT ? fut_pb[e] : pst_pb[e];
                    jtv = FUT ? fut_jt[e] : pst_jt[e];
                }
            spb[t] = __builtin_amdgcn_readfirstlane(pbv);
            sjt[t] = __builtin_amdgcn_readfirstlane(jtv);
        }
    }
    f32x4 S[NIT][NJW];
#pragma unroll
    for (int it = 0; it < NIT; ++it)
#pragma unroll
        for (int jw = 0; jw < NJW; ++jw) S[it][jw] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (io.seed != nullptr) {
        const f32x4 *gs = reinterpret_cast<const f32x4 *>(io.seed);
#pragma unroll
        for (int it = 0; it < NIT; ++it)
#pragma unroll
            for (int jw = 0; jw < NJW; ++jw) {
                const int ks = it >> 1, t = it & 1;
                S[it][jw] = gs[(size_t)((2 * ks + (g >> 1)) * TL::NJT + NJW * w + jw) * 64 + 16 * (2 * (g & 1) + t) + m];
            }
    }
    if (io.sin != nullptr) {
#pragma unroll
        for (int it = 0; it < NIT; ++it)
#pragma unroll
            for (int jw = 0; jw < NJW; ++jw)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int i = 32 * (it >> 1) + 8 * g + 4 * (it & 1) + q, j = 16 * (NJW * w + jw) + m;
                    if (i < di && j < dj) S[it][jw][q] += io.sin[(size_t)i * io.lds + j];
                }
    }
    u32x4 soph[KS][NJW], sopl[KS][NJW];
    auto pack_state = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
            for (int jw = 0; jw < NJW; ++jw) {
                u32x2 h0, l0, h1, l1;
                split4(S[2 * ks][jw], h0, l0);
                split4(S[2 * ks + 1][jw], h1, l1);
                soph[ks][jw] = cat(h0, h1);
                sopl[ks][jw] = cat(l0, l1);
            }
    };
    pack_state();
    // The (scores) x C product of a chunk is finished at the start of the NEXT chunk, after the barrier that ends this
    // one: by then every wavefront's score tiles are in LDS, and no second barrier in the middle of a chunk is needed
    // (which would hold the loader wavefronts as well).  Carried across the barrier: the partial outputs o (A_c S_c),
    // the C fragments, and the score tiles in the LDS buffer of the chunk's parity.
    u32x2 *sPh = sP, *sPl = sP + 2 * 16 * 64;  // [2 buffers][16 tiles][64 lanes], hi then lo
    f32x4 o[4][NJW];
    u32x4 cfh[NJW][2], cfl[NJW][2], pfh[4][2], pfl[4][2];
    int pbuf = 0;  // score buffer written in the current chunk
    auto read_scores_of_previous = [&]() __attribute__((always_inline)) {
        const int base = (pbuf ^ 1) * 16 * 64;
#pragma unroll
        for (int pb = 0; pb < 4; ++pb)
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                const u32x2 z = {0u, 0u};
                if (live(pb, 2 * kb) || live(pb, 2 * kb + 1)) {
                    const int t0 = base + (pb * 4 + 2 * kb) * 64 + l, t1 = t0 + 64;
                    pfh[pb][kb] = cat(live(pb, 2 * kb) ? sPh[t0] : z, live(pb, 2 * kb + 1) ? sPh[t1] : z);
                    pfl[pb][kb] = cat(live(pb, 2 * kb) ? sPl[t0] : z, live(pb, 2 * kb + 1) ? sPl[t1] : z);
                }
            }
    };
    auto finish_previous = [&](int pprev) __attribute__((always_inline)) {
        const int row0 = (r.reversed ? r.nchunks - 1 - pprev : pprev) * kChunk;
        f32x4 acc2[4][NJW];
#pragma unroll
        for (int pb = 0; pb < 4; ++pb)
#pragma unroll
            for (int jw = 0; jw < NJW; ++jw) acc2[pb][jw] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int t = 0; t < 3; ++t)
#pragma unroll
            for (int pb = 0; pb < 4; ++pb)
#pragma unroll
                for (int jw = 0; jw < NJW; ++jw) {
                    if (live(pb, 0) || live(pb, 1))
                        o[pb][jw] = mfma_term(t, cfh[jw][0], cfl[jw][0], pfh[pb][0], pfl[pb][0], o[pb][jw]);
                    if (live(pb, 2) || live(pb, 3))
                        acc2[pb][jw] = mfma_term(t, cfh[jw][1], cfl[jw][1], pfh[pb][1], pfl[pb][1], acc2[pb][jw]);
                }
#pragma unroll
        for (int pb = 0; pb < 4; ++pb)
#pragma unroll
            for (int jw = 0; jw < NJW; ++jw) {
                const f32x4 acc = o[pb][jw] + acc2[pb][jw];
                const int col = 16 * (NJW * w + jw) + 4 * g;
                const uint32_t off = (col < dj) ? (uint32_t)((row0 + 16 * pb + m) * ldo + col) * 4u : kOobOffset;
                __builtin_amdgcn_raw_buffer_store_b128(bitcast<u32x4>(acc), rO, (int)off, 0, 0);
            }
    };
    __syncthreads();
    for (int p = r.p0; p < r.p1; ++p) {
        const int buf = (p - r.p0) & 1;
        pbuf = buf;
        const u16 *cAh = sA + buf * CT::SA, *cAl = sA + (2 + buf) * CT::SA;
        const u16 *cBh = sB + buf * CT::SA, *cBl = sB + (2 + buf) * CT::SA;
        const u16 *cCh = sC + buf * CT::SC, *cCl = sC + (2 + buf) * CT::SC;
        u32x4 sqh[2][KS], sql[2][KS], skh[2][KS], skl[2][KS];
        auto read_score = [&](int slot, int t) __attribute__((always_inline)) {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const int qa = (16 * spb[t] + m) * TL::BS + 32 * ks + 8 * g, ka = (16 * sjt[t] + m) * TL::BS + 32 * ks + 8 * g;
                sqh[slot][ks] = ld128(cAh + qa);
                sql[slot][ks] = ld128(cAl + qa);
                skh[slot][ks] = ld128(cBh + ka);
                skl[slot][ks] = ld128(cBl + ka);
            }
        };
        auto score_tile = [&](int slot, int t) __attribute__((always_inline)) {
            f32x4 acc[KS];
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) acc[ks] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int t = 0; t < 3; ++t)
#pragma unroll
                for (int ks = 0; ks < KS; ++ks)
                    acc[ks] = mfma_term(t, skh[slot][ks], skl[slot][ks], sqh[slot][ks], sql[slot][ks], acc[ks]);
#pragma unroll
            for (int ks = 1; ks < KS; ++ks) acc[0] += acc[ks];
            const int d0 = 16 * (sjt[t] - spb[t]) + 4 * g - m;  // key position - query position at element 0
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const bool keep = mask_rev ? (d0 + q >= 0) : (d0 + q <= 0);
                acc[0][q] = keep ? acc[0][q] : 0.f;
            }
            u32x2 hi, lo;
            split4(acc[0], hi, lo);
            sPh[pbuf * 16 * 64 + (spb[t] * 4 + sjt[t]) * 64 + l] = hi;
            sPl[pbuf * 16 * 64 + (spb[t] * 4 + sjt[t]) * 64 + l] = lo;
        };
        u32x4 qfh[2][KS], qfl[2][KS];
        auto read_q = [&](int slot, int pb) __attribute__((always_inline)) {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                qfh[slot][ks] = ld128(cAh + (16 * pb + m) * TL::BS + 32 * ks + 8 * g);
                qfl[slot][ks] = ld128(cAl + (16 * pb + m) * TL::BS + 32 * ks + 8 * g);
            }
        };
        auto state_product = [&](int slot, int pb) __attribute__((always_inline)) {
#pragma unroll
            for (int jw = 0; jw < NJW; ++jw) {
                f32x4 acc[KS];
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) acc[ks] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int t = 0; t < 3; ++t)
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks)
                        acc[ks] = mfma_term(t, soph[ks][jw], sopl[ks][jw], qfh[slot][ks], qfl[slot][ks], acc[ks]);
#pragma unroll
                for (int ks = 1; ks < KS; ++ks) acc[0] += acc[ks];
                o[pb][jw] = acc[0];
            }
        };
        u32x4 bfh[2][4], bfl[2][4];
        auto read_c = [&]() __attribute__((always_inline)) {
#pragma unroll
            for (int jw = 0; jw < NJW; ++jw)
#pragma unroll
                for (int kb = 0; kb < 2; ++kb) {
                    const int a0 = (32 * kb + 4 * g + (m >> 2)) * TL::CS + 16 * (NJW * w + jw) + 4 * (m & 3), a1 = a0 + 16 * TL::CS;
                    cfh[jw][kb] = cat(lds_read_tr16(cCh + a0), lds_read_tr16(cCh + a1));
                    cfl[jw][kb] = cat(lds_read_tr16(cCl + a0), lds_read_tr16(cCl + a1));
                }
        };
        auto read_b = [&](int slot, int kb, int it0) __attribute__((always_inline)) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int it = it0 + e;
                const int a0 = (32 * kb + 4 * g + (m >> 2)) * TL::BS + 32 * (it >> 1) + 8 * (m & 3) + 4 * (it & 1), a1 = a0 + 16 * TL::BS;
                bfh[slot][e] = cat(lds_read_tr16(cBh + a0), lds_read_tr16(cBh + a1));
                bfl[slot][e] = cat(lds_read_tr16(cBl + a0), lds_read_tr16(cBl + a1));
            }
        };
        auto update = [&](int slot, int kb, int it0) __attribute__((always_inline)) {
#pragma unroll
            for (int t = 0; t < 3; ++t)
#pragma unroll
                for (int e = 0; e < 4; ++e)
#pragma unroll
                    for (int jw = 0; jw < NJW; ++jw)
                        S[it0 + e][jw] = mfma_term(t, bfh[slot][e], bfl[slot][e], cfh[jw][kb], cfl[jw][kb], S[it0 + e][jw]);
        };

        read_score(0, 0);
        if (p > r.p0) read_scores_of_previous();
        sched_fence();
        read_score(1, 1);
        sched_fence();
        if (p > r.p0) finish_previous(p - 1);  // (scores) x C of the chunk before, whose score tiles every wavefront has by now
        sched_fence();
        score_tile(0, 0);
        sched_fence();
        read_score(0, 2);
        sched_fence();
        score_tile(1, 1);
        sched_fence();
        read_q(0, 0);
        sched_fence();
        score_tile(0, 2);
        sched_fence();
#pragma unroll
        for (int pb = 0; pb < 4; ++pb) {
            if (pb < 3) read_q((pb + 1) & 1, pb + 1);
            else {
                read_c();
                read_b(0, 0, 0);
            }
            sched_fence();
            state_product(pb & 1, pb);
            sched_fence();
        }
        constexpr int NB = 2 * (NIT / 4);
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            if (b + 1 < NB) read_b((b + 1) & 1, (b + 1) / (NIT / 4), 4 * ((b + 1) % (NIT / 4)));
            sched_fence();
            update(b & 1, b / (NIT / 4), 4 * (b % (NIT / 4)));
            sched_fence();
        }
        pack_state();
        chunk_barrier();
    }
    if (r.p1 > r.p0) {
        pbuf = (r.p1 - r.p0) & 1;  // (finish_previous reads the other buffer: the last chunk's)
        read_scores_of_previous();
        finish_previous(r.p1 - 1);
    }
    if (io.sout != nullptr) {
#pragma unroll
        for (int it = 0; it < NIT; ++it)
#pragma unroll
            for (int jw = 0; jw < NJW; ++jw)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int i = 32 * (it >> 1) + 8 * g + 4 * (it & 1) + q, j = 16 * (NJW * w + jw) + m;
                    if (i < di && j < dj) io.sout[(size_t)i * io.lds + j] = S[it][jw][q];
                }
    }
}

// One problem per workgroup: 4 compute wavefronts, 4 loader wavefronts; grid and state slots as scan_kernel.
template <int DI, int DJ, int PF>
__global__ __launch_bounds__(512) void split_scan_kernel(ProblemSetF set, int BH, int N, int nchunks, int cpg, int G) {
    using TL = Tiling<DI, DJ>;
    using CT = ColTiling<DI, DJ>;
    __shared__ __attribute__((aligned(16))) u16 sA[4 * CT::SA];  // [hi | lo] x [2 buffers]
    __shared__ __attribute__((aligned(16))) u16 sB[4 * CT::SA];
    __shared__ __attribute__((aligned(16))) u16 sC[4 * CT::SC];
    __shared__ __attribute__((aligned(16))) u32x2 sP[2 * 2 * 16 * 64];  // masked score tiles: [hi | lo] x [2 buffers]
    const int l = threadIdx.x & 63;
    const int wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const WorkItem wi = decode_workgroup(set.count, BH, set.xcds);
    if (wi.grp >= G) return;
    const ProblemF &pr = set.p[wi.prob];
    const int di = pr.di, dj = pr.dj;
    ScanRange r;
    r.N = N;
    r.nchunks = nchunks;
    r.p0 = wi.grp * cpg;
    r.p1 = min(r.p0 + cpg, nchunks);
    r.reversed = pr.reversed;
    r.mask_rev = pr.mask_rev;
    r.comp = 0;
    if (wv >= 4) {
        split_loader_role<DI, DJ, PF, 256>(pr.A + head_base(pr.bsA, pr.hsA, pr.H, wi.bh), pr.B + head_base(pr.bsB, pr.hsB, pr.H, wi.bh),
                                           pr.C + head_base(pr.bsC, pr.hsC, pr.H, wi.bh), di, dj, pr.lda, pr.ldb, pr.ldc, r,
                                           (int)threadIdx.x - 256, sA, sB, sC);
        return;
    }
    ColStateIO io;
    if (pr.gstate != nullptr) io.seed = pr.gstate + ((size_t)wi.bh * G + wi.grp) * set.sub * TL::STATE_FLOATS;
    if (pr.sin != nullptr) io.sin = pr.sin + (size_t)wi.bh * di * pr.lds;
    if (pr.sout != nullptr && wi.grp == G - 1) io.sout = pr.sout + (size_t)wi.bh * di * pr.lds;
    io.lds = pr.lds;
    float *O_head = pr.O + head_base(pr.bsO, pr.hsO, pr.H, wi.bh);
    if (pr.mask_rev != 0)
        split_compute_role<DI, DJ, true>(io, O_head, pr.ldo, di, dj, r, wv, l, sA, sB, sC, sP);
    else
        split_compute_role<DI, DJ, false>(io, O_head, pr.ldo, di, dj, r, wv, l, sA, sB, sC, sP);
}

}  // namespace cott
