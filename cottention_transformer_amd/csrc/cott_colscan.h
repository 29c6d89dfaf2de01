// Chunk recurrence for 128-wide heads (bf16 / fp16) with the state kept out of LDS.
//
// Same op and chunk recurrence as scan_kernel (cott_mfma.h):
//     out_c = ((A_c B_c^T) o mask) C_c + A_c S_c ;   S_{c+1} = S_c + B_c^T C_c
// but with a different split of the work inside a workgroup.  In scan_kernel four state wavefronts carry S and publish
// a 16-bit copy of it in LDS every chunk (DI x DJ x 2 bytes written, and read once by each output wavefront), and two
// output wavefronts do all the products that make up out_c: with 128 x 128 states 96 KiB of LDS traffic per chunk for
// the state alone and 108 matrix instructions per chunk on each of two wavefronts.
//
// Here every compute wavefront owns DJ / 4 COLUMNS of the state, all DI rows, in its accumulators, and produces the
// same columns of out_c for all 64 positions of the chunk:
//   * A_c S_c for its columns comes straight from its own accumulators: converted to 16 bits in registers they ARE the
//     A operand of the product (see the row order below), so the state is never written to or read from LDS;
//   * the ten masked score tiles on the live side of the diagonal are formed once per workgroup, three to a
//     wavefront, and handed round through 5 KiB of LDS; the product that needs them is finished at the start of the
//     next chunk, so the one barrier per chunk covers the hand-over;
//   * the C fragments of its columns serve both the score-times-C product and the state update.
// About 86 matrix instructions per wavefront and chunk on each of the four SIMDs, and 30 % less LDS traffic.
// Four loader wavefronts stage THREE tiles per chunk (the A rows as well: all four compute wavefronts read them) and
// write the finished output tile, which the compute wavefronts leave in LDS, to memory one chunk later as 16-byte
// row segments.  All tiles double-buffered.
//
// What it buys is modest, and the measurements that say why are worth keeping next to the code.  At B1 H16 N65536
// D128 (three gradient problems per head in 5 groups, 240 workgroups) this kernel with its compute wavefronts idle,
// i.e. the loaders alone moving the launch's 1.97 GB, takes 389 us (5.1 TB/s); with all matrix instructions but no
// LDS reads in the compute wavefronts 390 us; complete 434 us (scan_kernel: 467 us; 448 us with a second barrier per chunk for
// the score tiles instead of finishing each chunk after the barrier that ends it).  Under the profiler's counter
// collection, which leaves gaps between kernels, the complete kernel takes 404 us at 2.28 GHz against 383 us at
// 2.44 GHz idle (GRBM_GUI_ACTIVE over the duration): the data path through the chip scales with the core clock, the
// core clock gives way under the power the products draw, and in a loop of back-to-back launches it gives way
// further.  Work removed from a chunk (matrix instructions, LDS traffic) therefore shows up as time even though no
// unit is saturated; prefetch depths of 3 and 4 chunks, the order of the loaders' steps and issuing the LDS reads a
// pipeline step ahead of their products change nothing.
//
// Row order of a state tile.  The matrix instruction fixes where accumulator elements live: lane (g, m) holds rows
// 4g .. 4g+3 of column m of a 16 x 16 tile.  As the A operand of the next product the same lane must hold EIGHT
// consecutive steps of the contraction (8g .. 8g+7).  The state update is therefore done with the rows of two
// neighbouring tiles interleaved: tile 2ks + t (t = 0, 1), row 4g' + q holds state row 32ks + 8g' + 4t + q, which the
// transposing LDS read delivers for free (each lane of a quarter-wave names the 8-byte piece it contributes, so the
// four column groups of a tile may lie 16 bytes apart instead of side by side).  The accumulators of tiles 2ks and
// 2ks + 1 of a lane, packed to 16 bits, are then state rows 32ks + 8g .. 32ks + 8g + 7 of column m: operand order.
// States in memory (group-state slots, states saved for a backward pass, hand-over states) keep the plain layout of
// cott_mfma.h; they are gathered into this row order when a workgroup starts and scattered back where it writes them.
#pragma once
#include "cott_mfma.h"

namespace cott {

__device__ __forceinline__ u32x4 ld128(const u16 *p) { return *reinterpret_cast<const u32x4 *>(p); }

template <int DI, int DJ>
struct ColTiling {
    static_assert(DI % 32 == 0 && DJ % 64 == 0, "padded head dims: rows a multiple of 32, columns a multiple of 64");
    using TL = Tiling<DI, DJ>;
    static constexpr int NJW = TL::NJT / 4;  // column tiles owned by one compute wavefront
    static constexpr int SA = kChunk * TL::BS, SC = kChunk * TL::CS, SO = kChunk * TL::OS;
    static constexpr int LDS_BYTES = 2 * (2 * SA + SC + SO) * 2;
};

// Loader role: LT threads move the A, B and C tiles global -> registers -> LDS, PF chunks ahead, and send the output
// tile that the compute wavefronts finished one chunk earlier (i.e. the tile of the chunk two before) from LDS to memory.  Loads and stores are unconditional
// (rows past N read as zero and are dropped on the way out: buffer range check).
template <int DI, int DJ, int PF, int LT, bool STREAM>
__device__ __forceinline__ void col_loader_role(const u16 *A_head, const u16 *B_head, const u16 *C_head, u16 *O_head, int di,
                                                int dj, int lda, int ldb, int ldc, int ldo, const ScanRange &r, int tid,
                                                u16 *sA, u16 *sB, u16 *sC, const u16 *sO) {
    using TL = Tiling<DI, DJ>;
    using CT = ColTiling<DI, DJ>;
    static_assert((8 * DI) % LT == 0 && (8 * DJ) % LT == 0, "tile vectors divide over the loader threads");
    const rsrc_t rA = make_rsrc(A_head, ((uint32_t)(r.N - 1) * lda + di) * 2u);
    const rsrc_t rB = make_rsrc(B_head, ((uint32_t)(r.N - 1) * ldb + di) * 2u);
    const rsrc_t rC = make_rsrc(C_head, ((uint32_t)(r.N - 1) * ldc + dj) * 2u);
    const rsrc_t rO = make_rsrc(O_head, ((uint32_t)(r.N - 1) * ldo + dj) * 2u);
    auto write_out = [&](int p) __attribute__((always_inline)) {
        const int row0 = (r.reversed ? r.nchunks - 1 - p : p) * kChunk;
        const u16 *tile = sO + ((p - r.p0) & 1) * CT::SO;
#pragma unroll
        for (int u = 0; u < 8 * DJ / LT; ++u) {
            const int v = tid + LT * u;
            const int row = v / (DJ / 8), col = (v % (DJ / 8)) * 8;
            const u32x4 val = *reinterpret_cast<const u32x4 *>(tile + row * TL::OS + col);
            const uint32_t off = (col < dj) ? (uint32_t)((row0 + row) * ldo + col) * 2u : kOobOffset;
            __builtin_amdgcn_raw_buffer_store_b128(val, rO, (int)off, 0, 0);
        }
    };
    u32x4 ra[PF][8 * DI / LT], rb[PF][8 * DI / LT], rc[PF][8 * DJ / LT];
    auto load_chunk = [&](int s, int p) __attribute__((always_inline)) {
        const int pc = min(p, r.p1 - 1);
        const int row0 = (r.reversed ? r.nchunks - 1 - pc : pc) * kChunk;
        load_tile<DI, LT, STREAM>(ra[s], rA, row0, lda, tid);
        load_tile<DI, LT, STREAM>(rb[s], rB, row0, ldb, tid);
        load_tile<DJ, LT, STREAM>(rc[s], rC, row0, ldc, tid);
    };
#pragma unroll
    for (int s = 0; s < PF; ++s) load_chunk(s, r.p0 + s);
    store_tile<DI, TL::BS, LT>(sA, ra[0], di, tid);
    store_tile<DI, TL::BS, LT>(sB, rb[0], di, tid);
    store_tile<DJ, TL::CS, LT>(sC, rc[0], dj, tid);
    load_chunk(0, r.p0 + PF);
    __syncthreads();
    run_rounds<PF>(r.p0, r.p1, [&](int s, int p) __attribute__((always_inline)) {
        const int s1 = (s + 1) % PF;
        const int buf = (p - r.p0) & 1;
        store_tile<DI, TL::BS, LT>(sA + (buf ^ 1) * CT::SA, ra[s1], di, tid);
        store_tile<DI, TL::BS, LT>(sB + (buf ^ 1) * CT::SA, rb[s1], di, tid);
        store_tile<DJ, TL::CS, LT>(sC + (buf ^ 1) * CT::SC, rc[s1], dj, tid);
        load_chunk(s1, p + 1 + PF);
        if (p > r.p0 + 1) write_out(p - 2);  // (the compute wavefronts finish a chunk's tile at the start of the next chunk)
        chunk_barrier();
    });
    if (r.p1 > r.p0 + 1) write_out(r.p1 - 2);
    __syncthreads();  // the last chunk's tile is finished after the loop
    if (r.p1 > r.p0) write_out(r.p1 - 1);
}

// Loader role with the input preparation folded in (PrepSide, cott_mfma.h): A, B, C are the RAW q, k, v projections; every
// 16-byte piece is rotated / normalised (q, k) or scaled / masked (v) between the registers and the LDS tiles, and the
// prepared rows also go to qo / ko / vo for the backward pass.  A row of DI columns lives in DI / 8 consecutive loader
// lanes, which reduce its squared norm among themselves; the A and B pieces of a thread have the same row and columns
// and share their rotary table entries.  Side inputs (keep, count, table entries) travel with the pieces, PF chunks
// ahead; position ids one call earlier than the table entries they select.  first_half: this workgroup writes qo and
// ko (the two column halves of a head prepare the same q and k rows).
// SUMS: the group-state pass of such a forward (colsum_prep_kernel): only the B and C tiles are loaded, prepared and staged,
// nothing is written to memory (the scan that follows leaves the prepared rows).
template <class TR, int DI, int DJ, int PF, int LT, bool SUMS = false>
__device__ __forceinline__ void col_loader_role_prep(const u16 *A_head, const u16 *B_head, const u16 *C_head, u16 *O_head,
                                                     int di, int dj, int lda, int ldb, int ldc, int ldo, const ScanRange &r,
                                                     int tid, u16 *sA, u16 *sB, u16 *sC, const u16 *sO, const PrepSide &ps,
                                                     int bh, int c0, bool first_half) {
    using TL = Tiling<DI, DJ>;
    using CT = ColTiling<DI, DJ>;
    constexpr int NB = 8 * DI / LT, NC = 8 * DJ / LT;
    static_assert((8 * DI) % LT == 0 && (8 * DJ) % LT == 0, "tile vectors divide over the loader threads");
    const rsrc_t rA = make_rsrc(A_head, ((uint32_t)(r.N - 1) * lda + di) * 2u);
    const rsrc_t rB = make_rsrc(B_head, ((uint32_t)(r.N - 1) * ldb + di) * 2u);
    const rsrc_t rC = make_rsrc(C_head, ((uint32_t)(r.N - 1) * ldc + dj) * 2u);
    const rsrc_t rO = make_rsrc(O_head, ((uint32_t)(r.N - 1) * ldo + dj) * 2u);
    const uint32_t qk_bytes = first_half ? (uint32_t)r.N * di * 2u : 0u;
    const rsrc_t rQo = make_rsrc(ps.qo ? ps.qo + (size_t)bh * r.N * di : nullptr, ps.qo ? qk_bytes : 0u);
    const rsrc_t rKo = make_rsrc(ps.ko ? ps.ko + (size_t)bh * r.N * di : nullptr, ps.ko ? qk_bytes : 0u);
    const rsrc_t rVo = make_rsrc(ps.vo ? ps.vo + (size_t)bh * r.N * ps.dv + c0 : nullptr,
                                 ps.vo ? ((uint32_t)(r.N - 1) * ps.dv + dj) * 2u : 0u);
    const size_t tok0 = (size_t)(bh / ps.H) * r.N;
    const bool scaled = ps.cnt != nullptr && ps.sig != nullptr;
    const float sig = scaled ? ps.sig[bh % ps.H] : 0.f;
    auto write_out = [&](int p) __attribute__((always_inline)) {
        const int row0 = (r.reversed ? r.nchunks - 1 - p : p) * kChunk;
        const u16 *tile = sO + ((p - r.p0) & 1) * CT::SO;
#pragma unroll
        for (int u = 0; u < NC; ++u) {
            const int v = tid + LT * u;
            const int row = v / (DJ / 8), col = (v % (DJ / 8)) * 8;
            const u32x4 val = *reinterpret_cast<const u32x4 *>(tile + row * TL::OS + col);
            const uint32_t off = (col < dj) ? (uint32_t)((row0 + row) * ldo + col) * 2u : kOobOffset;
            __builtin_amdgcn_raw_buffer_store_b128(val, rO, (int)off, 0, 0);
        }
    };
    u32x4 ra[PF][NB], rb[PF][NB], rc[PF][NC];
    f32x4 sn[PF][NB], cs[PF][NB];
    uint32_t keep_ab[PF][NB], keep_c[PF][NC];  // the bytes as loaded: converting them here would wait for the load
    float cnt_c[PF][NC];
    auto row0_of = [&](int p) __attribute__((always_inline)) {
        const int pc = min(p, r.p1 - 1);
        return (r.reversed ? r.nchunks - 1 - pc : pc) * kChunk;
    };
    const bool has_pos = ps.pos != nullptr && ps.rot != nullptr;
    const rsrc_t rPos = make_rsrc_uniform(has_pos ? ps.pos + tok0 : nullptr, has_pos ? (uint32_t)r.N * 8u : 0u);
    u32x2 pnext[NB];
    auto fetch_positions = [&](int p) __attribute__((always_inline)) {
        const int row0 = row0_of(p);
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            const int srow = min(row0 + (tid + LT * u) / (DI / 8), r.N - 1);
            pnext[u] = __builtin_amdgcn_raw_buffer_load_b64(rPos, (int)((uint32_t)srow * 8u), 0, 0);
        }
    };
    fetch_positions(r.p0);
    auto load_chunk = [&](int s, int p) __attribute__((always_inline)) {
        const int row0 = row0_of(p);
        int trow[NB];
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            const int srow = min(row0 + (tid + LT * u) / (DI / 8), r.N - 1);
            const long long given = (long long)(((unsigned long long)pnext[u].y << 32) | pnext[u].x);
            trow[u] = clamp_row(ps, has_pos ? given : ps.pos0 + srow);
        }
        fetch_positions(p + 1);
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            const int v = tid + LT * u;
            const int row = row0 + v / (DI / 8), col = (v % (DI / 8)) * 8;
            if constexpr (!SUMS) ra[s][u] = buf_load16(rA, (uint32_t)(row * lda + col) * 2u);
            rb[s][u] = buf_load16(rB, (uint32_t)(row * ldb + col) * 2u);
            const int srow = min(row, r.N - 1);
            keep_ab[s][u] = ps.keep != nullptr ? (uint32_t)ps.keep[tok0 + srow] : 1u;
            if (ps.rot != nullptr && col < ps.R) {
                const float *t = ps.rot + (size_t)trow[u] * ps.R + col / 2;
                sn[s][u] = *reinterpret_cast<const f32x4 *>(t);
                cs[s][u] = *reinterpret_cast<const f32x4 *>(t + ps.R / 2);
            }
        }
#pragma unroll
        for (int u = 0; u < NC; ++u) {
            const int v = tid + LT * u;
            const int row = row0 + v / (DJ / 8), col = (v % (DJ / 8)) * 8;
            rc[s][u] = buf_load16(rC, (uint32_t)(row * ldc + col) * 2u);
            const int srow = min(row, r.N - 1);
            keep_c[s][u] = ps.keep != nullptr ? (uint32_t)ps.keep[tok0 + srow] : 1u;
            cnt_c[s][u] = scaled ? ps.cnt[tok0 + srow] : 0.f;
        }
    };
    // registers of stage s (chunk p) -> prepared tiles in the LDS buffers ta, tb, tc and in qo / ko / vo
    auto stage = [&](int s, int p, u16 *ta, u16 *tb, u16 *tc) __attribute__((always_inline)) {
        const int row0 = row0_of(p);
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            const int v = tid + LT * u;
            const int lrow = v / (DI / 8), col = (v % (DI / 8)) * 8;
            const bool rotate = ps.rot != nullptr && col < ps.R;
            const u32x4 yb = prep_qk_piece<TR, DI / 8>(rb[s][u], col, di, rotate, sn[s][u], cs[s][u], (float)keep_ab[s][u], ps.eps);
            *reinterpret_cast<u32x4 *>(tb + lrow * TL::BS + col) = yb;
            if constexpr (!SUMS) {
                const u32x4 ya = prep_qk_piece<TR, DI / 8>(ra[s][u], col, di, rotate, sn[s][u], cs[s][u], (float)keep_ab[s][u], ps.eps);
                *reinterpret_cast<u32x4 *>(ta + lrow * TL::BS + col) = ya;
                const uint32_t off = (col < di && p < r.p1) ? (uint32_t)((row0 + lrow) * di + col) * 2u : kOobOffset;
                __builtin_amdgcn_raw_buffer_store_b128(ya, rQo, (int)off, 0, 0);
                __builtin_amdgcn_raw_buffer_store_b128(yb, rKo, (int)off, 0, 0);
            }
        }
#pragma unroll
        for (int u = 0; u < NC; ++u) {
            const int v = tid + LT * u;
            const int lrow = v / (DJ / 8), col = (v % (DJ / 8)) * 8;
            const u32x4 y = prep_v_piece<TR>(rc[s][u], col < dj, (float)keep_c[s][u], cnt_c[s][u], sig, scaled);
            *reinterpret_cast<u32x4 *>(tc + lrow * TL::CS + col) = y;
            if constexpr (!SUMS) {
                const uint32_t off = (col < dj && p < r.p1) ? (uint32_t)((row0 + lrow) * ps.dv + col) * 2u : kOobOffset;
                __builtin_amdgcn_raw_buffer_store_b128(y, rVo, (int)off, 0, 0);
            }
        }
    };
#pragma unroll
    for (int s = 0; s < PF; ++s) load_chunk(s, r.p0 + s);
    stage(0, r.p0, sA, sB, sC);
    load_chunk(0, r.p0 + PF);
    __syncthreads();
    run_rounds<PF>(r.p0, r.p1, [&](int s, int p) __attribute__((always_inline)) {
        const int s1 = (s + 1) % PF;
        const int buf = (p - r.p0) & 1;
        stage(s1, p + 1, sA + (buf ^ 1) * CT::SA, sB + (buf ^ 1) * CT::SA, sC + (buf ^ 1) * CT::SC);
        load_chunk(s1, p + 1 + PF);
        if constexpr (!SUMS)
            if (p > r.p0 + 1) write_out(p - 2);
        chunk_barrier();
    });
    if constexpr (!SUMS)
        if (r.p1 > r.p0 + 1) write_out(r.p1 - 2);
    __syncthreads();
    if constexpr (!SUMS)
        if (r.p1 > r.p0) write_out(r.p1 - 1);
}

// Where the compute wavefront `w` of a workgroup finds and leaves its state (all pointers already at this head, and
// group where that applies; any may be null).
struct ColStateIO {
    const float *seed = nullptr;      // group prefix, plain tile layout with DJ / 16 tiles per tile row
    const float *seed_t = nullptr;    // the TRANSPOSE of this state in the plain tile layout, seed_t_njt tiles per tile row
    int seed_t_njt = 0;
    const float *sin = nullptr;       // row-major [di][lds] hand-over state to start from
    float *sout = nullptr;            // ... and to leave at the end (last group only)
    int lds = 0;
    float *sums = nullptr;            // SUMS: where the sum of B^T C over the chunks walked goes, plain tile layout
    float *save = nullptr;            // states for a backward pass (ProblemT::save): first slot of this head
    int save_njt = 0, save_jt0 = 0, save_slot = 0, save_cpg = 1, save_n = 0;
};

// Compute role: wavefront w of 4 owns column tiles NJW * w .. NJW * w + NJW - 1.  FUT: the scores that count are
// those of keys at or after the query (ops that sum over the future, or over the past in complement form).
// The ten score tiles on the live side of the diagonal are dealt three to a wavefront (the last wavefront forms its
// one tile three times) and left in LDS (sP: 16 tiles of 512 bytes in accumulator order, which is operand order for the
// next product, double-buffered); every wavefront reads the tiles of all blocks after the barrier that ends the chunk
// and finishes the chunk's outputs then, before it starts on the next chunk.
// The chunk is written as a software pipeline: the LDS reads of step k + 1 are issued, as a block, before the matrix
// instructions of step k, and scheduling fences keep the compiler from sinking them back down to their first use
// (left to itself it places every read a few instructions before the product that needs it, and the wavefront then
// pays the full LDS latency some forty times per chunk).
__device__ __forceinline__ void sched_fence() { __builtin_amdgcn_sched_barrier(0); }

// SUMS: only the state update runs, from a zero state, and the sum is left in io.sums (colsum_prep_kernel).
template <class TR, int DI, int DJ, bool FUT, bool SUMS = false>
__device__ __forceinline__ void col_compute_role(const ColStateIO &io, int di, int dj, const ScanRange &r, int w, int l,
                                                   const u16 *sA, const u16 *sB, const u16 *sC, u16 *sO, u32x2 *sP) {
    using TL = Tiling<DI, DJ>;
    using CT = ColTiling<DI, DJ>;
    constexpr int KS = TL::KS, NIT = TL::NIT, NJW = CT::NJW;
    static_assert(NIT == 2 * KS && NIT % 4 == 0, "two row tiles per contraction step, row tiles in batches of four");
    const int g = l >> 4, m = l & 15;
    const bool mask_rev = r.mask_rev != 0, comp = r.comp != 0;
    auto live = [&](int pb, int jt) __attribute__((always_inline)) { return FUT ? jt >= pb : jt <= pb; };
    // score tiles of this wavefront: (position block, key tile), four bits each, three per wavefront
    //   FUT:  w0 (0,0) (0,1) (0,2)   w1 (0,3) (1,1) (1,2)   w2 (1,3) (2,2) (2,3)   w3 (3,3) x 3
    //   else: w0 (0,0) (1,0) (1,1)   w1 (2,0) (2,1) (2,2)   w2 (3,0) (3,1) (3,2)   w3 (3,3) x 3
    int spb[3], sjt[3];
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
    auto plain_index = [&](int it, int jt, int njt) __attribute__((always_inline)) {
        const int ks = it >> 1, t = it & 1;
        return (size_t)((2 * ks + (g >> 1)) * njt + jt) * 64 + 16 * (2 * (g & 1) + t) + m;
    };
    if (io.seed != nullptr) {
        const f32x4 *gs = reinterpret_cast<const f32x4 *>(io.seed);
#pragma unroll
        for (int it = 0; it < NIT; ++it)
#pragma unroll
            for (int jw = 0; jw < NJW; ++jw) S[it][jw] = gs[plain_index(it, NJW * w + jw, TL::NJT)];
    }
    if (io.seed_t != nullptr) {
        float *scr = reinterpret_cast<float *>(sO) + w * 512;
        const f32x4 *src = reinterpret_cast<const f32x4 *>(io.seed_t);
#pragma unroll
        for (int jw = 0; jw < NJW; ++jw) {
            const int jt = NJW * w + jw;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const f32x4 t0 = src[(size_t)(jt * io.seed_t_njt + 2 * ks) * 64 + l];
                const f32x4 t1 = src[(size_t)(jt * io.seed_t_njt + 2 * ks + 1) * 64 + l];
                *reinterpret_cast<f32x4 *>(scr + 4 * l) = t0;
                *reinterpret_cast<f32x4 *>(scr + 256 + 4 * l) = t1;
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const int i = 32 * ks + 8 * g + 4 * t + q;
                        const float x = scr[(g >> 1) * 256 + (16 * (m >> 2) + ((8 * g + 4 * t) & 15) + q) * 4 + (m & 3)];
                        if (i < di && 16 * jt + m < dj) S[2 * ks + t][jw][q] += x;
                    }
            }
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
    u32x4 sop[KS][NJW];
    auto pack_state = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
            for (int jw = 0; jw < NJW; ++jw)
                sop[ks][jw] = u32x4{TR::pack2(S[2 * ks][jw][0], S[2 * ks][jw][1]), TR::pack2(S[2 * ks][jw][2], S[2 * ks][jw][3]),
                                    TR::pack2(S[2 * ks + 1][jw][0], S[2 * ks + 1][jw][1]),
                                    TR::pack2(S[2 * ks + 1][jw][2], S[2 * ks + 1][jw][3])};
    };
    pack_state();
    const uint32_t flip = comp ? 0x80008000u : 0u;
    // The (scores) x C product of a chunk is finished at the start of the NEXT chunk, after the barrier that ends this
    // one: by then every wavefront's score tiles are in LDS, and no second barrier in the middle of a chunk is needed
    // (which would hold the loader wavefronts as well).  Carried across the barrier: the partial outputs o (A_c S_c),
    // the C fragments, and the score tiles in the LDS buffer of the chunk's parity.
    f32x4 o[4][NJW];
    u32x4 cf[NJW][2];
    auto finish = [&](int pbuf) __attribute__((always_inline)) {  // adds (scores) x C to o and leaves the tile in the staging buffer of that chunk
        const u32x2 *tiles = sP + pbuf * 16 * 64;
        u16 *cO = sO + pbuf * CT::SO;
        u32x4 pf[2][2];  // the score tiles of a block are read one block ahead of their products
        auto read_block = [&](int slot, int pb) __attribute__((always_inline)) {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                const u32x2 z = {0u, 0u};
                if (live(pb, 2 * kb) || live(pb, 2 * kb + 1))
                    pf[slot][kb] = cat(live(pb, 2 * kb) ? tiles[(pb * 4 + 2 * kb) * 64 + l] : z,
                                       live(pb, 2 * kb + 1) ? tiles[(pb * 4 + 2 * kb + 1) * 64 + l] : z);
            }
        };
        read_block(0, 0);
        sched_fence();
#pragma unroll
        for (int pb = 0; pb < 4; ++pb) {
            if (pb < 3) read_block((pb + 1) & 1, pb + 1);
            sched_fence();
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                if (!(live(pb, 2 * kb) || live(pb, 2 * kb + 1))) continue;
#pragma unroll
                for (int jw = 0; jw < NJW; ++jw) o[pb][jw] = TR::mfma(cf[jw][kb], pf[pb & 1][kb], o[pb][jw]);
            }
#pragma unroll
            for (int jw = 0; jw < NJW; ++jw)
                *reinterpret_cast<u32x2 *>(cO + (16 * pb + m) * TL::OS + 16 * (NJW * w + jw) + 4 * g) =
                    u32x2{TR::pack2(o[pb][jw][0], o[pb][jw][1]), TR::pack2(o[pb][jw][2], o[pb][jw][3])};
            sched_fence();
        }
    };
    __syncthreads();
    for (int p = r.p0; p < r.p1; ++p) {
        const int buf = (p - r.p0) & 1;
        const u16 *cA = sA + buf * CT::SA, *cB = sB + buf * CT::SA, *cC = sC + buf * CT::SC;
        u32x2 *cP = sP + buf * 16 * 64;
        // fragment readers (each a block of LDS reads, nothing else)
        u32x4 sq[2][KS], sk[2][KS];  // query rows and key rows of a score tile, two tiles in flight
        auto read_score = [&](int slot, int t) __attribute__((always_inline)) {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                sq[slot][ks] = ld128(cA + (16 * spb[t] + m) * TL::BS + 32 * ks + 8 * g);
                sk[slot][ks] = ld128(cB + (16 * sjt[t] + m) * TL::BS + 32 * ks + 8 * g);
            }
        };
        auto score_tile = [&](int slot, int t) __attribute__((always_inline)) {
            f32x4 a0 = {0.f, 0.f, 0.f, 0.f}, a1 = a0;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                if (ks & 1) a1 = TR::mfma(sk[slot][ks], sq[slot][ks], a1);
                else a0 = TR::mfma(sk[slot][ks], sq[slot][ks], a0);
            }
            f32x4 acc = a0 + a1;
            const int d0 = 16 * (sjt[t] - spb[t]) + 4 * g - m;  // key position - query position at element 0
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const bool keep = mask_rev ? (d0 + q >= 0) : (d0 + q <= 0);
                acc[q] = (keep != comp) ? (comp ? -acc[q] : acc[q]) : 0.f;
            }
            cP[(spb[t] * 4 + sjt[t]) * 64 + l] = u32x2{TR::pack2(acc[0], acc[1]), TR::pack2(acc[2], acc[3])};
        };
        u32x4 qf[2][KS];
        auto read_q = [&](int slot, int pb) __attribute__((always_inline)) {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) qf[slot][ks] = ld128(cA + (16 * pb + m) * TL::BS + 32 * ks + 8 * g);
        };
        auto state_product = [&](int slot, int pb) __attribute__((always_inline)) {  // out^T tiles (columns 16jt + 4g .. + 3, position 16pb + m)
#pragma unroll
            for (int jw = 0; jw < NJW; ++jw) {
                f32x4 o1 = {0.f, 0.f, 0.f, 0.f}, o2 = o1;
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    if (ks & 1) o2 = TR::mfma(sop[ks][jw], qf[slot][ks], o2);
                    else o1 = TR::mfma(sop[ks][jw], qf[slot][ks], o1);
                }
                o[pb][jw] = o1 + o2;
            }
        };
        u32x4 bf[2][4];
        auto read_c = [&]() __attribute__((always_inline)) {
#pragma unroll
            for (int jw = 0; jw < NJW; ++jw)
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
                    cf[jw][kb] = cat(lds_read_tr16(cC + (32 * kb + 4 * g + (m >> 2)) * TL::CS + 16 * (NJW * w + jw) + 4 * (m & 3)),
                                     lds_read_tr16(cC + (32 * kb + 16 + 4 * g + (m >> 2)) * TL::CS + 16 * (NJW * w + jw) + 4 * (m & 3)));
        };
        auto read_b = [&](int slot, int kb, int it0) __attribute__((always_inline)) {  // B^T fragments of row tiles it0 .. it0 + 3, rows interleaved
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int it = it0 + e;
                const int c = 32 * (it >> 1) + 8 * (m & 3) + 4 * (it & 1);
                bf[slot][e] = cat(lds_read_tr16(cB + (32 * kb + 4 * g + (m >> 2)) * TL::BS + c),
                                  lds_read_tr16(cB + (32 * kb + 16 + 4 * g + (m >> 2)) * TL::BS + c));
            }
        };
        auto update = [&](int slot, int kb, int it0) __attribute__((always_inline)) {  // S += B_c^T C_c (complement form: -=)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const u32x4 b = bf[slot][e] ^ u32x4{flip, flip, flip, flip};
#pragma unroll
                for (int jw = 0; jw < NJW; ++jw) S[it0 + e][jw] = TR::mfma(b, cf[jw][kb], S[it0 + e][jw]);
            }
        };

        if constexpr (SUMS) {
            read_c();
            read_b(0, 0, 0);
            sched_fence();
            constexpr int NBS = 2 * (NIT / 4);
#pragma unroll
            for (int b = 0; b < NBS; ++b) {
                if (b + 1 < NBS) read_b((b + 1) & 1, (b + 1) / (NIT / 4), 4 * ((b + 1) % (NIT / 4)));
                sched_fence();
                update(b & 1, b / (NIT / 4), 4 * (b % (NIT / 4)));
                sched_fence();
            }
            chunk_barrier();
            continue;
        }
        if (p > r.p0) finish(buf ^ 1);
        read_score(0, 0);
        sched_fence();
        read_score(1, 1);
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
        constexpr int NB = 2 * (NIT / 4);  // batches of four row tiles over the two key halves
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            if (b + 1 < NB) read_b((b + 1) & 1, (b + 1) / (NIT / 4), 4 * ((b + 1) % (NIT / 4)));
            sched_fence();
            update(b & 1, b / (NIT / 4), 4 * (b % (NIT / 4)));
            sched_fence();
        }
        pack_state();
        if (io.save != nullptr) {  // (an op that walks forwards: p is the chunk's place in the sequence)
            const int back = r.nchunks - 1 - p;
            if (back % io.save_cpg == 0 && back / io.save_cpg < io.save_n) {
                f32x4 *dst = reinterpret_cast<f32x4 *>(io.save + (size_t)(back / io.save_cpg) * io.save_slot);
#pragma unroll
                for (int it = 0; it < NIT; ++it)
#pragma unroll
                    for (int jw = 0; jw < NJW; ++jw)
                        if (16 * (NJW * w + jw) < dj) dst[plain_index(it, io.save_jt0 + NJW * w + jw, io.save_njt)] = S[it][jw];
            }
        }
        chunk_barrier();
    }
    if constexpr (!SUMS) {
        if (r.p1 > r.p0) finish((r.p1 - 1 - r.p0) & 1);
    }
    __syncthreads();  // (the loader wavefronts send the last tile out after this)
    if constexpr (SUMS) {
        f32x4 *dst = reinterpret_cast<f32x4 *>(io.sums);
#pragma unroll
        for (int it = 0; it < NIT; ++it)
#pragma unroll
            for (int jw = 0; jw < NJW; ++jw) dst[plain_index(it, NJW * w + jw, TL::NJT)] = S[it][jw];
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

// One problem per workgroup: 4 compute wavefronts, 4 loader wavefronts.  Same grid, problem set and state slots as
// scan_kernel.
// PREP: q, k, v are the raw projections and are prepared inside the kernel (PrepSide; forward direction).
template <class TR, int DI, int DJ, int PF, bool STREAM, bool PREP = false>
__global__ __launch_bounds__(512) void colscan_kernel(ProblemSet set, int BH, int N, int nchunks, int cpg, int G,
                                                      PrepSide prep) {
    using TL = Tiling<DI, DJ>;
    using CT = ColTiling<DI, DJ>;
    __shared__ __attribute__((aligned(16))) u16 sA[2 * CT::SA];
    __shared__ __attribute__((aligned(16))) u16 sB[2 * CT::SA];
    __shared__ __attribute__((aligned(16))) u16 sC[2 * CT::SC];
    __shared__ __attribute__((aligned(16))) u16 sO[2 * CT::SO];
    __shared__ __attribute__((aligned(16))) u32x2 sP[2 * 16 * 64];  // masked score tiles of the current and the previous chunk
    static_assert(2 * CT::SO * 2 >= 4 * 2048, "room to turn the transposed seeds");
    const int l = threadIdx.x & 63;
    const int wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const WorkItem wi = decode_workgroup(set.count, BH, set.xcds);
    if (wi.grp >= G) return;
    const Problem &pr = set.p[wi.prob];
    const int di = pr.di, dj = pr.dj;
    ScanRange r;
    r.N = N;
    r.nchunks = nchunks;
    r.p0 = wi.grp * cpg;
    r.p1 = min(r.p0 + cpg, nchunks);
    r.reversed = pr.reversed;
    r.mask_rev = pr.mask_rev;
    r.comp = pr.comp;
    if (wv >= 4) {
        if constexpr (PREP) {
            col_loader_role_prep<TR, DI, DJ, PF, 256>(pr.A + head_base(pr.bsA, pr.hsA, pr.H, wi.bh),
                                                      pr.B + head_base(pr.bsB, pr.hsB, pr.H, wi.bh),
                                                      pr.C + head_base(pr.bsC, pr.hsC, pr.H, wi.bh),
                                                      pr.O + head_base(pr.bsO, pr.hsO, pr.H, wi.bh), di, dj, pr.lda, pr.ldb,
                                                      pr.ldc, pr.ldo, r, (int)threadIdx.x - 256, sA, sB, sC, sO, prep, wi.bh,
                                                      pr.c0, pr.c0 == 0);
            return;
        }
        col_loader_role<DI, DJ, PF, 256, STREAM>(pr.A + head_base(pr.bsA, pr.hsA, pr.H, wi.bh),
                                                 pr.B + head_base(pr.bsB, pr.hsB, pr.H, wi.bh),
                                                 pr.C + head_base(pr.bsC, pr.hsC, pr.H, wi.bh),
                                                 pr.O + head_base(pr.bsO, pr.hsO, pr.H, wi.bh), di, dj, pr.lda, pr.ldb, pr.ldc,
                                                 pr.ldo, r, (int)threadIdx.x - 256, sA, sB, sC, sO);
        return;
    }
    ColStateIO io;
    const size_t slot = ((size_t)wi.bh * G + wi.grp) * set.sub * TL::STATE_FLOATS;
    if (pr.ext != nullptr) {  // the state the forward pass saved at this group's cut is this one's transpose
        io.seed_t = pr.ext + ((size_t)wi.bh * G + wi.grp) * pr.save_slot;
        io.seed_t_njt = pr.save_njt;
    } else if (pr.seed_from >= 0) {  // the twin problem's group prefix, transposed (square padded dims)
        if (set.p[pr.seed_from].gstate != nullptr) {
            io.seed_t = set.p[pr.seed_from].gstate + slot;
            io.seed_t_njt = TL::NIT;
        }
    } else if (pr.gstate != nullptr) {
        io.seed = pr.gstate + slot;
    }
    if (pr.sin != nullptr) io.sin = pr.sin + (size_t)wi.bh * di * pr.lds;
    if (pr.sout != nullptr && wi.grp == G - 1) io.sout = pr.sout + (size_t)wi.bh * di * pr.lds;
    io.lds = pr.lds;
    if (pr.save != nullptr) {
        io.save = pr.save + (size_t)wi.bh * pr.save_n * pr.save_slot;
        io.save_njt = pr.save_njt;
        io.save_jt0 = pr.c0 / 16;
        io.save_slot = pr.save_slot;
        io.save_cpg = pr.save_cpg;
        io.save_n = pr.save_n;
    }
    if ((pr.mask_rev != 0) != (pr.comp != 0))
        col_compute_role<TR, DI, DJ, true>(io, di, dj, r, wv, l, sA, sB, sC, sO, sP);
    else
        col_compute_role<TR, DI, DJ, false>(io, di, dj, r, wv, l, sA, sB, sC, sO, sP);
}

// The group-state pass of a forward that prepares its inputs itself, for 128-wide q / k rows: sum of k_hat^T v_hat over
// each piece of each group of chunks, with the roles of colscan_kernel: four loader wavefronts prepare and stage the k and
// v tiles, four compute wavefronts each keep a quarter of the sum's columns.  Same grid, pieces and slots as
// group_state_kernel, whose single role does all of this (N = 65536, 16 heads: 299 us there).
template <class TR, int DI, int DJ, int PF>
__global__ __launch_bounds__(512) void colsum_prep_kernel(ProblemSet set, int BH, int N, int nchunks, int cpg, int G,
                                                          int ngroups, PrepSide prep) {
    using TL = Tiling<DI, DJ>;
    using CT = ColTiling<DI, DJ>;
    __shared__ __attribute__((aligned(16))) u16 sB[2 * CT::SA];
    __shared__ __attribute__((aligned(16))) u16 sC[2 * CT::SC];
    const int l = threadIdx.x & 63;
    const int wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int sub = set.sub;
    const WorkItem wi = decode_workgroup(set.nact * sub, BH, set.xcds);
    if (wi.grp >= ngroups) return;
    const Problem &pr = set.p[set.act[wi.prob / sub]];
    const int grp = wi.grp, piece = wi.prob % sub;
    if (grp == G - 1 && ngroups == G && !pr.comp) return;
    if (pr.seed_from >= 0 || pr.ext != nullptr) return;
    const int cps = (cpg + sub - 1) / sub;  // chunks per piece
    ScanRange r;
    r.N = N;
    r.nchunks = nchunks;
    r.p0 = grp * cpg + piece * cps;
    r.p1 = min(r.p0 + cps, min((grp + 1) * cpg, nchunks));
    r.reversed = pr.reversed;
    r.mask_rev = pr.mask_rev;
    r.comp = 0;
    float *slot = pr.gstate + (((size_t)wi.bh * G + grp) * sub + piece) * TL::STATE_FLOATS;
    if (r.p1 <= r.p0) {  // a piece past the end of its group: its slot is zero
        for (int e = threadIdx.x; e < TL::STATE_FLOATS / 4; e += 512) reinterpret_cast<f32x4 *>(slot)[e] = f32x4{0.f, 0.f, 0.f, 0.f};
        return;
    }
    if (wv >= 4) {
        col_loader_role_prep<TR, DI, DJ, PF, 256, true>(nullptr, pr.B + head_base(pr.bsB, pr.hsB, pr.H, wi.bh),
                                                        pr.C + head_base(pr.bsC, pr.hsC, pr.H, wi.bh), nullptr, pr.di, pr.dj,
                                                        pr.lda, pr.ldb, pr.ldc, pr.ldo, r, (int)threadIdx.x - 256, nullptr, sB,
                                                        sC, nullptr, prep, wi.bh, pr.c0, false);
        return;
    }
    ColStateIO io;
    io.sums = slot;
    col_compute_role<TR, DI, DJ, false, true>(io, pr.di, pr.dj, r, wv, l, nullptr, sB, sC, nullptr, nullptr);
}

}  // namespace cott
