// Chunked-scan kernels for 16-bit storage types (bf16 / fp16) on gfx950 MFMA.
//
// Generic op (per batch*head):  out[s,j] = sum_i A[s,i] * sum_{s' <= s (>= s if reversed)} B[s',i] C[s',j]
// restructured over chunks of 64 positions (scan order p, state S[i][j] carried in fp32):
//     out_c = ((A_c B_c^T) o mask) C_c + A_c S_c ;   S_{c+1} = S_c + B_c^T C_c
//
// One launch runs a SET of such problems over the same (BH, N) grid -- the two column halves of a
// forward pass, or the three gradients dQ = G(dO,V,K), dK = G(V,dO,Q,rev), dV = G(K,Q,dO,rev).  The
// workgroups that work on the same head are placed on the same XCD and start together, so an
// operand shared between problems (Q and K of the two halves; Q, K, V, dO of the gradients) comes
// from HBM once and from that XCD's L2 afterwards.
//
// When B*H alone cannot fill the chip the sequence of one head is also cut into G groups of
// consecutive chunks: group_state_kernel sums B^T C over each group, state_prefix_kernel turns the
// per-group sums into exclusive prefixes, scan_kernel runs the recurrence seeded with its prefix.
#pragma once
#include "cott_common.h"
#include <type_traits>

namespace cott {

constexpr int kChunk = 64;     // positions per chunk
constexpr int kThreads = 256;  // 4 wavefronts per workgroup
constexpr int kMaxProblems = 6;
constexpr int kWaveStageStride = 64 + 8;  // elements per row of an output wavefront's own staging tile [16 IB][64]

// One generic op.  A, B: rows of `di` elements, contiguous.  C, O: `dj` columns taken from rows of
// `ldc` elements (the pointers already include the first column), so a problem can own a column
// slice of a wider tensor.  gstate: G slots of DI*DJ floats per head (G > 1 or non-causal).
// sin / sout (either may be null): row-major fp32 [di][lds] state per head, likewise offset to the
// first column; the scan starts from sin and its last group writes the final state to sout.
template <class E>
struct ProblemT {
    const E *A, *B, *C;
    E *O;
    float *gstate;
    const float *sin;
    float *sout;
    int di, dj, ldc, reversed, lds;
    // reversed: the order in which the chunks are WALKED (1 = from the end of the sequence).  mask_rev: the side of
    // the diagonal the op sums over (0: positions <= s, 1: positions >= s).  They differ for an op in complement
    // form (comp = 1), which walks against its own direction: its state starts from the sum over everything the op
    // has to see at the first chunk walked and is DEcreased chunk by chunk, so the state at a chunk still includes
    // that chunk, and the score products take the other side of the diagonal with a minus sign:
    //     out_c = A_c S_incl - ((A_c B_c^T) o (1 - mask)) C_c ,   S_incl <- S_incl - B_c^T C_c .
    // This lets an op that sums over the past share every tile it reads with ops that sum over the future.
    int mask_rev, comp;
    // seed_from >= 0: this op's state is the TRANSPOSE of the state of problem `seed_from` of the same set (its B
    // and C are that problem's C and B, same walking order, square padded head dims): the group-state pass skips
    // it and its scan reads the other problem's slots transposed.
    int seed_from;
    int c0;  // first column of this problem's C / O slice within the full rows (column halves)
    // States handed from a forward to a backward pass.  save != null (an op that walks forwards over the past, not
    // in complement form): the state after every chunk p with (nchunks - 1 - p) % save_cpg == 0 goes to slot
    // (nchunks - 1 - p) / save_cpg (if < save_n) of this head, so slot g holds the sum over the chunks before
    // nchunks - g * save_cpg (slot 0: the whole sequence).  A slot holds the padded state as 16 x 16 tiles in the
    // accumulator layout: element [16 it + 4 g + q][16 jt + m] at ((it * save_njt + jt) * 64 + 16 g + m) * 4 + q,
    // save_njt tiles per tile row, save_slot floats per slot; a column-half problem writes its own tile columns
    // (c0 / 16 onwards).  One 16-byte store per lane and tile: a memory-bound scan has no vector-memory issue slots
    // to spare for narrower ones.
    // ext != null (an op in complement form cut into G groups of save_cpg chunks whose state is the TRANSPOSE of
    // the saved one): slot `group` of this head is the op's state at the first chunk it walks; the group-state and
    // prefix passes skip the op.
    float *save;
    const float *ext;
    int save_njt, save_slot, save_cpg, save_n;
    // Row strides of A, B and O in elements (C's is ldc) and, for each operand, where a head
    // starts: head bh is at (bh / H) * bs + (bh % H) * hs elements.  (BH,N,w) tensors have ld = w, hs = N * w,
    // bs = H * hs; (B,N,H,w) tensors, whose heads are interleaved inside a position, ld = H * w, hs = w,
    // bs = N * H * w.
    int lda, ldb, ldo, H;
    long hsA, bsA, hsB, bsB, hsC, bsC, hsO, bsO;
    // scan_pair_kernel only: a second problem G(A2, C, B) -> O2 served by the same workgroup (null = none)
    const E *A2;
    E *O2;
};

template <class E>
struct ProblemSetT {
    ProblemT<E> p[kMaxProblems];
    int count;
    int xcds;  // XCDs of the device: workgroup i is dispatched to XCD i % xcds (8 on an unpartitioned MI355X)
    // 16-bit kernels: the group-state pass cuts every group of the scan into `sub` pieces, one workgroup and one
    // slot each (slot (bh * G + grp) * sub + piece); the prefix pass leaves the scan's seed in the first of them
    int sub;
    // problems the group-state pass computes sums for (the others take their states from a twin problem or from
    // the forward pass): act[0 .. nact), so that its grid holds no workgroups that leave at once
    int act[kMaxProblems];
    int nact;
    int plain_two;  // scan_pair_kernel: the plain problem's workgroup runs two output wavefronts of two blocks
};
typedef ProblemT<u16> Problem;  // 16-bit storage (bf16 / fp16)
typedef ProblemSetT<u16> ProblemSet;

__device__ __forceinline__ size_t head_base(long bs, long hs, int H, int bh) {
    return (size_t)(bh / H) * (size_t)bs + (size_t)(bh % H) * (size_t)hs;
}

template <int DI, int DJ>
struct Tiling {
    static_assert(DI % 32 == 0 && DJ % 32 == 0, "padded head dims are multiples of 32");
    // LDS row strides (elements).  The paddings were chosen by measuring SQ_LDS_BANK_CONFLICT: 16/16/8 had
    // the fewest conflict cycles of the combinations tried.
    static constexpr int BS = DI + 16;           // [64][DI] tile: b128 row reads and transposing reads
    // ... of a [64][DJ] tile.  This tile is only read with transposing reads, which touch 4 consecutive
    // rows x 8 dwords per quarter-wave: a row stride of 8 (mod 32) dwords keeps them on distinct banks.
    static constexpr int CS = DJ + 16;
    static constexpr int SS = DI + 16;           // ... of the transposed 16-bit state [DJ][DI] (b128 row reads)
    static constexpr int NIT = DI / 16;          // 16-wide tiles along i
    static constexpr int NJT = DJ / 16;          // 16-wide tiles along j
    static constexpr int TPW = NIT * NJT / 4;    // fp32 state tiles owned by one wavefront
    static constexpr int KS = DI / 32;           // MFMA k-steps over i
    static constexpr int STATE_FLOATS = DI * DJ;
    static constexpr int OS = DJ + 8;            // ... of a staged output tile [64][DJ] (8-byte writes, 16-byte reads)
};

// ---- input preparation inside the causal forward (scan_kernel<..., PREP = true>) ------------------------
// q, k, v are the RAW projections; every tile is prepared on its way from registers to LDS (k, v: loader
// wavefronts) or to the MFMA operands (q: output wavefronts):
//     q_hat = keep * rot(q) / max(|q|, eps),  k_hat likewise,  v_hat = keep * v / max(cnt ^ sig[h], 1)
// with rot the GPT-J rotation of the first R columns by the table row of the position (row = pos[b][s], or pos0 + s
// when no position ids are given, clamped to the table).  The prepared rows also go to qo / ko / vo, (BH,N,D)
// tensors, for the backward pass.
struct PrepSide {
    const unsigned char *keep;  // (B,N) 0 / 1, or null
    const float *cnt;           // (B,N) and
    const float *sig;           // (H): value scaling, or both null
    const float *rot;           // (table_rows, R) [sin | cos], or null
    const long long *pos;       // (B,N) position ids (table row of every position), or null: row = pos0 + s
    long long pos0;
    int R, table_rows, H;
    int dv;                     // full width of the value rows (a problem may own a column slice of them)
    float eps;
    u16 *qo, *ko, *vo;          // prepared tensors for the backward pass, or null
};

template <class TR>
__device__ __forceinline__ void unpack8(u32x4 v, float *x) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        x[2 * i] = TR::to_float((u16)(v[i] & 0xffffu));
        x[2 * i + 1] = TR::to_float((u16)(v[i] >> 16));
    }
}
template <class TR>
__device__ __forceinline__ u32x4 pack8(const float *x) {
    return u32x4{TR::pack2(x[0], x[1]), TR::pack2(x[2], x[3]), TR::pack2(x[4], x[5]), TR::pack2(x[6], x[7])};
}
// the four pairs (x[2e], x[2e+1]) turned by the angles whose sines and cosines are sn[e], cs[e]
__device__ __forceinline__ void rotate8(float *x, f32x4 sn, f32x4 cs) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const float ev = x[2 * e], od = x[2 * e + 1];
        x[2 * e] = ev * cs[e] - od * sn[e];
        x[2 * e + 1] = od * cs[e] + ev * sn[e];
    }
}
__device__ __forceinline__ int clamp_row(const PrepSide &ps, long long t) {
    return (int)(t < 0 ? 0 : (t >= ps.table_rows ? ps.table_rows - 1 : t));
}
// Sum of v over the LANES (4, 8 or 16) consecutive, aligned lanes that hold one row, left in every one of them:
// data-parallel-primitive moves inside the vector ALU (quad swaps, then the mirrored half rows / rows, whose other
// half already holds its own partial sum in every lane) instead of permutes through the LDS crossbar.
template <int LANES>
__device__ __forceinline__ float lane_group_sum(float v) {
    static_assert(LANES == 4 || LANES == 8 || LANES == 16, "a row lives in 4, 8 or 16 lanes");
    auto moved = [](float x, auto ctrl) {
        return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), decltype(ctrl)::value,
                                                                     0xf, 0xf, false));
    };
    v += moved(v, std::integral_constant<int, 0xB1>{});                             // lanes 1,0,3,2 of each quad
    v += moved(v, std::integral_constant<int, 0x4E>{});                             // lanes 2,3,0,1
    if constexpr (LANES >= 8) v += moved(v, std::integral_constant<int, 0x141>{});  // mirrored half row (8 lanes)
    if constexpr (LANES >= 16) v += moved(v, std::integral_constant<int, 0x140>{}); // mirrored row (16 lanes)
    return v;
}

// One raw 16-byte piece (eight columns from `col`) of a q or k row -> rotated, normalised, masked.  The row lives in
// LANES consecutive lanes, which hold its other pieces; di: real width of the row; sn, cs: table entries of the piece's
// four pairs (used when rotate).
template <class TR, int LANES>
__device__ __forceinline__ u32x4 prep_qk_piece(u32x4 raw, int col, int di, bool rotate, f32x4 sn, f32x4 cs, float keep,
                                                float eps) {
    float x[8];
    unpack8<TR>(raw, x);
    if (col >= di) {
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] = 0.f;
    }
    if (rotate) rotate8(x, sn, cs);
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) ss += x[e] * x[e];
    ss = lane_group_sum<LANES>(ss);
    const float nrm = __builtin_amdgcn_sqrtf(ss);
    const float mul = keep * __builtin_amdgcn_rcpf(nrm > eps ? nrm : eps);
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] *= mul;
    return pack8<TR>(x);
}

// keep / max(cnt ^ sig, 1) of one position (keep alone when there is no value scaling)
__device__ __forceinline__ float value_scale(float keep, float cnt, float sig, bool scaled) {
    if (!scaled) return keep;
    const float p = cnt > 0.f ? __expf(sig * __logf(cnt)) : 0.f;
    return p > 1.f ? keep * __builtin_amdgcn_rcpf(p) : keep;
}
// one raw 16-byte piece of a v row -> scaled and masked (zero past the real width)
template <class TR>
__device__ __forceinline__ u32x4 prep_v_piece(u32x4 raw, bool inside, float keep, float cnt, float sig, bool scaled) {
    float x[8];
    unpack8<TR>(raw, x);
    const float mul = inside ? value_scale(keep, cnt, sig, scaled) : 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] *= mul;
    return inside ? pack8<TR>(x) : u32x4{0u, 0u, 0u, 0u};
}

// Workgroup -> (head, problem, group).  Linear id i runs on XCD i % xcds.  The (head, group) units, numbered
// group-major (unit = grp * BH + bh), are dealt round-robin over the XCDs: any number of heads loads all XCDs
// evenly, no XCD collects the units of one group (the first and last groups do less work), and with BH a
// multiple of the XCD count a head stays on one XCD.  Per XCD the ids are ordered (unit, problem), so the
// workgroups of one head and group are neighbours in the dispatch order of ONE XCD and share its L2.
struct WorkItem {
    int bh, prob, grp;
};
__device__ __forceinline__ WorkItem decode_workgroup(int nprob, int BH, int xcds) {
    const int i = blockIdx.x;
    const int xcd = i % xcds;
    const int slot = i / xcds;
    const int unit = (slot / nprob) * xcds + xcd;
    WorkItem wi;
    wi.prob = slot % nprob;
    wi.grp = unit / BH;  // >= G past the last unit: the caller returns
    wi.bh = unit % BH;
    return wi;
}
inline unsigned grid_for(int BH, int nprob, int G, int xcds) {
    return (unsigned)((((long)BH * G + xcds - 1) / xcds) * xcds * nprob);
}

// [64][D] tile, global -> registers, through a buffer descriptor of the head.  Thread t of NT owns 16-byte
// vectors t, t+NT, ...; rows past N read as zero (hardware range check).  Pure loads, no use of the
// result here, so nothing waits on them until the tile is staged.
template <int D, int NT = kThreads, bool STREAM = false>
__device__ __forceinline__ void load_tile(u32x4 *r, rsrc_t rs, int row0, int ld, int tid) {
#pragma unroll
    for (int u = 0; u < 8 * D / NT; ++u) {
        const int v = tid + NT * u;
        const int row = row0 + v / (D / 8);
        const int col = (v % (D / 8)) * 8;
        r[u] = buf_load16<STREAM>(rs, (uint32_t)(row * ld + col) * 2u);
    }
}

// registers -> LDS tile [64][D+8]; columns past the runtime width d are zeroed here, so padded
// positions add nothing to a product or a state.
template <int D, int STRIDE, int NT = kThreads>
__device__ __forceinline__ void store_tile(u16 *tile, const u32x4 *r, int d, int tid) {
#pragma unroll
    for (int u = 0; u < 8 * D / NT; ++u) {
        const int v = tid + NT * u;
        const int col = (v % (D / 8)) * 8;
        *reinterpret_cast<u32x4 *>(tile + (v / (D / 8)) * STRIDE + col) = (col < d) ? r[u] : u32x4{0u, 0u, 0u, 0u};
    }
}

// S[i][j] += sum_{tok<64} B[tok][i] * C[tok][j] for the tiles this wavefront owns
// (tile index t = w*TPW + u -> (t / NJT, t % NJT)).  Both operands are column fragments of the
// row-major LDS tiles, fetched with transposing reads; all fragments of a 32-token step are read
// before its MFMAs so the LDS latency is paid once per step, not once per tile.
// `flip`: 0, or 0x80008000 to subtract the product instead (sign bits of the B fragments).
template <class TR, int DI, int DJ>
__device__ __forceinline__ void state_update(f32x4 *S, const u16 *sB, const u16 *sC, int w, int g, int m,
                                             uint32_t flip = 0u) {
    using TL = Tiling<DI, DJ>;
    constexpr int ROWS = (TL::TPW + TL::NJT - 1) / TL::NJT;       // tile rows (values of `it`) per wavefront
    constexpr int COLS = TL::TPW < TL::NJT ? TL::TPW : TL::NJT;   // distinct `jt` per wavefront
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
        const int k0 = 32 * kb + 8 * g;
        u32x4 a[ROWS], b[COLS];
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            const int it = (w * TL::TPW + r * TL::NJT) / TL::NJT;
            a[r] = cat(lds_col4(sB, TL::BS, k0, 16 * it, m), lds_col4(sB, TL::BS, k0 + 4, 16 * it, m));
            a[r] ^= u32x4{flip, flip, flip, flip};
        }
#pragma unroll
        for (int c = 0; c < COLS; ++c) {
            const int jt = (w * TL::TPW + c) % TL::NJT;
            b[c] = cat(lds_col4(sC, TL::CS, k0, 16 * jt, m), lds_col4(sC, TL::CS, k0 + 4, 16 * jt, m));
        }
#pragma unroll
        for (int u = 0; u < TL::TPW; ++u) S[u] = TR::mfma(a[u / TL::NJT], b[u % COLS], S[u]);
    }
}

// Pipeline shared by both kernels: global loads run PF chunks ahead in PF register stages (static
// indices: the chunk loop is unrolled by PF), the LDS tiles are double-buffered so that chunk p+1
// is staged while chunk p is consumed, and ONE barrier separates consecutive chunks.  Every load
// and store in the loop is unconditional (prefetch past the end of the group re-reads its last
// chunk), which lets the compiler wait on exactly the stage it needs.

// Runs step(s, p) for p = p0 .. p1-1 with s = (p - p0) % PF a constant after unrolling (s indexes register
// stages that are reloaded PF chunks ahead).  The control flow is chosen for the wait counts the compiler derives
// from it, which are the most conservative over all paths into a point, whether they ever run or not:
//   * whole rounds of PF chunks run in a loop with a single exit and the remainder as straight-line code after
//     it: an exit test inside the round adds a path from the middle of a round back to its start, on which the
//     loads issued last look like the ones about to be used;
//   * the first round runs before the loop, so that the loop is only ever entered with the same loads and stores
//     in flight as on its back edge (after the prologue alone fewer are, and the oldest look younger).
// With either path present, a round waits for loads issued one chunk ago instead of PF chunks ago.
template <int PF, bool EXIT_INSIDE = false, class F>
__device__ __forceinline__ void run_rounds(int p0, int p1, F &&step) {
    int pb = p0;
    if (EXIT_INSIDE) {  // the plain form, for the callers that measured faster with it
        for (;; pb += PF) {
#pragma unroll
            for (int s = 0; s < PF; ++s) {
                if (pb + s >= p1) return;
                step(s, pb + s);
            }
        }
    }
    if (pb + PF <= p1) {
#pragma unroll
        for (int s = 0; s < PF; ++s) step(s, pb + s);
        for (pb += PF; pb + PF <= p1; pb += PF) {
#pragma unroll
            for (int s = 0; s < PF; ++s) step(s, pb + s);
        }
    }
#pragma unroll
    for (int s = 0; s < PF - 1; ++s)
        if (pb + s < p1) step(s, pb + s);  // uniform over the workgroup
}

// The per-chunk barrier; also a fence for the instruction scheduler, which otherwise moves the next chunk's
// register work (and with it the waits for that chunk's loads) above the barrier.
__device__ __forceinline__ void chunk_barrier() {
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
}

// Sum of B^T C over each piece of each group of chunks, written in register-native order:
// float4 index (w*TPW + u)*64 + lane of slot (bh*G + grp)*sub + piece.  `ngroups` of the G groups are launched
// (the causal scan never needs the last group's sum, except for ops in complement form; all_groups: the non-causal
// form, which needs every group of every op).
// PREP: B and C are the raw k and v projections of a forward pass whose scan prepares its inputs itself (PrepSide): the
// rows are rotated / normalised (B) and scaled / masked (C) on their way into the tiles, exactly as that scan does, so
// that the sums are those of the prepared tensors.  Nothing is written back here (the scan leaves the prepared rows).
template <class TR, int DI, int DJ, int PF, bool STREAM, bool PREP = false>
__global__ __launch_bounds__(kThreads, 2) void group_state_kernel(ProblemSet set, int BH, int N, int nchunks, int cpg,
                                                               int G, int ngroups, int all_groups, PrepSide prep) {
    using TL = Tiling<DI, DJ>;
    constexpr int SB = kChunk * TL::BS, SC = kChunk * TL::CS;
    __shared__ __attribute__((aligned(16))) u16 sB[2 * SB];
    __shared__ __attribute__((aligned(16))) u16 sC[2 * SC];
    const int tid = threadIdx.x, l = tid & 63, g = l >> 4, m = l & 15;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int sub = set.sub;
    // (head, group) units dealt over the XCDs like those of the scan that follows; only the problems that need sums
    // take part (workgroups that leave at once would still take dispatch slots, and the ones that stay then pile up
    // two to a CU beside idle CUs)
    const WorkItem wi = decode_workgroup(set.nact * sub, BH, set.xcds);
    if (wi.grp >= ngroups) return;
    const Problem &pr = set.p[set.act[wi.prob / sub]];
    const int grp = wi.grp, piece = wi.prob % sub;
    // `ngroups` == G is launched when some op of the set is in complement form; the others skip their last group
    if (grp == G - 1 && ngroups == G && !pr.comp && !all_groups) return;
    if (pr.seed_from >= 0 || pr.ext != nullptr) return;
    const int di = pr.di, dj = pr.dj, ldb = pr.ldb, ldc = pr.ldc, reversed = pr.reversed;
    const rsrc_t rB = make_rsrc(pr.B + head_base(pr.bsB, pr.hsB, pr.H, wi.bh), ((uint32_t)(N - 1) * ldb + di) * 2u);
    const rsrc_t rC = make_rsrc(pr.C + head_base(pr.bsC, pr.hsC, pr.H, wi.bh), ((uint32_t)(N - 1) * ldc + dj) * 2u);
    const int cps = (cpg + sub - 1) / sub;  // chunks per piece
    const int p0 = grp * cpg + piece * cps;
    const int p1 = min(p0 + cps, min((grp + 1) * cpg, nchunks));

    f32x4 S[TL::TPW];
#pragma unroll
    for (int u = 0; u < TL::TPW; ++u) S[u] = f32x4{0.f, 0.f, 0.f, 0.f};
    f32x4 *slot = reinterpret_cast<f32x4 *>(pr.gstate + (((size_t)wi.bh * G + grp) * sub + piece) * TL::STATE_FLOATS);
    if (p1 <= p0) {  // a piece past the end of its group: its slot is zero
#pragma unroll
        for (int u = 0; u < TL::TPW; ++u) slot[(w * TL::TPW + u) * 64 + l] = S[u];
        return;
    }

    constexpr int NB = DI / 32, NC = DJ / 32;
    u32x4 rb[PF][NB], rc[PF][NC];
    // PREP: the side inputs of a chunk (keep, count, rotary table entries of the rows of this thread's pieces) are
    // fetched ONE chunk before the chunk is staged, into a single set of registers and through buffer descriptors
    // (the tiles themselves run PF chunks ahead; with 128-wide tiles there are no registers for PF sets of side inputs),
    // and issued before that iteration's tile loads, so that waiting for them does not wait for those.  Position ids
    // are fetched one step earlier still, since the table entries' addresses depend on them.
    f32x4 sn[NB], cs[NB];
    uint32_t keep_b[NB], keep_c[NC];  // the bytes as loaded: converting them at once would wait for the load
    float cnt_c[NC];
    const size_t tok0 = PREP ? (size_t)(wi.bh / prep.H) * N : 0;
    const bool scaled = PREP && prep.cnt != nullptr && prep.sig != nullptr;
    const float sig = scaled ? prep.sig[wi.bh % prep.H] : 0.f;
    const bool has_pos = PREP && prep.pos != nullptr && prep.rot != nullptr;
    const rsrc_t rPos = make_rsrc_uniform(has_pos ? prep.pos + tok0 : nullptr, has_pos ? (uint32_t)N * 8u : 0u);
    const rsrc_t rKeep = make_rsrc(PREP && prep.keep ? prep.keep + tok0 : nullptr, PREP && prep.keep ? (uint32_t)N : 0u);
    const rsrc_t rCnt = make_rsrc(scaled ? prep.cnt + tok0 : nullptr, scaled ? (uint32_t)N * 4u : 0u);
    const bool rotary = PREP && prep.rot != nullptr;
    const rsrc_t rRot = make_rsrc(rotary ? prep.rot : nullptr, rotary ? (uint32_t)prep.table_rows * prep.R * 4u : 0u);
    u32x2 pnext[NB];
    auto row0_of = [&](int p) __attribute__((always_inline)) {
        const int pc = min(p, p1 - 1);
        return (reversed ? nchunks - 1 - pc : pc) * kChunk;
    };
    auto fetch_positions = [&](int p) __attribute__((always_inline)) {
        const int row0 = row0_of(p);
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            const int srow = min(row0 + (tid + kThreads * u) / (DI / 8), N - 1);
            pnext[u] = __builtin_amdgcn_raw_buffer_load_b64(rPos, (int)((uint32_t)srow * 8u), 0, 0);
        }
    };
    auto load_side = [&](int p) __attribute__((always_inline)) {  // side inputs of chunk p (uses the positions fetched one call earlier)
        const int row0 = row0_of(p);
        int trow[NB];
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            const int srow = min(row0 + (tid + kThreads * u) / (DI / 8), N - 1);
            const long long given = (long long)(((unsigned long long)pnext[u].y << 32) | pnext[u].x);
            trow[u] = clamp_row(prep, has_pos ? given : prep.pos0 + srow);
        }
        fetch_positions(p + 1);
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            const int v = tid + kThreads * u;
            const int srow = min(row0 + v / (DI / 8), N - 1), col = (v % (DI / 8)) * 8;
            keep_b[u] = prep.keep != nullptr ? (uint32_t)__builtin_amdgcn_raw_buffer_load_b8(rKeep, srow, 0, 0) : 1u;
            const uint32_t toff = (rotary && col < prep.R) ? (uint32_t)(trow[u] * prep.R + col / 2) * 4u : kOobOffset;
            sn[u] = bitcast<f32x4>(__builtin_amdgcn_raw_buffer_load_b128(rRot, (int)toff, 0, 0));
            cs[u] = bitcast<f32x4>(__builtin_amdgcn_raw_buffer_load_b128(rRot, (int)toff, prep.R * 2, 0));
        }
#pragma unroll
        for (int u = 0; u < NC; ++u) {
            const int srow = min(row0 + (tid + kThreads * u) / (DJ / 8), N - 1);
            keep_c[u] = prep.keep != nullptr ? (uint32_t)__builtin_amdgcn_raw_buffer_load_b8(rKeep, srow, 0, 0) : 1u;
            cnt_c[u] = bitcast<float>(__builtin_amdgcn_raw_buffer_load_b32(rCnt, srow * 4, 0, 0));
        }
    };
    auto load_chunk = [&](int s, int p) __attribute__((always_inline)) {
        const int row0 = row0_of(p);
        load_tile<DI, kThreads, STREAM>(rb[s], rB, row0, ldb, tid);
        load_tile<DJ, kThreads, STREAM>(rc[s], rC, row0, ldc, tid);
    };
    // registers of stage s -> LDS tiles tb, tc
    auto stage = [&](int s, u16 *tb, u16 *tc) __attribute__((always_inline)) {
        if constexpr (!PREP) {
            store_tile<DI, TL::BS>(tb, rb[s], di, tid);
            store_tile<DJ, TL::CS>(tc, rc[s], dj, tid);
        } else {
#pragma unroll
            for (int u = 0; u < NB; ++u) {
                const int v = tid + kThreads * u;
                const int col = (v % (DI / 8)) * 8;
                *reinterpret_cast<u32x4 *>(tb + (v / (DI / 8)) * TL::BS + col) = prep_qk_piece<TR, DI / 8>(
                    rb[s][u], col, di, rotary && col < prep.R, sn[u], cs[u], (float)keep_b[u], prep.eps);
                __builtin_amdgcn_sched_barrier(0);  // one piece at a time: eight unpacked columns each are enough registers
            }
#pragma unroll
            for (int u = 0; u < NC; ++u) {
                const int v = tid + kThreads * u;
                const int col = (v % (DJ / 8)) * 8;
                *reinterpret_cast<u32x4 *>(tc + (v / (DJ / 8)) * TL::CS + col) =
                    prep_v_piece<TR>(rc[s][u], col < dj, (float)keep_c[u], cnt_c[u], sig, scaled);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };
    auto finish = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < TL::TPW; ++u) slot[(w * TL::TPW + u) * 64 + l] = S[u];
    };
    if constexpr (PREP) {
        fetch_positions(p0);
        load_side(p0);
    }
#pragma unroll
    for (int s = 0; s < PF; ++s) load_chunk(s, p0 + s);
    stage(0, sB, sC);
    if constexpr (PREP) load_side(p0 + 1);
    load_chunk(0, p0 + PF);
    __syncthreads();
    run_rounds<PF>(p0, p1, [&](int s, int p) __attribute__((always_inline)) {
        const int s1 = (s + 1) % PF;
        const int buf = (p - p0) & 1;
        stage(s1, sB + (buf ^ 1) * SB, sC + (buf ^ 1) * SC);
        if constexpr (PREP) load_side(p + 2);
        load_chunk(s1, p + 1 + PF);
        state_update<TR, DI, DJ>(S, sB + buf * SB, sC + buf * SC, w, g, m);
        chunk_barrier();
    });
    finish();
}

// Over the G * sub slots of one head, element-wise.  mode 0: the first slot of group g gets the sum of all slots of
// the groups before g (only the first `ncomputed` groups hold data), or, for an op in complement form (all groups
// hold data), the total minus that sum.  mode 1: total into slot 0.  Slots are read in batches of independent
// loads and only written after they have been read.
template <class E>
__global__ __launch_bounds__(kThreads) void state_prefix_kernel(ProblemSetT<E> set, int BH, int G, int sub, int ncomputed,
                                                                int state_floats, int mode) {
    constexpr int BATCH = 8;
    const int sf4 = state_floats / 4;
    const int blocks_per_state = (sf4 + kThreads - 1) / kThreads;
    const int e = (blockIdx.x % blocks_per_state) * kThreads + threadIdx.x;
    const int rest = blockIdx.x / blocks_per_state;
    const int prob = rest % set.count, bh = rest / set.count;
    if (e >= sf4 || bh >= BH || set.p[prob].seed_from >= 0 || set.p[prob].ext != nullptr) return;
    const int nslots = G * sub;
    const bool comp = mode == 0 && set.p[prob].comp;
    const int nread = (mode == 1 || comp) ? nslots : ncomputed * sub;
    f32x4 *p = reinterpret_cast<f32x4 *>(set.p[prob].gstate + (size_t)bh * nslots * state_floats) + e;
    const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
    f32x4 total = zero;
    if (mode == 1 || comp) {
        for (int s0 = 0; s0 < nslots; s0 += BATCH) {
            f32x4 t[BATCH];
#pragma unroll
            for (int u = 0; u < BATCH; ++u) t[u] = (s0 + u < nslots) ? p[(size_t)(s0 + u) * sf4] : zero;
#pragma unroll
            for (int u = 0; u < BATCH; ++u) total += t[u];
        }
        if (mode == 1) {
            p[0] = total;
            return;
        }
    }
    f32x4 run = zero;
    for (int s0 = 0; s0 < nslots; s0 += BATCH) {
        f32x4 t[BATCH];
#pragma unroll
        for (int u = 0; u < BATCH; ++u) t[u] = (s0 + u < nread) ? p[(size_t)(s0 + u) * sf4] : zero;
#pragma unroll
        for (int u = 0; u < BATCH; ++u) {
            const int s = s0 + u;
            if (s < nslots && s % sub == 0) p[(size_t)s * sf4] = comp ? total - run : run;
            run += t[u];
        }
    }
}

// ---- the chunk recurrence --------------------------------------------------------------------------
//
// A workgroup handles one group of chunks of one head with wavefronts in three roles that share the
// SIMDs, so that each role's LDS / VALU / memory latencies are covered by the other roles' work and
// no role's per-chunk dependency chain carries the others':
//   * "output" wavefronts, each owning IB blocks of 16 output positions of the chunk.  A block's
//     scores are formed transposed, P^T = B_c A_blk^T, tile by tile, so the accumulator layout IS the
//     operand layout of the next product and the masked scores never leave registers; then
//     out_blk^T = C_c^T P^T + S^T A_blk^T, stored as 8-byte row segments.  Score tiles above the
//     diagonal are computed and zeroed.
//   * four "state" wavefronts carry the fp32 state S += B_c^T C_c in their accumulators and publish
//     its 16-bit copy for the next chunk.
//   * "loader" wavefronts move the B and C tiles global -> registers -> LDS, PF chunks ahead.
// One barrier per chunk joins the roles (every role function below executes 1 + (p1 - p0) barriers);
// LDS tiles and the 16-bit state are double-buffered.

// Position of a workgroup in the scan: chunks [p0, p1) in scan order of `nchunks`.
struct ScanRange {
    int N, nchunks, p0, p1, reversed;  // reversed: walking order
    int mask_rev, comp;                // see ProblemT
};

// Loader role: LT threads stage the B tile (rows of di) and the C tile (dj columns of rows of ldc).
// Output tiles staged in LDS by the output wavefronts (see output_role) and written to memory by the loader
// wavefronts one chunk later: up to two tiles per chunk (the problems of a pair), each [64][DJ] with row
// stride Tiling::OS, double-buffered; O[i] null = no such tile.
struct StagedOut {
    u16 *O[2];      // head base of each output tensor
    int dj[2], ld[2];
    const u16 *sO;  // [2 buffers][2 tiles][64 * OS]
};

template <int DI, int DJ, int PF, int LT, bool STREAM = false>
__device__ __forceinline__ void loader_role(const u16 *B_head, const u16 *C_head, int di, int dj, int ldb, int ldc,
                                            const ScanRange &r, int tid, u16 *sB, u16 *sC,
                                            const StagedOut *so = nullptr) {
    using TL = Tiling<DI, DJ>;
    constexpr int SB = kChunk * TL::BS, SC = kChunk * TL::CS, SO = kChunk * TL::OS;
    const rsrc_t rB = make_rsrc(B_head, ((uint32_t)(r.N - 1) * ldb + di) * 2u);
    const rsrc_t rC = make_rsrc(C_head, ((uint32_t)(r.N - 1) * ldc + dj) * 2u);
    // the staged tile(s) of chunk p (scan order): 16-byte row segments, rows past N dropped by the range check
    auto write_out = [&](int p) __attribute__((always_inline)) {
        const int row0 = (r.reversed ? r.nchunks - 1 - p : p) * kChunk;
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            if (so->O[t] == nullptr) continue;
            const rsrc_t rO = make_rsrc(so->O[t], ((uint32_t)(r.N - 1) * so->ld[t] + so->dj[t]) * 2u);
            const u16 *tile = so->sO + (((p - r.p0) & 1) * 2 + t) * SO;
#pragma unroll
            for (int u = 0; u < 8 * DJ / LT; ++u) {
                const int v = tid + LT * u;
                const int row = v / (DJ / 8), col = (v % (DJ / 8)) * 8;
                const u32x4 val = *reinterpret_cast<const u32x4 *>(tile + row * TL::OS + col);
                const uint32_t off = (col < so->dj[t]) ? (uint32_t)((row0 + row) * so->ld[t] + col) * 2u : kOobOffset;
                __builtin_amdgcn_raw_buffer_store_b128(val, rO, (int)off, 0, 0);
            }
        }
    };
    u32x4 rb[PF][8 * DI / LT], rc[PF][8 * DJ / LT];
    auto load_chunk = [&](int s, int p) __attribute__((always_inline)) {
        const int pc = min(p, r.p1 - 1);
        const int row0 = (r.reversed ? r.nchunks - 1 - pc : pc) * kChunk;
        load_tile<DI, LT, STREAM>(rb[s], rB, row0, ldb, tid);
        load_tile<DJ, LT, STREAM>(rc[s], rC, row0, ldc, tid);
    };
#pragma unroll
    for (int s = 0; s < PF; ++s) load_chunk(s, r.p0 + s);
    store_tile<DI, TL::BS, LT>(sB, rb[0], di, tid);
    store_tile<DJ, TL::CS, LT>(sC, rc[0], dj, tid);
    load_chunk(0, r.p0 + PF);
    __syncthreads();
    run_rounds<PF>(r.p0, r.p1, [&](int s, int p) __attribute__((always_inline)) {
        const int s1 = (s + 1) % PF;
        const int buf = (p - r.p0) & 1;
        // stage chunk p+1 (its loads were issued PF-1 chunks ago) and refill the register stage
        store_tile<DI, TL::BS, LT>(sB + (buf ^ 1) * SB, rb[s1], di, tid);
        store_tile<DJ, TL::CS, LT>(sC + (buf ^ 1) * SC, rc[s1], dj, tid);
        load_chunk(s1, p + 1 + PF);
        if (so != nullptr && p > r.p0) write_out(p - 1);
        chunk_barrier();
    });
    if (so != nullptr && r.p1 > r.p0) write_out(r.p1 - 1);
}

// Loader role with the input preparation folded in (see PrepSide): same pipeline as loader_role, for THREE tiles:
// the A rows (q) are staged here too, prepared, into sA, from where the output wavefronts take them, so that the
// preparation stays off their per-chunk chain.  The side inputs of a chunk (keep, count, table entries; the A and
// B tiles have the same rows and columns per thread and share the table entries) are fetched together with it, PF
// chunks ahead, and the prepared rows are also written to qo / ko / vo.  first_half: this workgroup writes qo and ko
// (with column halves both workgroups of a head stage the same q and k tiles).  A row of DI elements lives in
// DI / 8 consecutive lanes, which reduce its squared norm with lane shuffles.
template <class TR, int DI, int DJ, int PF, int LT>
__device__ __forceinline__ void loader_role_prep(const u16 *A_head, const u16 *B_head, const u16 *C_head, int di, int dj,
                                                 int lda, int ldb, int ldc, const ScanRange &r, int tid, u16 *sA, u16 *sB,
                                                 u16 *sC, const StagedOut *so, const PrepSide &ps, int bh, int c0,
                                                 bool first_half) {
    using TL = Tiling<DI, DJ>;
    constexpr int SB = kChunk * TL::BS, SC = kChunk * TL::CS, SO = kChunk * TL::OS;
    constexpr int NB = 8 * DI / LT, NC = 8 * DJ / LT;
    const rsrc_t rA = make_rsrc(A_head, ((uint32_t)(r.N - 1) * lda + di) * 2u);
    const rsrc_t rB = make_rsrc(B_head, ((uint32_t)(r.N - 1) * ldb + di) * 2u);
    const rsrc_t rC = make_rsrc(C_head, ((uint32_t)(r.N - 1) * ldc + dj) * 2u);
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
        const rsrc_t rO = make_rsrc(so->O[0], ((uint32_t)(r.N - 1) * so->ld[0] + so->dj[0]) * 2u);
        const u16 *tile = so->sO + (((p - r.p0) & 1) * 2) * SO;
#pragma unroll
        for (int u = 0; u < (8 * DJ + LT - 1) / LT; ++u) {
            const int v = tid + LT * u;
            const int row = v / (DJ / 8), col = (v % (DJ / 8)) * 8;
            if (v < 8 * DJ) {
                const u32x4 val = *reinterpret_cast<const u32x4 *>(tile + row * TL::OS + col);
                const uint32_t off = (col < so->dj[0]) ? (uint32_t)((row0 + row) * so->ld[0] + col) * 2u : kOobOffset;
                __builtin_amdgcn_raw_buffer_store_b128(val, rO, (int)off, 0, 0);
            }
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
    // Position ids, when given, are fetched one call of load_chunk ahead of the table entries they select (a load whose
    // address depends on a load issued in the same call would make that call wait for everything in flight).  The
    // chunks are loaded in walking order, so the next call is the next chunk.  A descriptor of zero bytes stands in
    // when there are none: the loads return zero and the row is pos0 + s.
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
            ra[s][u] = buf_load16(rA, (uint32_t)(row * lda + col) * 2u);
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
            const u32x4 ya = prep_qk_piece<TR, DI / 8>(ra[s][u], col, di, rotate, sn[s][u], cs[s][u], (float)keep_ab[s][u], ps.eps);
            const u32x4 yb = prep_qk_piece<TR, DI / 8>(rb[s][u], col, di, rotate, sn[s][u], cs[s][u], (float)keep_ab[s][u], ps.eps);
            *reinterpret_cast<u32x4 *>(ta + lrow * TL::BS + col) = ya;
            *reinterpret_cast<u32x4 *>(tb + lrow * TL::BS + col) = yb;
            const uint32_t off = (col < di) ? (uint32_t)((row0 + lrow) * di + col) * 2u : kOobOffset;
            __builtin_amdgcn_raw_buffer_store_b128(ya, rQo, (int)off, 0, 0);
            __builtin_amdgcn_raw_buffer_store_b128(yb, rKo, (int)off, 0, 0);
        }
#pragma unroll
        for (int u = 0; u < NC; ++u) {
            const int v = tid + LT * u;
            const int lrow = v / (DJ / 8), col = (v % (DJ / 8)) * 8;
            const u32x4 y = prep_v_piece<TR>(rc[s][u], col < dj, (float)keep_c[s][u], cnt_c[s][u], sig, scaled);
            *reinterpret_cast<u32x4 *>(tc + lrow * TL::CS + col) = y;
            const uint32_t off = (col < dj) ? (uint32_t)((row0 + lrow) * ps.dv + col) * 2u : kOobOffset;
            __builtin_amdgcn_raw_buffer_store_b128(y, rVo, (int)off, 0, 0);
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
        stage(s1, p + 1, sA + (buf ^ 1) * SB, sB + (buf ^ 1) * SB, sC + (buf ^ 1) * SC);
        load_chunk(s1, p + 1 + PF);
        if (so != nullptr && p > r.p0) write_out(p - 1);
        chunk_barrier();
    });
    if (so != nullptr && r.p1 > r.p0) write_out(r.p1 - 1);
}

// State role (wavefront w of 4).  seed: register-native group prefix or null; sin / sout: row-major
// fp32 hand-over states or null (sout only written when `last_group`).  sS: 16-bit copy transposed to
// [j][i] for the A_blk S product (a twin problem whose B and C are this problem's C and B reads the same copy
// transposed, see output_role).
// Forward-to-backward state hand-over of one workgroup (see ProblemT::save / ext): ext points at the slot of this
// head and group, save at the first slot of this head.
struct StateIO {
    const float *ext = nullptr;
    float *save = nullptr;
    int njt = 0, jt0 = 0, slot = 0, save_cpg = 1, save_n = 0;  // njt, slot: ProblemT::save_njt, save_slot; jt0 = c0 / 16
};

template <class TR, int DI, int DJ>
__device__ __forceinline__ void state_role(const float *seed, bool seed_transposed, const float *sin, float *sout, int lds, bool last_group,
                                           int di, int dj, const ScanRange &r, int w, int l, const u16 *sB,
                                           const u16 *sC, u16 *sS, const StateIO &io = StateIO()) {
    using TL = Tiling<DI, DJ>;
    constexpr int SB = kChunk * TL::BS, SC = kChunk * TL::CS, SSZ = DJ * TL::SS;
    const int g = l >> 4, m = l & 15;
    f32x4 S[TL::TPW];
#pragma unroll
    for (int u = 0; u < TL::TPW; ++u) S[u] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (seed != nullptr && !seed_transposed) {
        const f32x4 *gs = reinterpret_cast<const f32x4 *>(seed);
#pragma unroll
        for (int u = 0; u < TL::TPW; ++u) S[u] = gs[(w * TL::TPW + u) * 64 + l];
    }
    // A state held as 16 x 16 tiles in the accumulator layout (float4 index tile * 64 + lane), read TRANSPOSED: element
    // [16it + 4g + q][16jt + m] of this state is element [16jt + m][16it + 4g + q] of the other one, i.e. its tile
    // (jt, it), lane (g' = m / 4, m' = 4g + q), component m % 4.  Each source tile is loaded as it lies (one coalesced
    // 16-byte load per lane) and turned through a 1 KiB piece of LDS of this wavefront's own: 64 scattered 4-byte
    // loads per lane took several microseconds per workgroup.  The piece lies in the second buffer of the B tile,
    // which nobody writes before the first barrier.
    auto add_transposed = [&](const float *src, int src_njt) __attribute__((always_inline)) {
        float *scr = reinterpret_cast<float *>(const_cast<u16 *>(sB) + SB) + w * 256;
        f32x4 tile[TL::TPW];
#pragma unroll
        for (int u = 0; u < TL::TPW; ++u) {
            const int t = w * TL::TPW + u;
            tile[u] = reinterpret_cast<const f32x4 *>(src)[(size_t)((t % TL::NJT) * src_njt + t / TL::NJT) * 64 + l];
        }
#pragma unroll
        for (int u = 0; u < TL::TPW; ++u) {
            const int t = w * TL::TPW + u;
            const int it = t / TL::NJT, jt = t % TL::NJT;
            *reinterpret_cast<f32x4 *>(scr + 4 * l) = tile[u];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float x = scr[((m >> 2) * 16 + 4 * g + q) * 4 + (m & 3)];
                // (tiles outside the real dims are never written by the pass that saved them)
                if (16 * it + 4 * g + q < di && 16 * jt + m < dj) S[u][q] += x;
            }
        }
    };
    static_assert(SB * 2 >= 4 * 1024, "room for one tile per state wavefront");
    if constexpr (DI == DJ) {
        if (seed != nullptr && seed_transposed) add_transposed(seed, TL::NJT);
    }
    // accumulator element r of tile (it, jt) is S[16it + 4g + r][16jt + m]
    if (sin != nullptr) {
#pragma unroll
        for (int u = 0; u < TL::TPW; ++u) {
            const int t = w * TL::TPW + u;
            const int i0 = 16 * (t / TL::NJT) + 4 * g, j = 16 * (t % TL::NJT) + m;
#pragma unroll
            for (int q = 0; q < 4; ++q)
                if (i0 + q < di && j < dj) S[u][q] += sin[(size_t)(i0 + q) * lds + j];
        }
    }
    if (io.ext != nullptr) add_transposed(io.ext, io.njt);  // the state the forward pass saved is this one's transpose
    auto put_state = [&](u16 *dst) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < TL::TPW; ++u) {
            const int t = w * TL::TPW + u;
            const int it = t / TL::NJT, jt = t % TL::NJT;
            u32x2 pk = {TR::pack2(S[u][0], S[u][1]), TR::pack2(S[u][2], S[u][3])};
            *reinterpret_cast<u32x2 *>(dst + (16 * jt + m) * TL::SS + 16 * it + 4 * g) = pk;
        }
    };
    put_state(sS);
    __syncthreads();
    for (int p = r.p0; p < r.p1; ++p) {
        const int buf = (p - r.p0) & 1;
        state_update<TR, DI, DJ>(S, sB + buf * SB, sC + buf * SC, w, g, m, r.comp ? 0x80008000u : 0u);
        put_state(sS + (buf ^ 1) * SSZ);
        if (io.save != nullptr) {  // (this op walks forwards: p is the chunk's place in the sequence)
            const int back = r.nchunks - 1 - p;
            if (back % io.save_cpg == 0 && back / io.save_cpg < io.save_n) {
                f32x4 *dst = reinterpret_cast<f32x4 *>(io.save + (size_t)(back / io.save_cpg) * io.slot);
#pragma unroll
                for (int u = 0; u < TL::TPW; ++u) {
                    const int t = w * TL::TPW + u;
                    // (tile columns past this problem's width belong to the other column half, or to nobody)
                    if (16 * (t % TL::NJT) < dj) dst[((t / TL::NJT) * io.njt + io.jt0 + t % TL::NJT) * 64 + l] = S[u];
                }
            }
        }
        __syncthreads();
    }
    if (sout != nullptr && last_group) {
#pragma unroll
        for (int u = 0; u < TL::TPW; ++u) {
            const int t = w * TL::TPW + u;
            const int i0 = 16 * (t / TL::NJT) + 4 * g, j = 16 * (t % TL::NJT) + m;
#pragma unroll
            for (int q = 0; q < 4; ++q)
                if (i0 + q < di && j < dj) sout[(size_t)(i0 + q) * lds + j] = S[u][q];
        }
    }
}

// Output role: one wavefront, IB blocks of 16 positions starting at block `blk0` of each chunk.
// lda, ldc: row strides of A and of O.
// cB: tile read by rows (the B operand of this problem), cC: tile read by columns (its C operand),
// cS: its 16-bit state; all three double-buffered with the strides of Tiling<DI, DJ>.
// sOt: null = store the outputs to memory from here; else the [2 buffers] of this problem's staged output tile
// (buffer stride 2 * 64 * OS), written with 8-byte LDS stores and sent to memory by the loader wavefronts, so that
// this wavefront's chain of LDS reads and MFMAs never waits for the vector-memory pipeline to take a store.
// PREP: the A rows are not loaded from memory here: the loader wavefronts stage them, prepared, in sA (a tile like
// sB, double-buffered; see loader_role_prep).
// SKIP != 0 (two blocks per wavefront): the wavefront owns the blocks {0, 3} (SKIP = 1, 3) or {1, 2} (SKIP = 2, 4) of
// a chunk instead of two neighbours, and leaves out the score tiles that lie entirely on the masked side of the
// diagonal together with the products that would only see their zeros: 5 of 8 score tiles and 3 of 4 steps of the
// score-times-C products remain for either wavefront.  SKIP = 1, 2: the scores of keys at or after the query are the
// ones that count (ops that sum over the future, or over the past in complement form); SKIP = 3, 4: those of keys
// at or before it.  The caller picks the variant that matches the problem's mask.
// SKIP = 5 + b / 9 + b (one block per wavefront): the wavefront owns block b = 0..3 and leaves out the score tiles
// of keys before (5 + b) / after (9 + b) its block in the same way.
// TRS: sS holds the 16-bit copy of the TRANSPOSE of this problem's state (the copy published for a twin problem whose
// B and C are this problem's C and B); it is then read with transposing LDS reads.
template <class TR, int DI, int DJ, int PF, int IB, bool STREAM = false, bool PREP = false, int SKIP = 0, bool TRS = false,
          bool WST = false>
__device__ __forceinline__ void output_role(const u16 *A_head, u16 *O_head, int di, int dj, int lda, int ldc,
                                            const ScanRange &r, int blk0, int l, const u16 *sB, const u16 *sC,
                                            const u16 *sS, u16 *sOt = nullptr, const u16 *sA = nullptr, u16 *sW = nullptr) {
    using TL = Tiling<DI, DJ>;
    constexpr int SB = kChunk * TL::BS, SC = kChunk * TL::CS, SSZ = DJ * TL::SS;
    const int g = l >> 4, m = l & 15;
    static_assert(SKIP == 0 || (SKIP <= 4 ? IB == 2 : (IB == 1 && SKIP <= 12)), "block pairing needs two blocks per wavefront");
    // block (16 positions of the chunk) number `ib` of this wavefront; whether its score tile against key tile jt
    // can hold anything (SKIP: keys >= queries are kept)
    auto blk = [&](int ib) __attribute__((always_inline)) {
        if constexpr (SKIP >= 5) return (SKIP - 5) & 3;
        else return SKIP == 0 ? blk0 + ib : ((SKIP & 1) ? (ib == 0 ? 0 : 3) : (ib == 0 ? 1 : 2));
    };
    auto live = [&](int ib, int jt) __attribute__((always_inline)) {
        if constexpr (SKIP == 0) return true;
        else if constexpr (SKIP <= 4) return SKIP <= 2 ? jt >= blk(ib) : jt <= blk(ib);
        else return SKIP <= 8 ? jt >= SKIP - 5 : jt <= SKIP - 9;
    };
    auto live_step = [&](int kb) __attribute__((always_inline)) {  // whether any block of this wavefront uses keys 32 kb .. 32 kb + 31
        bool any = false;
#pragma unroll
        for (int ib = 0; ib < IB; ++ib) any = any || live(ib, 2 * kb) || live(ib, 2 * kb + 1);
        return any;
    };
    const rsrc_t rA = make_rsrc(A_head, ((uint32_t)(r.N - 1) * lda + di) * 2u);
    const rsrc_t rO = make_rsrc(O_head, ((uint32_t)(r.N - 1) * ldc + dj) * 2u);
    const int reversed = r.reversed;
    const bool mask_rev = r.mask_rev != 0, comp = r.comp != 0;
    u32x4 qn[PF][IB][TL::KS], qc[IB][TL::KS];
    auto load_q = [&](int s, int p) __attribute__((always_inline)) {
        if constexpr (!PREP) {
            const int pc = min(p, r.p1 - 1);
            const int row = (reversed ? r.nchunks - 1 - pc : pc) * kChunk + m;
#pragma unroll
            for (int ib = 0; ib < IB; ++ib)
#pragma unroll
                for (int ks = 0; ks < TL::KS; ++ks)
                    qn[s][ib][ks] = buf_load16<STREAM>(rA, (uint32_t)((row + 16 * blk(ib)) * lda + 32 * ks + 8 * g) * 2u);
        }
    };
#pragma unroll
    for (int s = 0; s < PF; ++s) load_q(s, r.p0 + s);
    __syncthreads();
    // (the large tiles keep the exit test inside the round: with 8 column tiles and 4 contraction steps per block
    // the single-exit form measured 8 % slower there, at D = 128 on long sequences)
    run_rounds<PF, (DI * DJ > 64 * 64)>(r.p0, r.p1, [&](int s, int p) __attribute__((always_inline)) {
        {
            const int buf = (p - r.p0) & 1;
            const u16 *cB = sB + buf * SB, *cC = sC + buf * SC, *cS = sS + buf * SSZ;
            const int row0 = (reversed ? r.nchunks - 1 - p : p) * kChunk;
            if constexpr (!PREP) {
#pragma unroll
                for (int ib = 0; ib < IB; ++ib)
#pragma unroll
                    for (int ks = 0; ks < TL::KS; ++ks)
                        qc[ib][ks] = (32 * ks + 8 * g < di) ? qn[s][ib][ks] : u32x4{0u, 0u, 0u, 0u};
            } else {
                const u16 *cA = sA + buf * SB;
#pragma unroll
                for (int ib = 0; ib < IB; ++ib)
#pragma unroll
                    for (int ks = 0; ks < TL::KS; ++ks)
                        qc[ib][ks] = *reinterpret_cast<const u32x4 *>(cA + (16 * blk(ib) + m) * TL::BS + 32 * ks + 8 * g);
            }
            load_q(s, p + PF);

            // Operand fragments of the output products come in batches of JB column tiles; the reads of a batch are
            // issued one batch ahead (the first before the score products), so their LDS latency runs under MFMAs.
            constexpr int JBmax = (IB == 1) ? 8 : 4;
            constexpr int JB = (JBmax / TL::KS < 1) ? 1 : ((JBmax / TL::KS < TL::NJT) ? (JBmax / TL::KS) : TL::NJT);
            constexpr int NBATCH = TL::NJT / JB;
            u32x4 vf[2][JB][2], sf[2][JB][TL::KS];
            auto read_batch = [&](int slot, int j0) __attribute__((always_inline)) {
#pragma unroll
                for (int jj = 0; jj < JB; ++jj) {
                    const int jt = j0 + jj;
#pragma unroll
                    for (int kb = 0; kb < 2; ++kb)
                        if (live_step(kb))
                            vf[slot][jj][kb] = cat(lds_col4(cC, TL::CS, 32 * kb + 4 * g, 16 * jt, m),
                                                   lds_col4(cC, TL::CS, 32 * kb + 16 + 4 * g, 16 * jt, m));
#pragma unroll
                    for (int ks = 0; ks < TL::KS; ++ks)
                        sf[slot][jj][ks] =
                            TRS ? cat(lds_col4(cS, TL::SS, 32 * ks + 8 * g, 16 * jt, m),
                                      lds_col4(cS, TL::SS, 32 * ks + 8 * g + 4, 16 * jt, m))
                                : *reinterpret_cast<const u32x4 *>(cS + (16 * jt + m) * TL::SS + 32 * ks + 8 * g);
                }
            };

            // masked scores, transposed: pk[ib][jt] = P^T[16jt+4g .. +3][16(blk0+ib)+m]; fragment
            // reads first, MFMAs after, so the LDS latency is paid once per batch
            u32x2 pk[IB][4];
            {
                u32x4 kf[4][TL::KS];
#pragma unroll
                for (int jt = 0; jt < 4; ++jt) {
                    if (!(live(0, jt) || live(IB - 1, jt))) continue;
#pragma unroll
                    for (int ks = 0; ks < TL::KS; ++ks)
                        kf[jt][ks] = *reinterpret_cast<const u32x4 *>(cB + (16 * jt + m) * TL::BS + 32 * ks + 8 * g);
                }
                read_batch(0, 0);
#pragma unroll
                for (int ib = 0; ib < IB; ++ib)
#pragma unroll
                    for (int jt = 0; jt < 4; ++jt) {
                        if (!live(ib, jt)) {
                            pk[ib][jt] = u32x2{0u, 0u};
                            continue;
                        }
                        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                        for (int ks = 0; ks < TL::KS; ++ks) acc = TR::mfma(kf[jt][ks], qc[ib][ks], acc);
                        const int d0 = 16 * (jt - blk(ib)) + 4 * g - m;  // key pos - query pos at element 0
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            const bool keep = mask_rev ? (d0 + q >= 0) : (d0 + q <= 0);
                            acc[q] = (keep != comp) ? (comp ? -acc[q] : acc[q]) : 0.f;
                        }
                        pk[ib][jt] = u32x2{TR::pack2(acc[0], acc[1]), TR::pack2(acc[2], acc[3])};
                    }
            }

            const int orow = row0 + m;
#pragma unroll
            for (int bt = 0; bt < NBATCH; ++bt) {
                const int j0 = bt * JB, slot = bt & 1;
                if (bt + 1 < NBATCH) read_batch(slot ^ 1, j0 + JB);
#pragma unroll
                for (int ib = 0; ib < IB; ++ib)
#pragma unroll
                    for (int jj = 0; jj < JB; ++jj) {
                        const int jt = j0 + jj;
                        // With four contraction steps (DI = 128) a tile's 2 + 4 products run as three chains of two: a
                        // dependent MFMA waits for the whole latency of the one before and such a batch has only
                        // IB tiles to interleave (5 % faster there; at DI <= 64 the extra accumulators only cost
                        // registers, spilling in the pair kernel).
                        f32x4 o = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                        for (int kb = 0; kb < 2; ++kb)
                            if (live(ib, 2 * kb) || live(ib, 2 * kb + 1))
                                o = TR::mfma(vf[slot][jj][kb], cat(pk[ib][2 * kb], pk[ib][2 * kb + 1]), o);
                        if constexpr (TL::KS >= 4) {
                            f32x4 o2 = {0.f, 0.f, 0.f, 0.f}, o3 = o2;
#pragma unroll
                            for (int ks = 0; ks < TL::KS; ks += 2) {
                                o2 = TR::mfma(sf[slot][jj][ks], qc[ib][ks], o2);
                                o3 = TR::mfma(sf[slot][jj][ks + 1], qc[ib][ks + 1], o3);
                            }
                            o += o2 + o3;
                        } else {
#pragma unroll
                            for (int ks = 0; ks < TL::KS; ++ks) o = TR::mfma(sf[slot][jj][ks], qc[ib][ks], o);
                        }
                        const int col = 16 * jt + 4 * g;
                        const u32x2 val = {TR::pack2(o[0], o[1]), TR::pack2(o[2], o[3])};
                        if constexpr (WST) {
                            *reinterpret_cast<u32x2 *>(sW + (16 * ib + m) * kWaveStageStride + (col & 63)) = val;
                        } else if (sOt != nullptr) {
                            *reinterpret_cast<u32x2 *>(sOt + buf * (2 * kChunk * TL::OS) +
                                                       (16 * blk(ib) + m) * TL::OS + col) = val;
                        } else {
                            const uint32_t off = (col < dj) ? (uint32_t)((orow + 16 * blk(ib)) * ldc + col) * 2u : kOobOffset;
                            buf_store8(rO, off, val);
                        }
                    }
                if constexpr (WST) {
                    // 64 finished columns of this wavefront's rows: back out of its staging tile as 16-byte pieces,
                    // eight lanes to a 128-byte row segment, and to memory as whole cache lines
                    static_assert(!WST || (JB == 1 || JB == 2 || JB == 4), "a flush covers four column tiles");
                    if (((bt + 1) * JB) % 4 == 0) {
                        const int c0 = 16 * ((bt + 1) * JB - 4);
#pragma unroll
                        for (int u = 0; u < 2 * IB; ++u) {
                            const int lrow = (l >> 3) + 8 * u, col = c0 + 8 * (l & 7);
                            const u32x4 val = *reinterpret_cast<const u32x4 *>(sW + lrow * kWaveStageStride + 8 * (l & 7));
                            const int prow = row0 + 16 * blk(u / 2) + (lrow & 15);
                            const uint32_t off = (col < dj) ? (uint32_t)(prow * ldc + col) * 2u : kOobOffset;
                            __builtin_amdgcn_raw_buffer_store_b128(val, rO, (int)off, 0, 0);
                        }
                    }
                }
            }
            chunk_barrier();
        }
    });
}

// Calls f(integral_constant<int, v>) with v = block (0..3) + (future ? 0 : 4), i.e. SKIP - 5 of output_role, for an
// output wavefront that owns one block of 16 positions.
template <class F>
__device__ __forceinline__ void one_block_variant(int block, bool future, F &&f) {
    switch (block + (future ? 0 : 4)) {
        case 0: f(std::integral_constant<int, 0>{}); break;
        case 1: f(std::integral_constant<int, 1>{}); break;
        case 2: f(std::integral_constant<int, 2>{}); break;
        case 3: f(std::integral_constant<int, 3>{}); break;
        case 4: f(std::integral_constant<int, 4>{}); break;
        case 5: f(std::integral_constant<int, 5>{}); break;
        case 6: f(std::integral_constant<int, 6>{}); break;
        default: f(std::integral_constant<int, 7>{}); break;
    }
}

// One problem per workgroup: OW output wavefronts (IB = 4/OW blocks each), 4 state, LW loader.
// PREP: q, k, v are the raw projections and are prepared inside the kernel (PrepSide; forward direction, G = 1).
// WST: every output wavefront passes its tiles through a small staging tile of its own in LDS and stores them as
// 16-byte pieces that make up whole 128-byte row segments (where a workgroup-wide staged tile, STAGED, has no room).
template <class TR, int DI, int DJ, int PF, int OW, int LW, bool STAGED = false, bool STREAM = false, bool PREP = false,
          bool WST = false>
__global__ __launch_bounds__(64 * (OW + 4 + LW)) void scan_kernel(ProblemSet set, int BH, int N, int nchunks,
                                                                  int cpg, int G, PrepSide prep) {
    using TL = Tiling<DI, DJ>;
    static_assert(OW == 2 || OW == 4, "two or four output wavefronts");
    static_assert(LW == 2 || LW == 4, "two or four loader wavefronts");
    constexpr int IB = 4 / OW;
    constexpr int LT = 64 * LW;  // loader threads
    static_assert((8 * DI) % LT == 0 && (8 * DJ) % LT == 0, "tile vectors divide over the loader threads");
    constexpr int SB = kChunk * TL::BS, SC = kChunk * TL::CS, SSZ = DJ * TL::SS;
    __shared__ __attribute__((aligned(16))) u16 sB[2 * SB];
    __shared__ __attribute__((aligned(16))) u16 sC[2 * SC];
    __shared__ __attribute__((aligned(16))) u16 sS[2 * SSZ];
    // STAGED: output tiles go through LDS and leave as 16-byte row segments from the loader wavefronts (StagedOut;
    // the layout has room for two tiles per buffer, this kernel uses the first)
    __shared__ __attribute__((aligned(16))) u16 sO[STAGED ? 2 * 2 * kChunk * TL::OS : 8];
    __shared__ __attribute__((aligned(16))) u16 sA[PREP ? 2 * SB : 8];  // PREP: the prepared A rows, staged like sB
    static_assert(!WST || (!STAGED && 4 / OW == 2 && DJ % 64 == 0), "wave-staged stores: two blocks per wavefront");
    __shared__ __attribute__((aligned(16))) u16 sWst[WST ? OW * 32 * kWaveStageStride : 8];
    const int l = threadIdx.x & 63;
    const int wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const WorkItem wi = decode_workgroup(set.count, BH, set.xcds);
    if (wi.grp >= G) return;
    const Problem &pr = set.p[wi.prob];
    const int di = pr.di, dj = pr.dj, ldc = pr.ldc;
    ScanRange r;
    r.N = N;
    r.nchunks = nchunks;
    r.p0 = wi.grp * cpg;
    r.p1 = min(r.p0 + cpg, nchunks);
    r.reversed = pr.reversed;
    r.mask_rev = pr.mask_rev;
    r.comp = pr.comp;
    if (wv >= OW + 4) {
        StagedOut so;
        so.O[0] = pr.O + head_base(pr.bsO, pr.hsO, pr.H, wi.bh);
        so.dj[0] = dj;
        so.ld[0] = pr.ldo;
        so.O[1] = nullptr;
        so.dj[1] = 0;
        so.ld[1] = 0;
        so.sO = sO;
        if constexpr (PREP)
            loader_role_prep<TR, DI, DJ, PF, LT>(pr.A + head_base(pr.bsA, pr.hsA, pr.H, wi.bh),
                                                 pr.B + head_base(pr.bsB, pr.hsB, pr.H, wi.bh),
                                                 pr.C + head_base(pr.bsC, pr.hsC, pr.H, wi.bh), di, dj, pr.lda, pr.ldb, ldc,
                                                 r, (int)threadIdx.x - 64 * (OW + 4), sA, sB, sC, STAGED ? &so : nullptr,
                                                 prep, wi.bh, pr.c0, pr.c0 == 0);
        else
            loader_role<DI, DJ, PF, LT, STREAM>(pr.B + head_base(pr.bsB, pr.hsB, pr.H, wi.bh), pr.C + head_base(pr.bsC, pr.hsC, pr.H, wi.bh),
                                                di, dj, pr.ldb, ldc, r, (int)threadIdx.x - 64 * (OW + 4), sB, sC, STAGED ? &so : nullptr);
    } else if (wv >= OW) {
        const float *slots = pr.ext ? nullptr : (pr.seed_from >= 0 ? set.p[pr.seed_from].gstate : pr.gstate);
        StateIO io;
        io.njt = pr.save_njt;
        io.slot = pr.save_slot;
        if (pr.ext != nullptr) io.ext = pr.ext + ((size_t)wi.bh * G + wi.grp) * pr.save_slot;
        if (pr.save != nullptr) {
            io.save = pr.save + (size_t)wi.bh * pr.save_n * pr.save_slot;
            io.jt0 = pr.c0 / 16;
            io.save_cpg = pr.save_cpg;
            io.save_n = pr.save_n;
        }
        state_role<TR, DI, DJ>(
            slots ? slots + ((size_t)wi.bh * G + wi.grp) * set.sub * TL::STATE_FLOATS : nullptr, pr.seed_from >= 0,
            pr.sin ? pr.sin + (size_t)wi.bh * di * pr.lds : nullptr, pr.sout ? pr.sout + (size_t)wi.bh * di * pr.lds : nullptr,
            pr.lds, wi.grp == G - 1, di, dj, r, wv - OW, l, sB, sC, sS, io);
    } else {
        const u16 *A_head = pr.A + head_base(pr.bsA, pr.hsA, pr.H, wi.bh);
        u16 *O_head = pr.O + head_base(pr.bsO, pr.hsO, pr.H, wi.bh);
        if constexpr (IB == 2) {
            // two wavefronts of two blocks: blocks {0,3} and {1,2}, dead score tiles left out (see output_role)
            const bool future = (pr.mask_rev != 0) != (pr.comp != 0);
            u16 *sW = sWst + (WST ? wv * 32 * kWaveStageStride : 0);
            if (future) {
                if (wv == 0)
                    output_role<TR, DI, DJ, PF, 2, STREAM, PREP, 1, false, WST>(A_head, O_head, di, dj, pr.lda, pr.ldo, r, 0, l,
                                                                                      sB, sC, sS, STAGED ? sO : nullptr, sA, sW);
                else
                    output_role<TR, DI, DJ, PF, 2, STREAM, PREP, 2, false, WST>(A_head, O_head, di, dj, pr.lda, pr.ldo, r, 0, l,
                                                                                      sB, sC, sS, STAGED ? sO : nullptr, sA, sW);
            } else {
                if (wv == 0)
                    output_role<TR, DI, DJ, PF, 2, STREAM, PREP, 3, false, WST>(A_head, O_head, di, dj, pr.lda, pr.ldo, r, 0, l,
                                                                                      sB, sC, sS, STAGED ? sO : nullptr, sA, sW);
                else
                    output_role<TR, DI, DJ, PF, 2, STREAM, PREP, 4, false, WST>(A_head, O_head, di, dj, pr.lda, pr.ldo, r, 0, l,
                                                                                      sB, sC, sS, STAGED ? sO : nullptr, sA, sW);
            }
        } else {
            // one block per wavefront: the variant that knows its block and the side of the diagonal that counts
            one_block_variant(wv, (pr.mask_rev != 0) != (pr.comp != 0), [&](auto tag) {
                output_role<TR, DI, DJ, PF, 1, STREAM, PREP, 5 + decltype(tag)::value>(
                    A_head, O_head, di, dj, pr.lda, pr.ldo, r, wv, l, sB, sC, sS, STAGED ? sO : nullptr, sA);
            });
        }
    }
}

// Gradient launch for square head dims: two kinds of workgroup in one grid of 4 + 4 + LW wavefronts.
//   * a plain problem (dQ): four output wavefronts of one block each, as in scan_kernel;
//   * a PAIR of problems X = G(A, B, C) and Y = G(A2, C, B) that scan the same way (dK = G(V, dO, Q) and
//     dV = G(K, Q, dO)): their tiles are the same two tiles with the roles swapped and their states are
//     transposes of each other, so one workgroup stages the tiles once, carries the state once (publishing
//     both orientations) and gives two output wavefronts of two blocks to each problem.
// This puts the three gradients of a head on two workgroups instead of three, i.e. 2*BH workgroups:
// one per CU at the headline shape instead of one and a half.
// OWP = output wavefronts per problem of a pair (2 of two blocks, or 4 of one block); a plain problem
// always uses four of one block and leaves the other OWP*2 - 4 output wavefronts idle at the barriers.
template <class TR, int D, int PF, int LW, int OWP>
__global__ __launch_bounds__(64 * (2 * OWP + 4 + LW)) void scan_pair_kernel(ProblemSet set, int BH, int N, int nchunks,
                                                                            int cpg, int G) {
    using TL = Tiling<D, D>;
    static_assert(TL::BS == TL::CS, "the two tiles are read both ways");
    static_assert(OWP == 2 || OWP == 4, "two or four output wavefronts per problem");
    constexpr int NOUT = 2 * OWP, IBP = 4 / OWP;
    constexpr int LT = 64 * LW;
    constexpr int SB = kChunk * TL::BS, SC = kChunk * TL::CS, SSZ = D * TL::SS;
    __shared__ __attribute__((aligned(16))) u16 sB[2 * SB];
    __shared__ __attribute__((aligned(16))) u16 sC[2 * SC];
    __shared__ __attribute__((aligned(16))) u16 sS[2 * SSZ];
    __shared__ __attribute__((aligned(16))) u16 sO[2 * 2 * kChunk * TL::OS];
    const int l = threadIdx.x & 63;
    const int wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const WorkItem wi = decode_workgroup(set.count, BH, set.xcds);
    if (wi.grp >= G) return;
    const Problem &pr = set.p[wi.prob];
    const int di = pr.di, dj = pr.dj, ldc = pr.ldc;
    const bool pair = pr.A2 != nullptr;
    constexpr int SO = kChunk * TL::OS;
    ScanRange r;
    r.N = N;
    r.nchunks = nchunks;
    r.p0 = wi.grp * cpg;
    r.p1 = min(r.p0 + cpg, nchunks);
    r.reversed = pr.reversed;
    r.mask_rev = pr.mask_rev;
    // The plain problem (dQ) runs in complement form when the forward pass has left its states (ProblemT::ext): it
    // then walks the sequence from the end like the pair and reads the tiles the pair's workgroup reads, at about
    // the same time.  The pair itself never does.
    r.comp = pair ? 0 : pr.comp;
    const float *seed = (pr.gstate && pr.ext == nullptr)
                            ? pr.gstate + ((size_t)wi.bh * G + wi.grp) * set.sub * TL::STATE_FLOATS : nullptr;
    if (wv >= NOUT + 4) {
        StagedOut so;
        so.O[0] = pr.O + head_base(pr.bsO, pr.hsO, pr.H, wi.bh);
        so.dj[0] = dj;
        so.ld[0] = pr.ldo;
        so.O[1] = pair ? pr.O2 + (size_t)wi.bh * N * di : nullptr;
        so.dj[1] = di;
        so.ld[1] = di;
        so.sO = sO;
        loader_role<D, D, PF, LT>(pr.B + head_base(pr.bsB, pr.hsB, pr.H, wi.bh), pr.C + head_base(pr.bsC, pr.hsC, pr.H, wi.bh),
                                  di, dj, pr.ldb, ldc, r, (int)threadIdx.x - 64 * (NOUT + 4), sB, sC, &so);
    } else if (wv >= NOUT) {
        // one 16-bit copy of the state serves both problems of a pair: the second reads it transposed
        StateIO io;
        if (!pair && pr.ext != nullptr) {
            io.ext = pr.ext + ((size_t)wi.bh * G + wi.grp) * pr.save_slot;
            io.njt = pr.save_njt;
            io.slot = pr.save_slot;
        }
        state_role<TR, D, D>(seed, false, nullptr, nullptr, 0, false, di, dj, r, wv - NOUT, l, sB, sC, sS, io);
    } else if (!pair) {
        const u16 *A_head = pr.A + head_base(pr.bsA, pr.hsA, pr.H, wi.bh);
        const bool future = (pr.mask_rev != 0) != (r.comp != 0);
        if (set.plain_two && wv < 2) {
            // two output wavefronts of two blocks, the pace of the pair's workgroup next door
            if (future) {
                if (wv == 0) output_role<TR, D, D, PF, 2, false, false, 1>(A_head, nullptr, di, dj, pr.lda, pr.ldo, r, 0, l, sB, sC, sS, sO);
                else output_role<TR, D, D, PF, 2, false, false, 2>(A_head, nullptr, di, dj, pr.lda, pr.ldo, r, 0, l, sB, sC, sS, sO);
            } else {
                if (wv == 0) output_role<TR, D, D, PF, 2, false, false, 3>(A_head, nullptr, di, dj, pr.lda, pr.ldo, r, 0, l, sB, sC, sS, sO);
                else output_role<TR, D, D, PF, 2, false, false, 4>(A_head, nullptr, di, dj, pr.lda, pr.ldo, r, 0, l, sB, sC, sS, sO);
            }
        } else if (!set.plain_two && wv < 4) {
            one_block_variant(wv, future, [&](auto tag) {
                output_role<TR, D, D, PF, 1, false, false, 5 + decltype(tag)::value>(A_head, nullptr, di, dj, pr.lda, pr.ldo, r, wv,
                                                                                     l, sB, sC, sS, sO);
            });
        } else {
            for (int p = r.p0 - 1; p < r.p1; ++p) __syncthreads();  // idle: keep the barrier count
        }
    } else if (wv < OWP) {
        const u16 *A_head = pr.A + head_base(pr.bsA, pr.hsA, pr.H, wi.bh);
        if constexpr (IBP == 2) {  // the pair sums over the future: blocks {0, 3} and {1, 2}, dead score tiles left out
            if (wv == 0)
                output_role<TR, D, D, PF, 2, false, false, 1>(A_head, nullptr, di, dj, pr.lda, pr.ldo, r, 0, l, sB, sC, sS, sO);
            else
                output_role<TR, D, D, PF, 2, false, false, 2>(A_head, nullptr, di, dj, pr.lda, pr.ldo, r, 0, l, sB, sC, sS, sO);
        } else {
            output_role<TR, D, D, PF, IBP>(A_head, nullptr, di, dj, pr.lda, pr.ldo, r, IBP * wv, l, sB, sC, sS, sO);
        }
    } else {
        // Y: contracted dim dj of X, output dim di of X; its row-read tile is X's C tile and vice versa
        // the second problem's own operands (A2, O2) are plain (BH,N,w) tensors
        const u16 *A_head = pr.A2 + (size_t)wi.bh * N * dj;
        if constexpr (IBP == 2) {
            if (wv == OWP)
                output_role<TR, D, D, PF, 2, false, false, 1, true>(A_head, nullptr, dj, di, dj, di, r, 0, l, sC, sB, sS, sO + SO);
            else
                output_role<TR, D, D, PF, 2, false, false, 2, true>(A_head, nullptr, dj, di, dj, di, r, 0, l, sC, sB, sS, sO + SO);
        } else {
            output_role<TR, D, D, PF, IBP, false, false, 0, true>(A_head, nullptr, dj, di, dj, di, r, IBP * (wv - OWP), l, sC,
                                                                  sB, sS, sO + SO);
        }
    }
}

// Non-causal apply pass: out = A * S_total for one group of chunks, the state taken from slot 0 of
// the head and held as 16-bit A-operand tiles in LDS.  Wavefront w owns rows 16w..16w+15 of a chunk.
template <class TR, int DI, int DJ, int PF>
__global__ __launch_bounds__(kThreads) void apply_kernel(ProblemSet set, int BH, int N, int nchunks, int cpg, int G) {
    using TL = Tiling<DI, DJ>;
    __shared__ __attribute__((aligned(16))) u16 sS[DJ * TL::SS];
    __shared__ __attribute__((aligned(16))) u16 sOw[kChunk * TL::CS];  // 16 staging rows per wavefront for its outputs
    const int tid = threadIdx.x, l = tid & 63, g = l >> 4, m = l & 15;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const WorkItem wi = decode_workgroup(set.count, BH, set.xcds);
    if (wi.grp >= G) return;
    const Problem &pr = set.p[wi.prob];
    const int di = pr.di, dj = pr.dj, lda = pr.lda, ldo = pr.ldo;
    const rsrc_t rA = make_rsrc(pr.A + head_base(pr.bsA, pr.hsA, pr.H, wi.bh), ((uint32_t)(N - 1) * lda + di) * 2u);
    const rsrc_t rO = make_rsrc(pr.O + head_base(pr.bsO, pr.hsO, pr.H, wi.bh), ((uint32_t)(N - 1) * ldo + dj) * 2u);
    const int p0 = wi.grp * cpg;
    const int p1 = min(p0 + cpg, nchunks);
    {
        const f32x4 *gs = reinterpret_cast<const f32x4 *>(pr.gstate + (size_t)wi.bh * G * set.sub * TL::STATE_FLOATS);
#pragma unroll
        for (int u = 0; u < TL::TPW; ++u) {
            const f32x4 sv = gs[(w * TL::TPW + u) * 64 + l];
            const int t = w * TL::TPW + u;
            const int it = t / TL::NJT, jt = t % TL::NJT;
            u32x2 pk = {TR::pack2(sv[0], sv[1]), TR::pack2(sv[2], sv[3])};
            *reinterpret_cast<u32x2 *>(sS + (16 * jt + m) * TL::SS + 16 * it + 4 * g) = pk;
        }
    }
    u32x4 qn[PF][TL::KS];
    auto load_q = [&](int s, int p) __attribute__((always_inline)) {
        const int row = min(p, p1 - 1) * kChunk + 16 * w + m;
#pragma unroll
        for (int ks = 0; ks < TL::KS; ++ks) qn[s][ks] = buf_load16(rA, (uint32_t)(row * lda + 32 * ks + 8 * g) * 2u);
    };
#pragma unroll
    for (int s = 0; s < PF; ++s) load_q(s, p0 + s);
    __syncthreads();
    u32x4 sf[TL::NJT][TL::KS];  // this wavefront reads the whole state once
#pragma unroll
    for (int jt = 0; jt < TL::NJT; ++jt)
#pragma unroll
        for (int ks = 0; ks < TL::KS; ++ks)
            sf[jt][ks] = *reinterpret_cast<const u32x4 *>(sS + (16 * jt + m) * TL::SS + 32 * ks + 8 * g);
    run_rounds<PF>(p0, p1, [&](int s, int p) __attribute__((always_inline)) {
        {
            u32x4 qc[TL::KS];
#pragma unroll
            for (int ks = 0; ks < TL::KS; ++ks) qc[ks] = (32 * ks + 8 * g < di) ? qn[s][ks] : u32x4{0u, 0u, 0u, 0u};
            load_q(s, p + PF);
            // (outputs staged per wavefront and stored as 16-byte pieces of whole rows, as in noncausal_kernel)
            u16 *sW = sOw + (16 * w) * TL::CS;
#pragma unroll
            for (int jt = 0; jt < TL::NJT; ++jt) {
                f32x4 o = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < TL::KS; ++ks) o = TR::mfma(sf[jt][ks], qc[ks], o);
                *reinterpret_cast<u32x2 *>(sW + m * TL::CS + 16 * jt + 4 * g) = u32x2{TR::pack2(o[0], o[1]), TR::pack2(o[2], o[3])};
            }
            constexpr int PPR = DJ / 8;  // 16-byte pieces per row
#pragma unroll
            for (int u = 0; u < DJ / 32; ++u) {
                const int v = l + 64 * u, lrow = v / PPR, col = (v % PPR) * 8;
                const u32x4 val = *reinterpret_cast<const u32x4 *>(sW + lrow * TL::CS + col);
                const uint32_t off = (col < dj) ? (uint32_t)((p * kChunk + 16 * w + lrow) * ldo + col) * 2u : kOobOffset;
                __builtin_amdgcn_raw_buffer_store_b128(val, rO, (int)off, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);  // keep the next chunk's waits out of this one
        }
    });
}

// Non-causal form for a head that one workgroup handles alone (no sequence groups): pass 1 sums
// S = B^T C over the whole sequence in fp32 accumulators (the group_state loop), pass 2 applies
// out = A S chunk by chunk with the 16-bit state held in registers.  No workspace, one launch.
// PF2: chunks of A rows in flight in pass 2.  PF2 > PF: the first PF2 chunks are requested before pass 1 starts instead
// of at the hand-over (sequences of 4 to 8 chunks, three gradient problems per head: B32 H12 N512 D64 gradients 46.6 -> 43.0 us;
// the forward pass alone loses 0.7 us of 21.4 with it and keeps PF2 = PF; 3, 4 and 6 chunks measured alike, 8 worse).
// PREP: A, B, C are the raw projections; their rows are normalised (A, B), scaled (C) and masked on the way in
// (PrepSide, no rotation) and the prepared tensors are written to qo / ko / vo for the backward pass.  A column half
// (c0 > 0) prepares the same A and B rows as its twin and leaves writing them to the first half.
template <class TR, int DI, int DJ, int PF, int PF2 = PF, bool PREP = false>
__global__ __launch_bounds__(kThreads) void noncausal_kernel(ProblemSet set, int BH, int N, int nchunks, PrepSide prep) {
    using TL = Tiling<DI, DJ>;
    constexpr int SB = kChunk * TL::BS, SC = kChunk * TL::CS;
    constexpr int NB = DI / 32, NC = DJ / 32;  // 16-byte pieces per thread of a B / C tile
    static_assert(!PREP || PF2 == PF, "the preparing variant keeps one prefetch depth");
    __shared__ __attribute__((aligned(16))) u16 sB[2 * SB];
    __shared__ __attribute__((aligned(16))) u16 sC[2 * SC];
    __shared__ __attribute__((aligned(16))) u16 sS[DJ * TL::SS];
    const int tid = threadIdx.x, l = tid & 63, g = l >> 4, m = l & 15;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const WorkItem wi = decode_workgroup(set.count, BH, set.xcds);
    if (wi.grp >= 1) return;
    const Problem &pr = set.p[wi.prob];
    const int di = pr.di, dj = pr.dj, lda = pr.lda, ldb = pr.ldb, ldc = pr.ldc, ldo = pr.ldo;
    const rsrc_t rA = make_rsrc(pr.A + head_base(pr.bsA, pr.hsA, pr.H, wi.bh), ((uint32_t)(N - 1) * lda + di) * 2u);
    const rsrc_t rB = make_rsrc(pr.B + head_base(pr.bsB, pr.hsB, pr.H, wi.bh), ((uint32_t)(N - 1) * ldb + di) * 2u);
    const rsrc_t rC = make_rsrc(pr.C + head_base(pr.bsC, pr.hsC, pr.H, wi.bh), ((uint32_t)(N - 1) * ldc + dj) * 2u);
    const rsrc_t rO = make_rsrc(pr.O + head_base(pr.bsO, pr.hsO, pr.H, wi.bh), ((uint32_t)(N - 1) * ldo + dj) * 2u);
    // PREP: side inputs of this head's batch element and the prepared tensors, (B,H,N,width)
    const bool first_half = pr.c0 == 0;
    const uint32_t qk_bytes = (PREP && first_half) ? (uint32_t)N * di * 2u : 0u;
    const rsrc_t rQo = make_rsrc(PREP && prep.qo ? prep.qo + (size_t)wi.bh * N * di : nullptr, prep.qo ? qk_bytes : 0u);
    const rsrc_t rKo = make_rsrc(PREP && prep.ko ? prep.ko + (size_t)wi.bh * N * di : nullptr, prep.ko ? qk_bytes : 0u);
    const rsrc_t rVo = make_rsrc(PREP && prep.vo ? prep.vo + (size_t)wi.bh * N * prep.dv + pr.c0 : nullptr,
                                 (PREP && prep.vo) ? ((uint32_t)(N - 1) * prep.dv + dj) * 2u : 0u);
    const size_t tok0 = PREP ? (size_t)(wi.bh / prep.H) * N : 0;
    const bool scaled = PREP && prep.cnt != nullptr && prep.sig != nullptr;
    const float sig = scaled ? prep.sig[wi.bh % prep.H] : 0.f;

    u32x4 qn[PF2][TL::KS];
    uint32_t keep_q[PF2];
    auto load_q = [&](int s, int p) __attribute__((always_inline)) {
        const int row = min(p, nchunks - 1) * kChunk + 16 * w + m;
#pragma unroll
        for (int ks = 0; ks < TL::KS; ++ks) qn[s][ks] = buf_load16(rA, (uint32_t)(row * lda + 32 * ks + 8 * g) * 2u);
        if constexpr (PREP) keep_q[s] = prep.keep != nullptr ? (uint32_t)prep.keep[tok0 + min(row, N - 1)] : 1u;
    };

    // ---- pass 1: S = sum over all chunks of B_c^T C_c
    f32x4 S[TL::TPW];
#pragma unroll
    for (int u = 0; u < TL::TPW; ++u) S[u] = f32x4{0.f, 0.f, 0.f, 0.f};
    {
        u32x4 rb[PF][NB], rc[PF][NC];
        uint32_t keep_b[PF][NB], keep_c[PF][NC];  // the bytes as loaded: converting them at once would wait for the load
        float cnt_c[PF][NC];
        auto load_chunk = [&](int s, int p) __attribute__((always_inline)) {
            const int row0 = min(p, nchunks - 1) * kChunk;
            load_tile<DI>(rb[s], rB, row0, ldb, tid);
            load_tile<DJ>(rc[s], rC, row0, ldc, tid);
            if constexpr (PREP) {
#pragma unroll
                for (int u = 0; u < NB; ++u) {
                    const int srow = min(row0 + (tid + kThreads * u) / (DI / 8), N - 1);
                    keep_b[s][u] = prep.keep != nullptr ? (uint32_t)prep.keep[tok0 + srow] : 1u;
                }
#pragma unroll
                for (int u = 0; u < NC; ++u) {
                    const int srow = min(row0 + (tid + kThreads * u) / (DJ / 8), N - 1);
                    keep_c[s][u] = prep.keep != nullptr ? (uint32_t)prep.keep[tok0 + srow] : 1u;
                    cnt_c[s][u] = scaled ? prep.cnt[tok0 + srow] : 0.f;
                }
            }
        };
        // registers of stage s (chunk p) -> LDS tiles tb, tc; PREP: prepared on the way, and out to ko / vo
        auto stage = [&](int s, int p, u16 *tb, u16 *tc) __attribute__((always_inline)) {
            if constexpr (!PREP) {
                store_tile<DI, TL::BS>(tb, rb[s], di, tid);
                store_tile<DJ, TL::CS>(tc, rc[s], dj, tid);
            } else {
                const int row0 = min(p, nchunks - 1) * kChunk;
#pragma unroll
                for (int u = 0; u < NB; ++u) {
                    const int v = tid + kThreads * u;
                    const int lrow = v / (DI / 8), col = (v % (DI / 8)) * 8;
                    float x[8];
                    unpack8<TR>(rb[s][u], x);
                    float ss = 0.f;
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        if (col >= di) x[e] = 0.f;
                        ss += x[e] * x[e];
                    }
                    ss = lane_group_sum<DI / 8>(ss);
                    const float nrm = __builtin_amdgcn_sqrtf(ss);
                    const float mul = (float)keep_b[s][u] * __builtin_amdgcn_rcpf(nrm > prep.eps ? nrm : prep.eps);
#pragma unroll
                    for (int e = 0; e < 8; ++e) x[e] *= mul;
                    const u32x4 y = pack8<TR>(x);
                    *reinterpret_cast<u32x4 *>(tb + lrow * TL::BS + col) = y;
                    const uint32_t off = (col < di && p < nchunks) ? (uint32_t)((row0 + lrow) * di + col) * 2u : kOobOffset;
                    __builtin_amdgcn_raw_buffer_store_b128(y, rKo, (int)off, 0, 0);
                }
#pragma unroll
                for (int u = 0; u < NC; ++u) {
                    const int v = tid + kThreads * u;
                    const int lrow = v / (DJ / 8), col = (v % (DJ / 8)) * 8;
                    float x[8];
                    unpack8<TR>(rc[s][u], x);
                    const float mul = (col < dj) ? value_scale((float)keep_c[s][u], cnt_c[s][u], sig, scaled) : 0.f;
#pragma unroll
                    for (int e = 0; e < 8; ++e) x[e] *= mul;
                    const u32x4 y = (col < dj) ? pack8<TR>(x) : u32x4{0u, 0u, 0u, 0u};
                    *reinterpret_cast<u32x4 *>(tc + lrow * TL::CS + col) = y;
                    const uint32_t off = (col < dj && p < nchunks) ? (uint32_t)((row0 + lrow) * prep.dv + col) * 2u : kOobOffset;
                    __builtin_amdgcn_raw_buffer_store_b128(y, rVo, (int)off, 0, 0);
                }
            }
        };
#pragma unroll
        for (int s = 0; s < PF; ++s) load_chunk(s, s);
        if constexpr (PF2 != PF) {
#pragma unroll
            for (int s = 0; s < PF2; ++s) load_q(s, s);
        }
        stage(0, 0, sB, sC);
        load_chunk(0, PF);
        __syncthreads();
        run_rounds<PF>(0, nchunks, [&](int s, int p) __attribute__((always_inline)) {
            const int s1 = (s + 1) % PF;
            const int buf = p & 1;
            stage(s1, p + 1, sB + (buf ^ 1) * SB, sC + (buf ^ 1) * SC);
            load_chunk(s1, p + 1 + PF);
            state_update<TR, DI, DJ>(S, sB + buf * SB, sC + buf * SC, w, g, m);
            chunk_barrier();
        });
    }
    if constexpr (PF2 == PF) {
#pragma unroll
        for (int s = 0; s < PF2; ++s) load_q(s, s);  // in flight while the state is converted
    }

    // ---- hand-over: 16-bit state, transposed to [j][i], through LDS into every wavefront's registers
#pragma unroll
    for (int u = 0; u < TL::TPW; ++u) {
        const int t = w * TL::TPW + u;
        const int it = t / TL::NJT, jt = t % TL::NJT;
        u32x2 pk = {TR::pack2(S[u][0], S[u][1]), TR::pack2(S[u][2], S[u][3])};
        *reinterpret_cast<u32x2 *>(sS + (16 * jt + m) * TL::SS + 16 * it + 4 * g) = pk;
    }
    __syncthreads();
    u32x4 sf[TL::NJT][TL::KS];
#pragma unroll
    for (int jt = 0; jt < TL::NJT; ++jt)
#pragma unroll
        for (int ks = 0; ks < TL::KS; ++ks)
            sf[jt][ks] = *reinterpret_cast<const u32x4 *>(sS + (16 * jt + m) * TL::SS + 32 * ks + 8 * g);

    // ---- pass 2: out_c = A_c S
    run_rounds<PF2>(0, nchunks, [&](int s, int p) __attribute__((always_inline)) {
        {
            u32x4 qc[TL::KS];
#pragma unroll
            for (int ks = 0; ks < TL::KS; ++ks) qc[ks] = (32 * ks + 8 * g < di) ? qn[s][ks] : u32x4{0u, 0u, 0u, 0u};
            const int orow = p * kChunk + 16 * w + m;
            if constexpr (PREP) {
                // a row of A lives in the four lanes m, m + 16, m + 32, m + 48 (eight columns of every 32 each)
                float x[TL::KS][8];
                float ss = 0.f;
#pragma unroll
                for (int ks = 0; ks < TL::KS; ++ks) {
                    unpack8<TR>(qc[ks], x[ks]);
#pragma unroll
                    for (int e = 0; e < 8; ++e) ss += x[ks][e] * x[ks][e];
                }
                ss += __shfl_xor(ss, 16, 64);
                ss += __shfl_xor(ss, 32, 64);
                const float nrm = __builtin_amdgcn_sqrtf(ss);
                const float mul = (float)keep_q[s] * __builtin_amdgcn_rcpf(nrm > prep.eps ? nrm : prep.eps);
#pragma unroll
                for (int ks = 0; ks < TL::KS; ++ks) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) x[ks][e] *= mul;
                    qc[ks] = pack8<TR>(x[ks]);
                    const int col = 32 * ks + 8 * g;
                    const uint32_t off = (col < di) ? (uint32_t)(orow * di + col) * 2u : kOobOffset;
                    __builtin_amdgcn_raw_buffer_store_b128(qc[ks], rQo, (int)off, 0, 0);
                }
            }
            if (PF2 == PF || p + PF2 < nchunks) load_q(s, p + PF2);
            // The 16 output rows of this wavefront go through its own staging rows in the first C tile (free since the
            // hand-over) and leave as 16-byte pieces of whole rows: 8-byte accumulator pieces written straight to
            // memory are quarter cache lines that have to meet in L2.  (One wavefront's LDS accesses execute in order.)
            u16 *sW = sC + (16 * w) * TL::CS;
#pragma unroll
            for (int jt = 0; jt < TL::NJT; ++jt) {
                f32x4 o = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < TL::KS; ++ks) o = TR::mfma(sf[jt][ks], qc[ks], o);
                *reinterpret_cast<u32x2 *>(sW + m * TL::CS + 16 * jt + 4 * g) = u32x2{TR::pack2(o[0], o[1]), TR::pack2(o[2], o[3])};
            }
            constexpr int PPR = DJ / 8;  // 16-byte pieces per row
#pragma unroll
            for (int u = 0; u < DJ / 32; ++u) {
                const int v = l + 64 * u, lrow = v / PPR, col = (v % PPR) * 8;
                const u32x4 val = *reinterpret_cast<const u32x4 *>(sW + lrow * TL::CS + col);
                const uint32_t off = (col < dj) ? (uint32_t)((p * kChunk + 16 * w + lrow) * ldo + col) * 2u : kOobOffset;
                __builtin_amdgcn_raw_buffer_store_b128(val, rO, (int)off, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);  // keep the next chunk's waits out of this one
        }
    });
}

}  // namespace cott
