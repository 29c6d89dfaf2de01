// Fused input preparation of the cosine-attention module and its backward: L2-normalise the rows
// of q and k, scale the rows of v by 1 / max(cnt^sig, 1), multiply all three by the 0/1 keep mask
// and convert to the dtype the attention kernels run in -- one pass over each tensor
// (GPT_Trainer/GPTCosAttention.py:229-248, BERT_Trainer/BertCosAttention.py:162-178 do this with
// eight separate elementwise / reduction kernels).  Bandwidth-bound: every element is read once
// and written once, rows are reduced with lane shuffles inside a wavefront.
#include "cott_common.h"
#include "cott_launch.h"
#include "../../include/cottention.h"

namespace cott {
namespace {

constexpr int kPrepThreads = 256;
constexpr int kMaxVec = 4;  // a lane holds up to kMaxVec groups of 4 elements of its row: rows of up to 1024 elements

template <class ACC>
struct Vec4 {
    ACC x[4];
};

template <class ACC>
__device__ __forceinline__ Vec4<ACC> load4(const void *base, int dtype, size_t idx) {
    Vec4<ACC> r;
    switch (dtype) {
        case COTT_F32: {
            const f32x4 v = *reinterpret_cast<const f32x4 *>(static_cast<const float *>(base) + idx);
#pragma unroll
            for (int i = 0; i < 4; ++i) r.x[i] = (ACC)v[i];
            break;
        }
        case COTT_F64: {
            const double *p = static_cast<const double *>(base) + idx;
#pragma unroll
            for (int i = 0; i < 4; ++i) r.x[i] = (ACC)p[i];
            break;
        }
        case COTT_F16: {
            const u32x2 v = *reinterpret_cast<const u32x2 *>(static_cast<const u16 *>(base) + idx);
            r.x[0] = (ACC)Fp16::to_float((u16)(v.x & 0xffffu));
            r.x[1] = (ACC)Fp16::to_float((u16)(v.x >> 16));
            r.x[2] = (ACC)Fp16::to_float((u16)(v.y & 0xffffu));
            r.x[3] = (ACC)Fp16::to_float((u16)(v.y >> 16));
            break;
        }
        default: {
            const u32x2 v = *reinterpret_cast<const u32x2 *>(static_cast<const u16 *>(base) + idx);
            r.x[0] = (ACC)Bf16::to_float((u16)(v.x & 0xffffu));
            r.x[1] = (ACC)Bf16::to_float((u16)(v.x >> 16));
            r.x[2] = (ACC)Bf16::to_float((u16)(v.y & 0xffffu));
            r.x[3] = (ACC)Bf16::to_float((u16)(v.y >> 16));
            break;
        }
    }
    return r;
}

template <class ACC>
__device__ __forceinline__ void store4(void *base, int dtype, size_t idx, const Vec4<ACC> &v) {
    switch (dtype) {
        case COTT_F32: {
            f32x4 o = {(float)v.x[0], (float)v.x[1], (float)v.x[2], (float)v.x[3]};
            *reinterpret_cast<f32x4 *>(static_cast<float *>(base) + idx) = o;
            break;
        }
        case COTT_F64: {
            double *p = static_cast<double *>(base) + idx;
#pragma unroll
            for (int i = 0; i < 4; ++i) p[i] = (double)v.x[i];
            break;
        }
        case COTT_F16: {
            u32x2 o = {Fp16::pack2((float)v.x[0], (float)v.x[1]), Fp16::pack2((float)v.x[2], (float)v.x[3])};
            *reinterpret_cast<u32x2 *>(static_cast<u16 *>(base) + idx) = o;
            break;
        }
        default: {
            u32x2 o = {Bf16::pack2((float)v.x[0], (float)v.x[1]), Bf16::pack2((float)v.x[2], (float)v.x[3])};
            *reinterpret_cast<u32x2 *>(static_cast<u16 *>(base) + idx) = o;
            break;
        }
    }
}

// Sum over the `lpr` (power of two, <= 64) consecutive lanes that hold one row.
__device__ __forceinline__ double row_sum(double v, int lpr) {
    for (int off = 1; off < lpr; off <<= 1) v += __shfl_xor(v, off, 64);
    return v;
}
// fp32: the steps inside a row of 16 lanes are data-parallel-primitive moves in the vector ALU (quad swaps, then the
// mirrored half row and row, whose other half already holds its partial sum in every lane); only rows of 32 or 64
// lanes go on through LDS permutes.
template <int CTRL>
__device__ __forceinline__ float dpp_moved(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ float row_sum(float v, int lpr) {
    if (lpr >= 2) v += dpp_moved<0xB1>(v);    // lanes 1,0,3,2 of each quad
    if (lpr >= 4) v += dpp_moved<0x4E>(v);    // lanes 2,3,0,1
    if (lpr >= 8) v += dpp_moved<0x141>(v);   // mirrored half row
    if (lpr >= 16) v += dpp_moved<0x140>(v);  // mirrored row
    for (int off = 16; off < lpr; off <<= 1) v += __shfl_xor(v, off, 64);
    return v;
}

struct PrepArgs {
    const void *x[3];    // q, k, v as given
    const void *g[3];    // backward: gradients with respect to the prepared tensors
    void *y[3];          // forward: prepared tensors; backward: gradients with respect to q, k, v
    const uint8_t *keep; // (B,N) 0/1 or null
    const float *cnt;    // (B,N) or null
    const float *sig;    // (H) or null
    float *dsig_rows;    // backward: (B,H,N) per-row derivative with respect to sig[h], or null
    long rows;           // B*H*N
    int H, N, dk, dv;
    int x_dtype, y_dtype, g_dtype;
    int lpr[3];          // lanes per row of q, k, v
    float eps;
    // Optional extras: q, k, v given as (B,N,H,D) (the layout the projections produce) instead of
    // (B,H,N,D), and the GPT-J rotary embedding applied to the first R columns of q and k.
    int x_bnhd;           // 1: x (and, backward, y) are (B,N,H,D); g (backward) / y (forward) stay (B,H,N,D)
    const float *rot;     // (P,R) table, row p = [sin(p f_0..f_{R/2-1}) | cos(...)], or null
    const long long *pos; // (B,N) row of the table per position (clamped to the table)
    int R, table_rows;
};

// Rotates the pairs (v[0],v[1]) and (v[2],v[3]) by +angle (inverse = false) or -angle; sn and cs hold the sines
// and cosines of the two pairs.
typedef __attribute__((ext_vector_type(2))) float f32x2;
template <class ACC>
__device__ __forceinline__ void rotate4(Vec4<ACC> &v, f32x2 sn, f32x2 cs, bool inverse) {
#pragma unroll
    for (int p = 0; p < 2; ++p) {
        const ACC s = inverse ? -(ACC)sn[p] : (ACC)sn[p], c = (ACC)cs[p];
        const ACC e = v.x[2 * p], o = v.x[2 * p + 1];
        v.x[2 * p] = e * c - o * s;
        v.x[2 * p + 1] = o * c + e * s;
    }
}

// Per-row scalars in fp32 use the hardware reciprocal and square root (1 ulp, no denormal fix-up sequences: the
// operands are clamped away from the denormal range); every lane of a row repeats them, and for head-sized
// rows the kernel is bound by instruction issue.
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }
__device__ __forceinline__ double fast_rcp(double x) { return 1.0 / x; }
__device__ __forceinline__ float fast_sqrt(float x) { return __builtin_amdgcn_sqrtf(x); }
__device__ __forceinline__ double fast_sqrt(double x) { return sqrt(x); }

// (hardware exp2 / log2: about 1e-6 relative, far inside the fp32 tolerance of the op)
__device__ __forceinline__ float pow_pos(float c, float s) { return c > 0.f ? __expf(s * __logf(c)) : 0.f; }
__device__ __forceinline__ double pow_pos(double c, double s) { return c > 0.0 ? exp(s * log(c)) : 0.0; }

// row = (b*H + h)*N + s.  Row counts below 2^32 (every realistic shape) take 32-bit divisions, which cost a
// fraction of the 64-bit ones.
__device__ __forceinline__ void split_row(long row, const PrepArgs &a, int &s, int &h, int &b) {
    if (a.rows <= 0xffffffffL) {
        const uint32_t r = (uint32_t)row, bh = r / (uint32_t)a.N;
        s = (int)(r - bh * (uint32_t)a.N);
        b = (int)(bh / (uint32_t)a.H);
        h = (int)(bh - (uint32_t)b * (uint32_t)a.H);
    } else {
        const long bh = row / a.N;
        s = (int)(row % a.N);
        h = (int)(bh % a.H);
        b = (int)(bh / a.H);
    }
}

// blockIdx.y selects the tensor (0 q, 1 k, 2 v).  A row of D elements lives in lpr consecutive
// lanes, 4 elements per lane and group; groups c = 0..NV-1 cover D up to 4*64*NV.  Each lane group
// handles R rows (row, row + stride, ...) whose loads are all issued before the first use, so that
// enough bytes are in flight per wavefront to cover the memory latency.  For head-sized rows the kernel is
// limited by instruction issue, not by bytes: the per-row work (index split, norm, division) is repeated by
// every lane of the row, so two groups per lane (half as many wavefronts) are faster than one, while more
// rows or groups per lane only cost registers.
// PAIRED (with ALL_BF16, NV == 2, row widths multiples of 8): the two groups of a lane are neighbours, columns 8 l .. 8 l + 7,
// and travel as one 16-byte load or store instead of two 8-byte ones (the kernel is bound by instruction issue).
template <class ACC, bool BACKWARD, int NV, int R, bool ALL_BF16 = false, bool PAIRED = false>
__global__ __launch_bounds__(kPrepThreads) void prep_kernel(PrepArgs a) {
    static_assert(!PAIRED || (ALL_BF16 && NV == 2), "paired groups: bf16 tensors, two groups per lane");
    // ALL_BF16: every tensor is bf16, known at compile time: no type dispatch around the loads and stores (the block's
    // shapes, B8 H16 N2048 D64 in the projections' layout with rotary, mask and scale: forward 48.5 -> 44.8 us,
    // backward 97.8 -> 91.5 us per call)
    const int x_dtype = ALL_BF16 ? (int)COTT_BF16 : a.x_dtype, y_dtype = ALL_BF16 ? (int)COTT_BF16 : a.y_dtype,
              g_dtype = ALL_BF16 ? (int)COTT_BF16 : a.g_dtype;
    const int t = blockIdx.y;
    const int D = t < 2 ? a.dk : a.dv;
    const int lpr = a.lpr[t];
    const int rpb = kPrepThreads / lpr;
    const long row0 = ((long)blockIdx.x * R) * rpb + threadIdx.x / lpr;
    const int lane = threadIdx.x % lpr;
    auto col_of = [&](int c) __attribute__((always_inline)) { return PAIRED ? 4 * (lane * NV + c) : 4 * (lane + c * lpr); };
    auto unpack_pair = [&](u32x4 v, Vec4<ACC> &lo, Vec4<ACC> &hi) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            lo.x[2 * i] = (ACC)Bf16::to_float((u16)(v[i] & 0xffffu));
            lo.x[2 * i + 1] = (ACC)Bf16::to_float((u16)(v[i] >> 16));
            hi.x[2 * i] = (ACC)Bf16::to_float((u16)(v[2 + i] & 0xffffu));
            hi.x[2 * i + 1] = (ACC)Bf16::to_float((u16)(v[2 + i] >> 16));
        }
    };

    Vec4<ACC> x[R][NV], g[R][NV];
    long rr[R];
    size_t xoff[R];
    bool act[R];
    const bool rotary = t < 2 && a.rot != nullptr;
    const bool side = t == 2 && a.cnt != nullptr && a.sig != nullptr;
    // Three rounds of loads, all issued before the first use: the per-row side inputs, the rows themselves, then
    // the table entries (which need the positions of the first round, back long before the rows are).
    uint8_t keep_in[R];
    long long pos_in[R];
    float cnt_in[R], sig_in[R];
#pragma unroll
    for (int u = 0; u < R; ++u) {
        const long row = row0 + (long)u * rpb;
        act[u] = row < a.rows;
        rr[u] = act[u] ? row : 0;
        int sq, hq, bq;  // position, head, batch element of the row
        split_row(rr[u], a, sq, hq, bq);
        xoff[u] = a.x_bnhd ? (size_t)(((long)bq * a.N + sq) * a.H + hq) * D : (size_t)rr[u] * D;
        const long tok = (long)bq * a.N + sq;
        keep_in[u] = a.keep != nullptr ? a.keep[tok] : (uint8_t)1;
        pos_in[u] = rotary ? a.pos[tok] : 0;
        cnt_in[u] = side ? a.cnt[tok] : 0.f;
        sig_in[u] = side ? a.sig[hq] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < R; ++u) {
        if constexpr (PAIRED) {
            const int col = col_of(0);
            u32x4 xv = {0u, 0u, 0u, 0u}, gv = xv;
            if (act[u] && col < D) {
                xv = *reinterpret_cast<const u32x4 *>(static_cast<const u16 *>(a.x[t]) + xoff[u] + col);
                if (BACKWARD) gv = *reinterpret_cast<const u32x4 *>(static_cast<const u16 *>(a.g[t]) + (size_t)rr[u] * D + col);
            }
            unpack_pair(xv, x[u][0], x[u][NV - 1]);
            if (BACKWARD) unpack_pair(gv, g[u][0], g[u][NV - 1]);
            continue;
        }
#pragma unroll
        for (int c = 0; c < NV; ++c) {
            const int col = col_of(c);
            if (act[u] && col < D) {
                x[u][c] = load4<ACC>(a.x[t], x_dtype, xoff[u] + col);
                if (BACKWARD) g[u][c] = load4<ACC>(a.g[t], g_dtype, (size_t)rr[u] * D + col);
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    x[u][c].x[i] = 0;
                    if (BACKWARD) g[u][c].x[i] = 0;
                }
            }
        }
    }
    // sines and cosines of a lane's pairs: two 8-byte loads per group (its column is a multiple of 4)
    f32x2 sn[R][NV], cs[R][NV];
    if (rotary) {
#pragma unroll
        for (int u = 0; u < R; ++u) {
            long long tp = pos_in[u];
            tp = tp < 0 ? 0 : (tp >= a.table_rows ? a.table_rows - 1 : tp);  // never read outside the table
            const float *sc = a.rot + (size_t)tp * a.R;
#pragma unroll
            for (int c = 0; c < NV; ++c) {
                const int col = col_of(c);
                if (col < a.R) {
                    sn[u][c] = *reinterpret_cast<const f32x2 *>(sc + col / 2);
                    cs[u][c] = *reinterpret_cast<const f32x2 *>(sc + col / 2 + a.R / 2);
                }
            }
        }
    }
#pragma unroll
    for (int u = 0; u < R; ++u) {
        const long r = rr[u];
        const ACC keep = keep_in[u] != 0 ? (ACC)1 : (ACC)0;
        // y = keep R x / |R x| with R the block rotation built from the table (orthogonal only up to the table's
        // rounding, so the norm is taken after the rotation).  Backward: dx = R^T J^T g with J the Jacobian of
        // the normalisation at x' = R x: the usual combination of g and x', rotated back at the end.
        if (rotary) {
#pragma unroll
            for (int c = 0; c < NV; ++c) {
                const int col = col_of(c);
                if (col < a.R) rotate4(x[u][c], sn[u][c], cs[u][c], false);
            }
        }
        ACC ss = 0, dot = 0;
#pragma unroll
        for (int c = 0; c < NV; ++c)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                ss += x[u][c].x[i] * x[u][c].x[i];
                if (BACKWARD) dot += x[u][c].x[i] * g[u][c].x[i];
            }
        ACC mul_x = 0, mul_g = 0;  // y = mul_x * x (forward);  dx = mul_g * g + mul_x * x (backward)
        if (t < 2) {
            ss = row_sum(ss, lpr);
            const ACC nrm = fast_sqrt(ss);
            const ACC den = nrm > (ACC)a.eps ? nrm : (ACC)a.eps;
            const ACC rden = fast_rcp(den);
            if (!BACKWARD) {
                mul_x = keep * rden;
            } else {
                dot = row_sum(dot, lpr);
                mul_g = keep * rden;
                // d/dx of x / max(|x|, eps): the norm term only exists where the norm is not clamped
                mul_x = nrm > (ACC)a.eps ? -keep * dot * (rden * rden * rden) : (ACC)0;
            }
        } else {
            ACC scale = 1;
            bool scaled = false;
            ACC c = 0;
            if (a.cnt != nullptr && a.sig != nullptr) {
                c = (ACC)cnt_in[u];
                const ACC p = pow_pos(c, (ACC)sig_in[u]);
                if (p > (ACC)1) {
                    scale = fast_rcp(p);
                    scaled = true;
                }
            }
            if (!BACKWARD) {
                mul_x = keep * scale;
            } else {
                mul_g = keep * scale;
                if (a.dsig_rows != nullptr) {
                    // y = x c^-sig  ->  dy/dsig = -ln(c) y ; zero where the scale is clamped to 1
                    dot = row_sum(dot, lpr);
                    if (act[u] && lane == 0) a.dsig_rows[r] = scaled ? (float)(-log(c) * keep * scale * dot) : 0.f;
                }
            }
        }
        u32x4 ypair;
#pragma unroll
        for (int c = 0; c < NV; ++c) {
            const int col = col_of(c);
            if (act[u] && col < D) {
                Vec4<ACC> y;
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    y.x[i] = BACKWARD ? mul_g * g[u][c].x[i] + mul_x * x[u][c].x[i] : mul_x * x[u][c].x[i];
                if (BACKWARD && rotary && col < a.R) rotate4(y, sn[u][c], cs[u][c], true);
                if constexpr (PAIRED) {
                    ypair[2 * c] = Bf16::pack2((float)y.x[0], (float)y.x[1]);
                    ypair[2 * c + 1] = Bf16::pack2((float)y.x[2], (float)y.x[3]);
                } else {
                    store4<ACC>(a.y[t], BACKWARD ? x_dtype : y_dtype, (BACKWARD ? xoff[u] : (size_t)r * D) + col, y);
                }
            }
        }
        if constexpr (PAIRED) {
            const int col = col_of(0);
            if (act[u] && col < D)
                *reinterpret_cast<u32x4 *>(static_cast<u16 *>(a.y[t]) + (BACKWARD ? xoff[u] : (size_t)r * D) + col) = ypair;
        }
    }
}

int lanes_per_row(int d, int nv) {
    int l = 1;
    while (4 * nv * l < d && l < 64) l <<= 1;
    return l;
}

}  // namespace

hipError_t launch_prep(bool backward, const void *const x[3], const void *const g[3], void *const y[3],
                       const uint8_t *keep, const float *cnt, const float *sig, float *dsig_rows, int B, int H, int N,
                       int dk, int dv, int x_dtype, int y_dtype, int g_dtype, float eps, int x_bnhd, const float *rot,
                       const long long *pos, int R, int table_rows, hipStream_t stream) {
    PrepArgs a;
    a.table_rows = table_rows > 0 ? table_rows : 1;
    a.x_bnhd = x_bnhd;
    a.rot = rot;
    a.pos = pos;
    a.R = R;
    for (int i = 0; i < 3; ++i) {
        a.x[i] = x[i];
        a.g[i] = g ? g[i] : nullptr;
        a.y[i] = y[i];
    }
    a.keep = keep;
    a.cnt = cnt;
    a.sig = sig;
    a.dsig_rows = dsig_rows;
    a.rows = (long)B * H * N;
    a.H = H;
    a.N = N;
    a.dk = dk;
    a.dv = dv;
    a.x_dtype = x_dtype;
    a.y_dtype = y_dtype;
    a.g_dtype = g_dtype;
    a.eps = eps;
    // one grid for the three tensors; rows per block differ per tensor, size x for the largest need
    const int big = dk > dv ? dk : dv;
    const bool wide = big > 256;              // four element groups per lane and one row instead of two and two
    const int rows_per_group = wide ? 1 : 2;
    const int nv = wide ? kMaxVec : (big > 4 ? 2 : 1);
    a.lpr[0] = a.lpr[1] = lanes_per_row(dk, nv);
    a.lpr[2] = lanes_per_row(dv, nv);
    const int min_rows = rows_per_group * kPrepThreads / (a.lpr[0] > a.lpr[2] ? a.lpr[0] : a.lpr[2]);
    const long blocks = (a.rows + min_rows - 1) / min_rows;
    if (blocks > 0x7fffffffL) return hipErrorInvalidValue;
    ProfScope prof(K_PREP, stream);
    const dim3 grid((unsigned)blocks, 3), blk(kPrepThreads);
    const bool f64 = x_dtype == COTT_F64;
    const bool all_bf16 = x_dtype == COTT_BF16 && y_dtype == COTT_BF16 && (!backward || g_dtype == COTT_BF16);
    // rows whose lanes can take 16 bytes each: widths multiples of 8 (16-byte aligned rows in either layout) that fill
    // the two groups of every lane, or leave whole lanes empty
    const bool paired = dk % 8 == 0 && dv % 8 == 0;
#define COTT_PREP(ACC, BWD) \
    do { \
        if (wide) prep_kernel<ACC, BWD, kMaxVec, 1><<<grid, blk, 0, stream>>>(a); \
        else if (nv == 2 && all_bf16 && paired) prep_kernel<float, BWD, 2, 2, true, true><<<grid, blk, 0, stream>>>(a); \
        else if (nv == 2 && all_bf16) prep_kernel<ACC, BWD, 2, 2, true><<<grid, blk, 0, stream>>>(a); \
        else if (nv == 2) prep_kernel<ACC, BWD, 2, 2><<<grid, blk, 0, stream>>>(a); \
        else prep_kernel<ACC, BWD, 1, 2><<<grid, blk, 0, stream>>>(a); \
    } while (0)
    if (backward) {
        if (f64) COTT_PREP(double, true);
        else COTT_PREP(float, true);
    } else {
        if (f64) COTT_PREP(double, false);
        else COTT_PREP(float, false);
    }
#undef COTT_PREP
    return hipGetLastError();
}

}  // namespace cott
