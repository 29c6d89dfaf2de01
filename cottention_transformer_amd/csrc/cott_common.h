// Shared device helpers for the gfx950 kernels: 16-bit storage traits, MFMA wrappers, LDS
// transposing reads and predicated global accesses.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace cott {

typedef uint16_t u16;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;

template <class To, class From>
__device__ __forceinline__ To bitcast(const From &x) {
    static_assert(sizeof(To) == sizeof(From), "bitcast size mismatch");
    return __builtin_bit_cast(To, x);
}

// v_mfma_f32_16x16x32_{bf16,f16}: D(16x16) += A(16x32) * B(32x16).  Lane l (m = l%16, g = l/16)
// holds A[m][8g..8g+7], B[8g..8g+7][m] and D[4g..4g+3][m].  Operands travel as four dwords.
struct Bf16 {
    static constexpr int kDtype = 3;
    __device__ static __forceinline__ f32x4 mfma(u32x4 a, u32x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(bitcast<bf16x8>(a), bitcast<bf16x8>(b), c, 0, 0, 0);
    }
    __device__ static __forceinline__ uint32_t pack2(float lo, float hi) {
        bf16x2 v = {(__bf16)lo, (__bf16)hi};
        return bitcast<uint32_t>(v);
    }
    __device__ static __forceinline__ float to_float(u16 x) { return bitcast<float>((uint32_t)x << 16); }
    __device__ static __forceinline__ u16 from_float(float f) { return bitcast<u16>((__bf16)f); }
};

struct Fp16 {
    static constexpr int kDtype = 2;
    __device__ static __forceinline__ f32x4 mfma(u32x4 a, u32x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(bitcast<f16x8>(a), bitcast<f16x8>(b), c, 0, 0, 0);
    }
    __device__ static __forceinline__ uint32_t pack2(float lo, float hi) {
        f16x2 v = {(_Float16)lo, (_Float16)hi};
        return bitcast<uint32_t>(v);
    }
    __device__ static __forceinline__ float to_float(u16 x) { return (float)bitcast<_Float16>(x); }
    __device__ static __forceinline__ u16 from_float(float f) { return bitcast<u16>((_Float16)f); }
};

// ds_read_b64_tr_b16: the 16 lanes of a quarter-wave each supply the address of four consecutive
// 16-bit elements (one row of a 16x4 block); lane i of the quarter receives elements
// block[4t + i/4][i%4], t = 0..3.  With lane i pointing at tile[k0 + i/4][c0 + 4*(i%4)] the lane
// ends up with tile[k0 + t][c0 + i], t = 0..3: four consecutive rows of ONE column, which is
// the MFMA operand order when the contraction runs down the rows of a row-major tile.
__device__ __forceinline__ u32x2 lds_read_tr16(const u16 *p) {
    s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *)p);
    return bitcast<u32x2>(v);
}

// Column fragment of a row-major LDS tile for lane column `m` (0..15): rows k0..k0+3 of column c0+m.
__device__ __forceinline__ u32x2 lds_col4(const u16 *tile, int stride, int k0, int c0, int m) {
    return lds_read_tr16(tile + (k0 + (m >> 2)) * stride + c0 + 4 * (m & 3));
}

__device__ __forceinline__ u32x4 cat(u32x2 lo, u32x2 hi) {
    u32x4 r = {lo.x, lo.y, hi.x, hi.y};
    return r;
}

__device__ __forceinline__ u32x4 ld_global16(const u16 *p, bool ok) {
    u32x4 z = {0u, 0u, 0u, 0u};
    return ok ? *reinterpret_cast<const u32x4 *>(p) : z;
}

// Raw buffer descriptor over `bytes` bytes at p.  Buffer loads past the end return zero and buffer
// stores past the end are dropped by the hardware range check, so tile loads and stores need no
// branches (which keeps the compiler's outstanding-load counting exact in pipelined loops).
typedef __amdgpu_buffer_rsrc_t rsrc_t;
__device__ __forceinline__ rsrc_t make_rsrc(const void *p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, (int)bytes, 0x00020000);
}
// The same for a pointer that is wavefront-uniform but was computed in vector registers (64-bit address arithmetic):
// a descriptor left there makes every load through it a loop over the distinct values found in the lanes.
__device__ __forceinline__ rsrc_t make_rsrc_uniform(const void *p, uint32_t bytes) {
    const uint64_t v = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return make_rsrc(reinterpret_cast<const void *>(((uint64_t)hi << 32) | lo), __builtin_amdgcn_readfirstlane(bytes));
}
// NT: non-temporal load, for data that no other workgroup reads and that is not read again before the caches have
// turned over (long sequences): such loads do not displace other lines and stream about a third faster.  Stores
// are never non-temporal: the 8-byte pieces of a row have to meet in L2 before the line goes to memory.
template <bool NT = false>
__device__ __forceinline__ u32x4 buf_load16(rsrc_t r, uint32_t byte_off) {
    return __builtin_amdgcn_raw_buffer_load_b128(r, (int)byte_off, 0, NT ? 2 : 0);
}
__device__ __forceinline__ void buf_store8(rsrc_t r, uint32_t byte_off, u32x2 v) {
    __builtin_amdgcn_raw_buffer_store_b64(v, r, (int)byte_off, 0, 0);
}
constexpr uint32_t kOobOffset = 0x80000000u;  // beyond any descriptor this library builds

}  // namespace cott
