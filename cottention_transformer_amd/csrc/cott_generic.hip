// Plain-FMA fallback launches (all dtypes) and the decode step.
#include "cott_generic.h"
#include "cott_launch.h"
#include "../../include/cottention.h"

namespace cott {
namespace {

constexpr size_t kLdsBudget = 150 * 1024;

struct GenericTiling {
    int CH, DJT;
    size_t bytes;
};

size_t generic_lds_bytes(int di, int CH, int DJT, size_t acc_size) {
    return ((size_t)2 * CH * (di + 1) + (size_t)CH * DJT + (size_t)CH * (CH + 1) + (size_t)di * DJT) * acc_size;
}

bool pick_tiling(int di, size_t acc_size, GenericTiling *out) {
    static const int cands[][2] = {{32, 32}, {32, 16}, {16, 16}, {8, 16}, {8, 8}, {4, 8}};
    for (const auto &c : cands) {
        const size_t b = generic_lds_bytes(di, c[0], c[1], acc_size);
        if (b <= kLdsBudget) {
            *out = GenericTiling{c[0], c[1], b};
            return true;
        }
    }
    return false;
}

size_t acc_size_of(int dtype) { return dtype == COTT_F64 ? sizeof(double) : sizeof(float); }

template <class ST, bool CAUSAL>
hipError_t run_generic(const OpDesc &a, int BH, int N, hipStream_t stream) {
    GenericTiling t;
    if (!pick_tiling(a.di, sizeof(typename ST::acc), &t)) return hipErrorInvalidValue;
    auto kern = generic_scan_kernel<ST, CAUSAL>;
    if (t.bytes > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)t.bytes);
        if (e != hipSuccess) return e;
    }
    const int nslices = (a.dj + t.DJT - 1) / t.DJT;
    typedef typename ST::elem E;
    ProfScope ps(K_GENERIC, stream);
    kern<<<dim3((unsigned)(BH * nslices)), dim3(256), t.bytes, stream>>>(
        static_cast<const E *>(a.A), static_cast<const E *>(a.B), static_cast<const E *>(a.C), static_cast<E *>(a.O),
        static_cast<const typename ST::acc *>(a.sin), static_cast<typename ST::acc *>(a.sout), N, a.di, a.dj, t.CH, t.DJT, nslices, a.reversed);
    return hipGetLastError();
}

template <class ST, class SF>
hipError_t run_decode(void *state, const void *q, const void *k, const void *v, void *o, int BH, int dk, int dv,
                      const DecodePrep &prep, hipStream_t stream) {
    typedef typename ST::elem E;
    ProfScope ps(K_DECODE, stream);
    const int nv = dv / 4;
    if ((nv == 8 || nv == 16 || nv == 32 || nv == 64) && dk <= 1024) {
        // one wavefront per head, four heads per workgroup
        const size_t lds_w = (size_t)4 * 2 * dk * sizeof(SF);
        if (lds_w > 48 * 1024) {  // (fp64 with dk = 1024: 64 KiB)
            hipError_t e0 = hipFuncSetAttribute(reinterpret_cast<const void *>(decode_wave_kernel<ST, SF, false, 3>),
                                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_w);
            if (e0 != hipSuccess) return e0;
            hipError_t e = prep.on ? hipFuncSetAttribute(reinterpret_cast<const void *>(decode_wave_kernel<ST, SF, true>),
                                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_w)
                                   : hipFuncSetAttribute(reinterpret_cast<const void *>(decode_wave_kernel<ST, SF, false>),
                                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_w);
            if (e != hipSuccess) return e;
        }
        // A state well beyond the 256 MB last-level cache is not found there by the next step: non-temporal loads
        // and stores then stream it 10 % faster (1 GiB: 437 -> 393 us per step); a state that fits is served from
        // that cache and keeps the plain accesses.
        if (!prep.on && (size_t)BH * dk * dv * sizeof(SF) >= ((size_t)384 << 20)) {
            decode_wave_kernel<ST, SF, false, 3><<<dim3((unsigned)((BH + 3) / 4)), dim3(256), lds_w, stream>>>(
                static_cast<SF *>(state), static_cast<const E *>(q), static_cast<const E *>(k), static_cast<const E *>(v),
                static_cast<E *>(o), BH, dk, dv, prep);
            return hipGetLastError();
        }
        if (prep.on)
            decode_wave_kernel<ST, SF, true><<<dim3((unsigned)((BH + 3) / 4)), dim3(256), lds_w, stream>>>(
                static_cast<SF *>(state), static_cast<const E *>(q), static_cast<const E *>(k), static_cast<const E *>(v),
                static_cast<E *>(o), BH, dk, dv, prep);
        else
            decode_wave_kernel<ST, SF, false><<<dim3((unsigned)((BH + 3) / 4)), dim3(256), lds_w, stream>>>(
                static_cast<SF *>(state), static_cast<const E *>(q), static_cast<const E *>(k), static_cast<const E *>(v),
                static_cast<E *>(o), BH, dk, dv, prep);
        return hipGetLastError();
    }
    if (prep.on) return hipErrorInvalidValue;  // the fused preparation exists in the one-wavefront-per-head kernel only
    const size_t lds = (size_t)2 * dk * sizeof(SF) + 256 * 4 * sizeof(SF);
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(decode_kernel<ST, SF>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
    }
    decode_kernel<ST, SF><<<dim3((unsigned)BH), dim3(256), lds, stream>>>(
        static_cast<SF *>(state), static_cast<const E *>(q), static_cast<const E *>(k), static_cast<const E *>(v),
        static_cast<E *>(o), dk, dv);
    return hipGetLastError();
}

}  // namespace

bool generic_fits(int dtype, int di) {
    GenericTiling t;
    return pick_tiling(di, acc_size_of(dtype), &t);
}

hipError_t launch_generic(int dtype, bool causal, const OpDesc &a, int BH, int N, hipStream_t stream) {
    switch (dtype) {
        case COTT_F32: return causal ? run_generic<StF32, true>(a, BH, N, stream) : run_generic<StF32, false>(a, BH, N, stream);
        case COTT_F64: return causal ? run_generic<StF64, true>(a, BH, N, stream) : run_generic<StF64, false>(a, BH, N, stream);
        case COTT_F16: return causal ? run_generic<StFp16, true>(a, BH, N, stream) : run_generic<StFp16, false>(a, BH, N, stream);
        case COTT_BF16: return causal ? run_generic<StBf16, true>(a, BH, N, stream) : run_generic<StBf16, false>(a, BH, N, stream);
    }
    return hipErrorInvalidValue;
}

namespace {
hipError_t decode_any(int dtype, void *state, const void *q, const void *k, const void *v, void *o, int BH, int dk, int dv,
                      const DecodePrep &prep, hipStream_t stream) {
    switch (dtype) {
        case COTT_F32: return run_decode<StF32, float>(state, q, k, v, o, BH, dk, dv, prep, stream);
        case COTT_F64: return run_decode<StF64, double>(state, q, k, v, o, BH, dk, dv, prep, stream);
        case COTT_F16: return run_decode<StFp16, float>(state, q, k, v, o, BH, dk, dv, prep, stream);
        case COTT_BF16: return run_decode<StBf16, float>(state, q, k, v, o, BH, dk, dv, prep, stream);
    }
    return hipErrorInvalidValue;
}
}  // namespace

hipError_t launch_decode(int dtype, void *state, const void *q, const void *k, const void *v, void *o, int BH,
                         int dk, int dv, hipStream_t stream) {
    DecodePrep none{};
    return decode_any(dtype, state, q, k, v, o, BH, dk, dv, none, stream);
}

hipError_t launch_decode_prep(int dtype, void *state, const void *q, const void *k, const void *v, void *o, int BH, int H,
                              int dk, int dv, const float *sig, float cnt, const float *rot, long long pos, int R,
                              float eps, hipStream_t stream) {
    DecodePrep p{};
    p.sig = sig;
    p.rot = rot;
    p.pos = pos;
    p.cnt = cnt;
    p.eps = eps;
    p.R = R;
    p.H = H;
    p.on = 1;
    return decode_any(dtype, state, q, k, v, o, BH, dk, dv, p, stream);
}

}  // namespace cott
