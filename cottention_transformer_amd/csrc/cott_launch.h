// Host-side launch interface between the C ABI (cott_api.hip) and the kernel translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>

namespace cott {

// One generic op  out = G(A, B, C)  over BH independent heads.
struct ScanArgs {
    const void *A, *B, *C;  // A,B: (BH,N,di)  C: (BH,N,dj)
    void *O;                // (BH,N,dj)
    float *ws;              // per-group state slots, BH*G*state_floats(di,dj) floats (MFMA path, G>1)
    int BH, N, di, dj;
    int reversed;
    int nchunks, cpg, G;    // MFMA path: chunks of 64, chunks per group, groups per head
    hipStream_t stream;
};

// Padded state size of the MFMA path (head dims padded to 32, 64 or 128).
inline int mfma_pad(int d) { return d <= 32 ? 32 : (d <= 64 ? 64 : 128); }
inline size_t mfma_state_floats(int di, int dj) { return (size_t)mfma_pad(di) * mfma_pad(dj); }

// dtype is COTT_F16 or COTT_BF16; 32 <= di,dj <= 128, multiples of 16.
hipError_t launch_causal_mfma_bf16(const ScanArgs &a);
hipError_t launch_causal_mfma_fp16(const ScanArgs &a);
hipError_t launch_noncausal_mfma_bf16(const ScanArgs &a);
hipError_t launch_noncausal_mfma_fp16(const ScanArgs &a);

// Plain-FMA fallback for any dtype / head dim.  Returns hipErrorInvalidValue if no tiling fits LDS.
hipError_t launch_generic(int dtype, bool causal, const ScanArgs &a);
bool generic_fits(int dtype, int di);

hipError_t launch_decode(int dtype, void *state, const void *q, const void *k, const void *v, void *o, int BH,
                         int dk, int dv, hipStream_t stream);

}  // namespace cott
