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

// Kernel families, as reported by cott_profile_read().
enum KernelId { K_GROUP_STATE = 0, K_STATE_PREFIX, K_SCAN, K_APPLY, K_BWD_DKDV, K_GENERIC, K_DECODE, K_COUNT };

// While profiling is enabled (cott_profile_enable), brackets the launches made in its lifetime
// with a pair of HIP events on the launch stream; otherwise does nothing.
class ProfScope {
  public:
    ProfScope(int kernel_id, hipStream_t stream);
    ~ProfScope();
    ProfScope(const ProfScope &) = delete;
    ProfScope &operator=(const ProfScope &) = delete;

  private:
    int id_;
    hipStream_t stream_;
    hipEvent_t start_;
    bool active_;
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
