// fp16 instantiations of the MFMA chunked-scan kernels.
#include "cott_mfma_launch.inc"
namespace cott {
hipError_t launch_causal_mfma_fp16(const SetArgs &a) { return dispatch<Fp16, true>(a); }
hipError_t launch_noncausal_mfma_fp16(const SetArgs &a) { return dispatch<Fp16, false>(a); }
}  // namespace cott
