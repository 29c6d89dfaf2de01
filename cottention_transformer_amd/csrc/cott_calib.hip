// A streaming kernel with the launch shape of the scan kernels and none of their arithmetic: what this GPU's memory
// gives a launch of W workgroups that each walk their own contiguous share of R tensors in blocks (two blocks of every
// tensor in flight, like the scan kernels' loader wavefronts) and write their share of Wr tensors.  The benchmark times
// it beside the scan kernels, through the same event brackets, to tell the memory system's part of a kernel's duration
// from the kernel's own.  No counterpart in the reference.
#include "cott_common.h"
#include "cott_launch.h"

#include "../../include/cottention.h"

namespace cott {
namespace {

typedef uint32_t u32x4v __attribute__((ext_vector_type(4)));

template <int NR, int NW>
__global__ void __launch_bounds__(256) stream_probe_kernel(const u32x4v *__restrict__ in, u32x4v *__restrict__ out,
                                                           long tensor16, int steps, int block16) {
    constexpr int U = 2;
    const long base = (long)blockIdx.x * steps * block16;
    const int per = block16 / 256;  // 16-byte pieces per thread and block: 1..4
    u32x4v buf[U][NR][4];
    u32x4v acc = {0u, 0u, 0u, 0u};
    auto load = [&](int slot, int s) {
#pragma unroll
        for (int t = 0; t < NR; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (i < per)
                    buf[slot][t][i] = __builtin_nontemporal_load(in + t * tensor16 + base + (long)s * block16 + i * 256 + threadIdx.x);
    };
#pragma unroll
    for (int u = 0; u < U; ++u)
        if (u < steps) load(u, u);
    for (int s0 = 0; s0 < steps; s0 += U) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int s = s0 + u;
            if (s >= steps) break;
#pragma unroll
            for (int t = 0; t < NR; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (i < per) acc += buf[u][t][i];
#pragma unroll
            for (int t = 0; t < NW; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (i < per) out[t * tensor16 + base + (long)s * block16 + i * 256 + threadIdx.x] = acc;
            if (s + U < steps) load(u, s + U);
        }
    }
}

}  // namespace
}  // namespace cott

extern "C" int cott_stream_probe(const void *in, void *out, size_t tensor_bytes, int n_read, int n_write, int workgroups,
                                 int block_bytes, void *stream) {
    using namespace cott;
    if (!in || !out || workgroups < 1 || (block_bytes != 4096 && block_bytes != 8192 && block_bytes != 16384) ||
        tensor_bytes == 0 || tensor_bytes % ((size_t)workgroups * block_bytes) != 0 ||
        (reinterpret_cast<uintptr_t>(in) & 15u) || (reinterpret_cast<uintptr_t>(out) & 15u))
        return COTT_ERR_INVALID;
    const int steps = (int)(tensor_bytes / ((size_t)workgroups * block_bytes));
    const long tensor16 = (long)(tensor_bytes / 16);
    const int block16 = block_bytes / 16;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const u32x4v *src = static_cast<const u32x4v *>(in);
    u32x4v *dst = static_cast<u32x4v *>(out);
    ProfScope prof(K_STREAM_PROBE, st);
    if (n_read == 3 && n_write == 1)
        stream_probe_kernel<3, 1><<<dim3(workgroups), dim3(256), 0, st>>>(src, dst, tensor16, steps, block16);
    else if (n_read == 4 && n_write == 3)
        stream_probe_kernel<4, 3><<<dim3(workgroups), dim3(256), 0, st>>>(src, dst, tensor16, steps, block16);
    else
        return COTT_ERR_INVALID;
    return hipGetLastError() == hipSuccess ? COTT_OK : COTT_ERR_HIP;
}
