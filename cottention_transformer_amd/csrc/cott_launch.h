// Host-side launch interface between the C ABI (cott_api.hip) and the kernel translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>

namespace cott {

// One generic op  out = G(A, B, C)  over BH independent heads; C and O may be a column slice
// (dj columns out of rows of ldc elements, pointers already offset to the first column).
struct OpDesc {
    const void *A, *B, *C;  // A,B: (BH,N,di)  C: (BH,N,ldc)
    void *O;                // (BH,N,ldc)
    int di, dj, ldc, reversed;
    // Optional hand-over of the recurrence state (causal ops only): (BH,di,lds) row-major, fp32
    // (fp64 for fp64 tensors), pointers offset to the first column like C and O.
    const void *sin = nullptr;  // start from this state instead of zero
    void *sout = nullptr;       // receives the state after the last position
    int lds = 0;
    // Layout of A, B, C, O (16-bit causal MFMA kernels only): 0 = (BH,N,width), 1 = (B,N,H,width) with the heads
    // of a position next to each other, as the projections of a transformer block produce and consume them.
    unsigned char lay[4] = {0, 0, 0, 0};
    int H = 1;  // heads per batch element; needed when any layout flag is set
    // Complement form (16-bit causal MFMA kernels, sets with sequence groups only): the op is walked against its
    // own direction so that it reads the same tiles at the same time as the other ops of its set.
    int comp = 0;
    int c0 = 0;  // first column of the C / O slice within the full rows (column halves)
    // >= 0: index (within the set) of the op whose state, transposed, is this op's state (see ProblemT::seed_from)
    int seed_from = -1;
    // States handed from a forward to a backward pass (16-bit causal MFMA kernels only; see ProblemT::save / ext):
    // (BH, save_n, save_slot) fp32 in 16 x 16 tiles, save_njt tiles per tile row.
    void *save = nullptr;
    const void *ext = nullptr;
    int save_njt = 0, save_slot = 0, save_cpg = 0, save_n = 0;
};

// A set of ops launched together over the same (BH, N); MFMA path: all share padded head dims.
struct SetArgs {
    OpDesc op[6];
    int count;
    float *ws;            // count * BH * G * state_floats floats of group-state slots, or null when unused
    int BH, N;
    int nchunks, cpg, G;  // chunks of 64, chunks per group, groups per head
    int sub = 1;          // pieces per group in the group-state pass (ws holds G * sub slots per head and problem)
    int scan_prof_id;     // K_SCAN for a forward launch, K_SCAN_GRAD for the three-gradient launch
    // pair > 0: op[pair] and op[pair + 1] are X = G(A,B,C) and Y = G(A2,C,B) with the same direction and square
    // padded head dims; one workgroup serves both (scan_pair_kernel).  The launch then has count - 1 problems
    // per head and the workspace count - 1 state slots per group.  pair must be count - 2.
    int pair = 0;
    // non-temporal loads in the group-state pass / in the scan: for tensors far larger than the caches, when no
    // two problems of the set read the same operand
    bool stream_state = false, stream_scan = false;
    int cus = 256, xcds = 8;  // CUs and XCDs of the device (placement and occupancy choices)
    // Input preparation inside the causal forward (16-bit, one group per head): q, k, v of the ops are the raw
    // projections; see PrepSide in cott_mfma.h for the meaning of the fields.  prep_on = false: none.
    struct Prep {
        bool on = false;
        const unsigned char *keep = nullptr;
        const float *cnt = nullptr, *sig = nullptr, *rot = nullptr;
        const long long *pos = nullptr;  // (B,N) position ids, or null: consecutive positions from pos0
        long long pos0 = 0;
        int R = 0, table_rows = 0, H = 1, dv = 0;
        float eps = 1e-12f;
        void *qo = nullptr, *ko = nullptr, *vo = nullptr;
    } prep;
    hipStream_t stream;
};

// Kernel families, as reported by cott_profile_read().
enum KernelId { K_GROUP_STATE = 0, K_STATE_PREFIX, K_SCAN, K_APPLY, K_SCAN_GRAD, K_GENERIC, K_DECODE, K_PREP, K_STREAM_PROBE, K_COUNT };

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

// 16-bit storage; every op: 32 <= di,dj <= 128, multiples of 16, same padded dims across the set.
hipError_t launch_causal_mfma_bf16(const SetArgs &a);
hipError_t launch_causal_mfma_fp16(const SetArgs &a);
hipError_t launch_noncausal_mfma_bf16(const SetArgs &a);
hipError_t launch_noncausal_mfma_fp16(const SetArgs &a);
// fp32 storage on the fp32 MFMA; same limits, no column-half problems, workspace also for the non-causal form.
hipError_t launch_causal_mfma_f32(const SetArgs &a);
hipError_t launch_noncausal_mfma_f32(const SetArgs &a);

// Plain-FMA fallback for any dtype / head dim, one op (full tensors: ldc == dj).
// Returns hipErrorInvalidValue if no tiling fits LDS.
hipError_t launch_generic(int dtype, bool causal, const OpDesc &op, int BH, int N, hipStream_t stream);
bool generic_fits(int dtype, int di);

// Fused input preparation (backward = false) or its backward; see cott_prep.hip.
hipError_t launch_prep(bool backward, const void *const x[3], const void *const g[3], void *const y[3],
                       const unsigned char *keep, const float *cnt, const float *sig, float *dsig_rows, int B, int H, int N,
                       int dk, int dv, int x_dtype, int y_dtype, int g_dtype, float eps, int x_bnhd, const float *rot,
                       const long long *pos, int R, int table_rows, hipStream_t stream);

hipError_t launch_decode(int dtype, void *state, const void *q, const void *k, const void *v, void *o, int BH,
                         int dk, int dv, hipStream_t stream);
// The same step on the raw projections of the new token: rotation by table row `pos` (rot null = none), L2
// normalisation of q and k, v / max(cnt^sig[h], 1) (sig null = none) happen inside the kernel.  dv / 4 in
// {8,16,32,64} and dk <= 256, else hipErrorInvalidValue.
hipError_t launch_decode_prep(int dtype, void *state, const void *q, const void *k, const void *v, void *o, int BH, int H,
                              int dk, int dv, const float *sig, float cnt, const float *rot, long long pos, int R,
                              float eps, hipStream_t stream);

}  // namespace cott
