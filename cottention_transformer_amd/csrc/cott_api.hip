// C ABI of libcottention_hip.so: argument validation, kernel selection, launch.
// Declared in include/cottention.h, which cites the reference interface each entry replaces.
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <mutex>
#include <vector>

#include "../../include/cottention.h"
#include "cott_launch.h"

namespace cott {
namespace {
struct ProfRecord {
    int id;
    hipEvent_t start, stop;
};
std::mutex g_prof_mu;
std::vector<ProfRecord> g_prof_records;
bool g_prof_on = false;
}  // namespace

ProfScope::ProfScope(int kernel_id, hipStream_t stream) : id_(kernel_id), stream_(stream), start_(nullptr), active_(false) {
    if (!g_prof_on) return;
    if (hipEventCreate(&start_) != hipSuccess) return;
    active_ = hipEventRecord(start_, stream_) == hipSuccess;
    if (!active_) (void)hipEventDestroy(start_);
}

ProfScope::~ProfScope() {
    if (!active_) return;
    hipEvent_t stop;
    if (hipEventCreate(&stop) != hipSuccess || hipEventRecord(stop, stream_) != hipSuccess) {
        (void)hipEventDestroy(start_);
        return;
    }
    std::lock_guard<std::mutex> lock(g_prof_mu);
    g_prof_records.push_back(ProfRecord{id_, start_, stop});
}
}  // namespace cott

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

size_t elem_size(int dtype) {
    switch (dtype) {
        case COTT_F32: return 4;
        case COTT_F64: return 8;
        case COTT_F16:
        case COTT_BF16: return 2;
    }
    return 0;
}

// Workgroups the chunked scan aims for: a few per CU of a 256-CU part.  COTT_TARGET_WGS overrides.
int target_workgroups() {
    static const int v = [] {
        const char *s = getenv("COTT_TARGET_WGS");
        const int x = s ? atoi(s) : 0;
        return x > 0 ? x : 768;
    }();
    return v;
}

struct Plan {
    int nchunks, cpg, G;
};

Plan make_plan(long BH, int N) {
    Plan p;
    p.nchunks = (N + 63) / 64;
    long want = (target_workgroups() + BH - 1) / BH;
    if (want < 1) want = 1;
    if (want > p.nchunks) want = p.nchunks;
    p.cpg = (int)((p.nchunks + want - 1) / want);
    p.G = (p.nchunks + p.cpg - 1) / p.cpg;
    return p;
}

bool use_mfma(int dtype, int di, int dj) {
    return (dtype == COTT_F16 || dtype == COTT_BF16) && di % 16 == 0 && dj % 16 == 0 && di >= 32 && dj >= 32 &&
           di <= 128 && dj <= 128;
}

// Shape rules shared by every (B,H,N,D) entry point.  `di` is the contracted head dim of the
// generic op and must obey the reference's rule (combined_kernel_general.cu:372-374).
int check_common(const char *fn, int B, int H, int N, int di, int dj, int dtype) {
    if (elem_size(dtype) == 0) return fail(COTT_ERR_INVALID, "%s: unknown dtype %d", fn, dtype);
    if (B < 0 || H < 0 || N < 0) return fail(COTT_ERR_INVALID, "%s: negative size (B=%d H=%d N=%d)", fn, B, H, N);
    if (di % 16 != 0) return fail(COTT_ERR_INVALID, "%s: D_attn must be divisible by 16 (got %d)", fn, di);
    if (di < 32) return fail(COTT_ERR_INVALID, "%s: D_attn must be greater than or equal to 16*2 (got %d)", fn, di);
    if (dj < 1) return fail(COTT_ERR_INVALID, "%s: D_value must be positive (got %d)", fn, dj);
    if ((long)B * H > (1L << 22)) return fail(COTT_ERR_UNSUPPORTED, "%s: B*H = %ld exceeds 2^22", fn, (long)B * H);
    const long dmax = di > dj ? di : dj;
    if ((long)N * dmax >= (1L << 31)) return fail(COTT_ERR_UNSUPPORTED, "%s: N*D = %ld exceeds 2^31", fn, (long)N * dmax);
    return COTT_OK;
}

size_t ws_bytes_for(long BH, int N, int di, int dj, int dtype) {
    if (BH <= 0 || N <= 0 || !use_mfma(dtype, di, dj)) return 0;
    const Plan p = make_plan(BH, N);
    if (p.G <= 1) return 0;
    return (size_t)BH * p.G * cott::mfma_state_floats(di, dj) * sizeof(float);
}

// out = G(A, B, C) on the best available kernel family.
int run_op(const char *fn, bool causal, const void *A, const void *B, const void *C, void *O, long BH, int N, int di,
           int dj, int dtype, int reversed, void *ws, size_t ws_bytes, hipStream_t stream) {
    cott::ScanArgs a;
    a.A = A; a.B = B; a.C = C; a.O = O;
    a.BH = (int)BH; a.N = N; a.di = di; a.dj = dj;
    a.reversed = reversed ? 1 : 0;
    a.stream = stream;
    a.ws = nullptr;
    a.nchunks = a.cpg = a.G = 1;
    hipError_t e;
    if (use_mfma(dtype, di, dj)) {
        const Plan p = make_plan(BH, N);
        a.nchunks = p.nchunks; a.cpg = p.cpg; a.G = p.G;
        const size_t need = (size_t)BH * p.G * cott::mfma_state_floats(di, dj) * sizeof(float);
        if (p.G > 1 || !causal) {
            if (ws == nullptr || ws_bytes < need || !aligned16(ws))
                return fail(COTT_ERR_WORKSPACE, "%s: workspace of %zu bytes (16-byte aligned) required, got %zu", fn, need,
                            ws ? ws_bytes : (size_t)0);
            a.ws = static_cast<float *>(ws);
        }
        if (dtype == COTT_BF16)
            e = causal ? cott::launch_causal_mfma_bf16(a) : cott::launch_noncausal_mfma_bf16(a);
        else
            e = causal ? cott::launch_causal_mfma_fp16(a) : cott::launch_noncausal_mfma_fp16(a);
    } else {
        if (!cott::generic_fits(dtype, di))
            return fail(COTT_ERR_UNSUPPORTED, "%s: head dim %d too large for dtype %d on this build", fn, di, dtype);
        e = cott::launch_generic(dtype, causal, a);
    }
    if (e != hipSuccess) return fail(COTT_ERR_HIP, "%s: HIP launch failed: %s", fn, hipGetErrorString(e));
    return COTT_OK;
}

size_t noncausal_ws_bytes(long BH, int N, int di, int dj, int dtype) {
    if (BH <= 0 || N <= 0 || !use_mfma(dtype, di, dj)) return 0;
    const Plan p = make_plan(BH, N);
    return (size_t)BH * p.G * cott::mfma_state_floats(di, dj) * sizeof(float);
}

}  // namespace

extern "C" {

int cott_version(void) { return 100; }

int cott_profile_enable(int on) {
    std::lock_guard<std::mutex> lock(cott::g_prof_mu);
    cott::g_prof_on = on != 0;
    return COTT_OK;
}

int cott_profile_read(int kernel_id, double *total_ms, long *launches) {
    if (kernel_id < 0 || kernel_id >= cott::K_COUNT || !total_ms || !launches)
        return fail(COTT_ERR_INVALID, "cott_profile_read: bad argument");
    std::lock_guard<std::mutex> lock(cott::g_prof_mu);
    double sum = 0.0;
    long n = 0;
    std::vector<cott::ProfRecord> keep;
    for (const cott::ProfRecord &r : cott::g_prof_records) {
        if (r.id != kernel_id) {
            keep.push_back(r);
            continue;
        }
        float ms = 0.f;
        if (hipEventSynchronize(r.stop) == hipSuccess && hipEventElapsedTime(&ms, r.start, r.stop) == hipSuccess) {
            sum += ms;
            ++n;
        }
        (void)hipEventDestroy(r.start);
        (void)hipEventDestroy(r.stop);
    }
    cott::g_prof_records.swap(keep);
    *total_ms = sum;
    *launches = n;
    return COTT_OK;
}

const char *cott_kernel_name(int kernel_id) {
    static const char *names[cott::K_COUNT] = {"group_state_kernel", "state_prefix_kernel", "scan_kernel<causal>",
                                               "scan_kernel<apply>", "bwd_dkdv_kernel",     "generic_scan_kernel",
                                               "decode_kernel"};
    return (kernel_id >= 0 && kernel_id < cott::K_COUNT) ? names[kernel_id] : "";
}

const char *cott_last_error(void) { return g_err; }

size_t cott_causal_workspace_bytes(int B, int H, int N, int Dk, int Dv, int dtype) {
    return ws_bytes_for((long)B * H, N, Dk, Dv, dtype);
}

int cott_causal_fwd(const void *q, const void *k, const void *v, void *o, int B, int H, int N, int Dk, int Dv,
                    int dtype, int reversed, void *workspace, size_t workspace_bytes, void *stream) {
    const char *fn = "cott_causal_fwd";
    if (int rc = check_common(fn, B, H, N, Dk, Dv, dtype)) return rc;
    if ((long)B * H * N == 0) return COTT_OK;
    if (!q || !k || !v || !o) return fail(COTT_ERR_INVALID, "%s: null tensor pointer", fn);
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o))
        return fail(COTT_ERR_INVALID, "%s: tensor pointers must be 16-byte aligned", fn);
    return run_op(fn, true, q, k, v, o, (long)B * H, N, Dk, Dv, dtype, reversed, workspace, workspace_bytes,
                  static_cast<hipStream_t>(stream));
}

size_t cott_causal_bwd_workspace_bytes(int B, int H, int N, int Dk, int Dv, int dtype) {
    const size_t a = ws_bytes_for((long)B * H, N, Dv, Dk, dtype);  // dQ, dK: contract over Dv
    const size_t b = ws_bytes_for((long)B * H, N, Dk, Dv, dtype);  // dV: contract over Dk
    return a > b ? a : b;
}

int cott_causal_bwd(const void *q, const void *k, const void *v, const void *d_o, void *dq, void *dk, void *dv,
                    int B, int H, int N, int Dk, int Dv, int dtype, void *workspace, size_t workspace_bytes,
                    void *stream) {
    const char *fn = "cott_causal_bwd";
    if (int rc = check_common(fn, B, H, N, Dk, Dv, dtype)) return rc;
    if (int rc = check_common(fn, B, H, N, Dv, Dk, dtype)) return rc;  // roles swap in dQ and dK
    if ((long)B * H * N == 0) return COTT_OK;
    if (!q || !k || !v || !d_o || !dq || !dk || !dv) return fail(COTT_ERR_INVALID, "%s: null tensor pointer", fn);
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(d_o) || !aligned16(dq) || !aligned16(dk) ||
        !aligned16(dv))
        return fail(COTT_ERR_INVALID, "%s: tensor pointers must be 16-byte aligned", fn);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const long BH = (long)B * H;
    // Operand permutations of Cuda_Kernel/Custom_Kernel.py:106-108.
    if (int rc = run_op(fn, true, d_o, v, k, dq, BH, N, Dv, Dk, dtype, 0, workspace, workspace_bytes, s)) return rc;
    if (int rc = run_op(fn, true, v, d_o, q, dk, BH, N, Dv, Dk, dtype, 1, workspace, workspace_bytes, s)) return rc;
    return run_op(fn, true, k, q, d_o, dv, BH, N, Dk, Dv, dtype, 1, workspace, workspace_bytes, s);
}

size_t cott_noncausal_workspace_bytes(int B, int H, int N, int Dk, int Dv, int dtype) {
    const size_t a = noncausal_ws_bytes((long)B * H, N, Dv, Dk, dtype);
    const size_t b = noncausal_ws_bytes((long)B * H, N, Dk, Dv, dtype);
    return a > b ? a : b;
}

int cott_noncausal_fwd(const void *q, const void *k, const void *v, void *o, int B, int H, int N, int Dk, int Dv,
                       int dtype, void *workspace, size_t workspace_bytes, void *stream) {
    const char *fn = "cott_noncausal_fwd";
    if (int rc = check_common(fn, B, H, N, Dk, Dv, dtype)) return rc;
    if ((long)B * H * N == 0) return COTT_OK;
    if (!q || !k || !v || !o) return fail(COTT_ERR_INVALID, "%s: null tensor pointer", fn);
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o))
        return fail(COTT_ERR_INVALID, "%s: tensor pointers must be 16-byte aligned", fn);
    return run_op(fn, false, q, k, v, o, (long)B * H, N, Dk, Dv, dtype, 0, workspace, workspace_bytes,
                  static_cast<hipStream_t>(stream));
}

int cott_noncausal_bwd(const void *q, const void *k, const void *v, const void *d_o, void *dq, void *dk, void *dv,
                       int B, int H, int N, int Dk, int Dv, int dtype, void *workspace, size_t workspace_bytes,
                       void *stream) {
    const char *fn = "cott_noncausal_bwd";
    if (int rc = check_common(fn, B, H, N, Dk, Dv, dtype)) return rc;
    if (int rc = check_common(fn, B, H, N, Dv, Dk, dtype)) return rc;
    if ((long)B * H * N == 0) return COTT_OK;
    if (!q || !k || !v || !d_o || !dq || !dk || !dv) return fail(COTT_ERR_INVALID, "%s: null tensor pointer", fn);
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(d_o) || !aligned16(dq) || !aligned16(dk) ||
        !aligned16(dv))
        return fail(COTT_ERR_INVALID, "%s: tensor pointers must be 16-byte aligned", fn);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const long BH = (long)B * H;
    // dq = d_o (v^T k) ; dk = v (d_o^T q) ; dv = k (q^T d_o)
    if (int rc = run_op(fn, false, d_o, v, k, dq, BH, N, Dv, Dk, dtype, 0, workspace, workspace_bytes, s)) return rc;
    if (int rc = run_op(fn, false, v, d_o, q, dk, BH, N, Dv, Dk, dtype, 0, workspace, workspace_bytes, s)) return rc;
    return run_op(fn, false, k, q, d_o, dv, BH, N, Dk, Dv, dtype, 0, workspace, workspace_bytes, s);
}

int cott_decode_step(void *state, const void *q, const void *k, const void *v, void *o, int B, int H, int Dk, int Dv,
                     int dtype, void *stream) {
    const char *fn = "cott_decode_step";
    if (elem_size(dtype) == 0) return fail(COTT_ERR_INVALID, "%s: unknown dtype %d", fn, dtype);
    if (B < 0 || H < 0 || Dk < 1 || Dv < 1) return fail(COTT_ERR_INVALID, "%s: bad size", fn);
    if (Dv % 4 != 0) return fail(COTT_ERR_UNSUPPORTED, "%s: Dv must be a multiple of 4 (got %d)", fn, Dv);
    if (Dk > 8192) return fail(COTT_ERR_UNSUPPORTED, "%s: Dk = %d exceeds 8192", fn, Dk);
    const long BH = (long)B * H;
    if (BH == 0) return COTT_OK;
    if (BH >= (1L << 31)) return fail(COTT_ERR_UNSUPPORTED, "%s: B*H too large", fn);
    if (!state || !q || !k || !v || !o) return fail(COTT_ERR_INVALID, "%s: null pointer", fn);
    if (!aligned16(state) || (dtype == COTT_F64 && (reinterpret_cast<uintptr_t>(state) & 31u)))
        return fail(COTT_ERR_INVALID, "%s: state must be 16-byte (fp64: 32-byte) aligned", fn);
    hipError_t e = cott::launch_decode(dtype, state, q, k, v, o, (int)BH, Dk, Dv, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return fail(COTT_ERR_HIP, "%s: HIP launch failed: %s", fn, hipGetErrorString(e));
    return COTT_OK;
}

}  // extern "C"
