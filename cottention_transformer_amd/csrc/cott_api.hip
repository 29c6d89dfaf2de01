// C ABI of libcottention_hip.so: argument validation, kernel selection, launch.
// Declared in include/cottention.h, which cites the reference interface each entry replaces.
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <atomic>
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

// Scratch memory of cott_causal_fwd_noalloc: the group-state slots that the other entry points take from the
// caller's workspace.  Every device the library runs on holds its own copy of this array until the process ends.
// In host code the name is only a handle for hipGetSymbolAddress; kernels receive the address it returns.
#define COTT_SCRATCH_BYTES (48u << 20)
static __device__ __align__(256) unsigned char scratch[COTT_SCRATCH_BYTES];

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

// Tuning switches exist only in builds made with -DCOTT_EXPERIMENTS; the shipped library reads no environment.
int exp_int(const char *name, int dflt) {
#ifdef COTT_EXPERIMENTS
    const char *s = getenv(name);
    if (s && *s) return atoi(s);
#else
    (void)name;
#endif
    return dflt;
}

// Workgroups a launch aims for: one per CU (a second workgroup on a CU adds only ~20 %
// throughput to these LDS-heavy kernels, so grids just above the CU count run almost twice as long).
// CUs of the current device, asked once per process (256 on an unpartitioned MI355X; the fallback when the query
// fails).  A partitioned device reports fewer and gets correspondingly smaller launch plans.
std::atomic<int> g_cus_given{0}, g_xcds_given{0};  // cott_plan_geometry: > 0 replaces the device's answer

int device_cus() {
    if (const int given = g_cus_given.load(std::memory_order_relaxed)) return given;
    static const int v = [] {
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) != hipSuccess) return 256;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) return 256;
        return cus;
    }();
    return v;
}
int device_xcds() {
    if (const int given = g_xcds_given.load(std::memory_order_relaxed)) return given;
    static const int v = [] {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess) return 8;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeNumberOfXccs, dev) != hipSuccess || n <= 0) return 8;
        return n;
    }();
    return v;
}
int target_workgroups() {
    static const int given = exp_int("COTT_TARGET_WGS", 0);
    return given > 0 ? given : device_cus();
}
// -1 auto, 0 never, 1 always split the output columns of each op in two.
int split_policy() {
    static const int v = exp_int("COTT_SPLIT", -1);
    return v;
}

bool use_mfma(int dtype, int di, int dj, int N) {
    const bool dims = di % 16 == 0 && dj % 16 == 0 && di >= 32 && dj >= 32 && di <= 128 && dj <= 128;
    if (dtype == COTT_F16 || dtype == COTT_BF16) return dims;
    // fp32: byte offsets within a head must stay below 2^32
    if (dtype == COTT_F32) return dims && (long)N * (di > dj ? di : dj) <= (1L << 29);
    return false;
}

// One full-tensor generic op out = G(A,B,C).
struct Op {
    const void *A, *B, *C;
    void *O;
    int di, dj, reversed;
    const void *sin = nullptr;  // (BH,di,dj) state to start from / to receive the final state (causal only)
    void *sout = nullptr;
    unsigned char lay[4] = {0, 0, 0, 0};  // A, B, C, O given as (B,N,H,width) instead of (BH,N,width)
    int H = 1;
    // states handed from a forward to a backward pass (cott_causal_fwd_save / cott_causal_bwd_saved)
    void *save = nullptr;       // (BH, save_n, pad(di) * pad(dj)) fp32 in 16 x 16 tiles: written by a forward op
    const void *ext = nullptr;  // the same array, read by the backward op that sums over the past (dQ)
    int save_cpg = 0, save_n = 0;
};

// How a set of `nops` ops with the same padded head dims is laid on the chip.
struct SetPlan {
    int halves;           // 1, or 2 = every op split into two column halves (two problems)
    int nchunks, cpg, G;  // sequence cut: chunks of 64, chunks per group, groups per head
    int sub;              // pieces per group in the group-state pass (one workgroup and one slot each)
    size_t ws_bytes;      // group-state slots
};

bool pair_enabled() {
    static const bool v = exp_int("COTT_PAIR", 1) != 0;
    return v;
}

// The last two of three causal ops form a pair when they are X = G(A,B,C), Y = G(A2,C,B), same direction, 16-bit
// storage, and all three ops share square padded head dims of at most 64 (dK and dV of a backward pass).
bool pair_eligible(const Op *ops, int n, int dtype, bool causal) {
    if (!pair_enabled() || !causal || n != 3 || !(dtype == COTT_F16 || dtype == COTT_BF16)) return false;
    const Op &x = ops[1], &y = ops[2];
    // (both sum over the future: the pair workgroups leave out the score tiles on the other side of the diagonal)
    if (!(x.B == y.C && x.C == y.B && x.reversed == 1 && y.reversed == 1 && x.di == y.dj && x.dj == y.di)) return false;
    const int pd = cott::mfma_pad(ops[0].di);
    if (pd > 64) return false;
    for (int i = 0; i < 3; ++i)
        if (cott::mfma_pad(ops[i].di) != pd || cott::mfma_pad(ops[i].dj) != pd || ops[i].sin || ops[i].sout) return false;
    return true;
}

SetPlan plan_set(long BH, int N, int nops, int di, int dj, bool causal, int dtype, bool no_split = false,
                 bool has_ext = false) {
    SetPlan p;
    // the kernels on the fp32 matrix pipe are bound by it, with four wavefronts per workgroup: two workgroups per CU
    // overlap well.  Causal fp32 ops of padded head dims 64 x 64 run from split operands on the bf16 matrix cores,
    // one workgroup of eight wavefronts per CU like the 16-bit kernels.
    const bool f32_split = dtype == COTT_F32 && causal && cott::mfma_pad(di) == 64 && cott::mfma_pad(dj) == 64 &&
                           exp_int("COTT_F32_SPLIT", 1) != 0;
    const long tgt = target_workgroups() * ((dtype == COTT_F32 && !f32_split) ? 2 : 1);
    const bool can_split = !no_split && dtype != COTT_F32 && dj >= 64 && dj % 32 == 0 && 2 * nops <= 6;
    const int pol = split_policy();
    const long xcds = device_xcds();
    p.nchunks = (N + 63) / 64;
    // Choose (column halves, sequence groups) to fill the target without exceeding it: halves cost
    // repeated score tiles but no memory traffic, groups cost one extra read of two operands.
    long best_total = -1;
    int best_h = 1, best_g = 1;
    long g_of[3] = {0, 0, 0};
    int cpg_of[3] = {0, 0, 0};
    for (int h = 1; h <= 2; ++h) {
        if (h == 2 && (!can_split || pol == 0)) continue;
        if (h == 1 && can_split && pol == 1) continue;
        const long base = BH * nops * h;
        // (head, group) units are dealt round-robin over the XCDs and the workgroups of a unit stay on one XCD:
        // the fullest XCD gets ceil(BH * g / xcds) units and must hold them at once
        const long units_per_xcd = tgt / xcds / (nops * h);
        long g = units_per_xcd * xcds / BH;
        if (g < 1) g = 1;
        if (g > p.nchunks) g = p.nchunks;
        const int cpg = (int)((p.nchunks + g - 1) / g);
        g = (p.nchunks + cpg - 1) / cpg;
        g_of[h] = g;
        cpg_of[h] = cpg;
        const long total = base * g;
        // prefer the fuller grid; on a tie prefer fewer groups (less re-reading)
        const bool better = best_total < 0 || (total <= tgt && best_total > tgt) ||
                            ((total <= tgt) == (best_total <= tgt) &&
                             ((total <= tgt) ? (total > best_total || (total == best_total && g < best_g))
                                             : (total < best_total)));
        if (better) {
            best_total = total;
            best_h = h;
            best_g = (int)g;
        }
    }
    // When the sequence has to be cut into groups with or without halves, halves save no traffic (every group but
    // the last is read twice either way) and only repeat the score tiles: whole problems in twice as many groups
    // are faster as long as a group keeps 16 or more chunks (measured on B*H = 16..96, N = 2k..64k, D = 64..128:
    // 3 to 25 % faster forward; with 4 or 8 chunks per group the halves win by 15 to 20 %).
    // A forward pass of 64 x 64 tiles whose whole problems would only fill the same number of workgroups as the
    // halves (twice the groups) needs groups of 32 chunks (B8 H8 D64 N4096..6144, groups of 16..24: halves in two
    // groups 35 / 41 / 46 us against 39 / 44 / 50 us; N8192, groups of 32: 69 against 66 us).
    const bool small_tiles = cott::mfma_pad(di) * cott::mfma_pad(dj) <= 64 * 64;
    const int whole_from = (nops == 1 && g_of[1] == 2 * g_of[2] && small_tiles) ? 32 : 16;
    if (best_h == 2 && g_of[1] > 1 && g_of[2] > 1 && cpg_of[1] >= whole_from) {
        best_h = 1;
        best_g = (int)g_of[1];
    }
    // Three gradient problems of few heads that fit the chip either as column halves of ONE group or as whole
    // problems in groups.  Whole problems let dQ walk with dK and dV (complement form, shared tiles) at the price of
    // the group-state and prefix passes, which pays from some group length on.  Measured on 128-wide heads, with /
    // without the states the forward pass leaves for dQ: when the groups give more workgroups than the halves
    // (B3 H8: 216 against 144) from 16 / 32 chunks per group (N4096, groups of 22: 71 us with states, 84 without,
    // halves 80; N8192: 124 / 146 / 171 us); when both give the same number (B4 H8, B5 H8) from 64 / 128 chunks
    // (B4 H8 N8192, groups of 64: 167 / 184 us, halves 196; N4096: 89 / 98 us, halves 80).
    if (causal && nops == 3 && can_split && pol < 0 && g_of[2] == 1 && g_of[1] > 1 && BH * nops * 2 <= tgt &&
        BH * nops * g_of[1] <= tgt) {
        const bool fuller = g_of[1] > 2;
        const int from = fuller ? (has_ext ? 16 : 32) : (has_ext ? 64 : 128);
        const bool groups = cpg_of[1] >= from;
        best_h = groups ? 1 : 2;
        best_g = groups ? (int)g_of[1] : 1;
    }
    // A forward pass (one problem per head) of 65..128 heads, likewise: column halves of one group (twice the score
    // products, q and k read twice through L2) against whole problems in groups (one more pass over part of k and
    // v, two more launches).  Where the groups give more workgroups (65..85 heads: three groups) they win from 16
    // chunks per group for 128 x 128 tiles and from 32 for smaller ones (B9 H8 D128 N4096, groups of 22: 88 against
    // 102 us, N2048: 56 against 41 us; D64 N8192, groups of 43: 73 against 97 us, N4096: 45 against 38 us); where both
    // give the same number they win from 64 chunks as long as the chip is not nearly full (B11 H8 D128 N16384: 361
    // against 420 us, B13 H8: 404 against 437 us, B15 H8: 473 against 472 us).
    if (causal && nops == 1 && can_split && pol < 0 && g_of[2] == 1 && g_of[1] > 1 && BH * 2 <= tgt &&
        BH * g_of[1] <= tgt) {
        const bool wide = cott::mfma_pad(di) * cott::mfma_pad(dj) >= 128 * 128;
        const bool groups = g_of[1] > 2 ? cpg_of[1] >= (wide ? 16 : 32) : (cpg_of[1] >= 64 && 2 * BH * 20 <= tgt * 17);
        best_h = groups ? 1 : 2;
        best_g = groups ? (int)g_of[1] : 1;
    }
    // Non-causal forward of small heads, more heads than CUs but at most half of the workgroups that can be resident
    // (three per CU): the one-workgroup-per-head kernel runs its two passes over a short sequence, and twice as many
    // half-width workgroups fill the chip (B32 H12 N512 D64: 21.3 -> 20.7 us, 31.0 -> 28.1 us with cold caches; N2048:
    // 113 -> 108 us).  Outside that range whole problems are faster (192 heads: 12.5 against 14.3 us; 768 heads: 34.3
    // against 38.4 us; 480 heads at N1024: 41.9 against 45.6 us; 128-wide heads: 53.5 against 56.6 us).
    if (!causal && nops == 1 && can_split && pol != 0 && BH > tgt && 2 * BH <= 3 * tgt && di <= 64 && dj <= 64 &&
        g_of[1] == 1 && g_of[2] == 1)
        best_h = 2;
    p.halves = best_h;
    p.cpg = (p.nchunks + best_g - 1) / best_g;
    p.G = (p.nchunks + p.cpg - 1) / p.cpg;
    const size_t state = cott::mfma_state_floats(di, dj / p.halves) * sizeof(float);
    // the fp32 kernels stage the non-causal state through the workspace even for one group
    const bool slots = p.G > 1 || (!causal && dtype == COTT_F32);
    p.sub = 1;
    p.ws_bytes = slots ? (size_t)nops * p.halves * BH * p.G * state : 0;
    return p;
}

// Whether the backward set runs as dQ + (dK, dV) pair.  The pair workgroup is heavier than a single problem, so
// when the three separate problems already fit the chip in one round without sequence groups (more than half and at
// most all of the CUs), they finish sooner (33 us against 41 us at B*H = 64, N = 2048, D = 64) ...
bool use_pair(const Op *ops, int n, long BH, int N, int dtype, bool causal) {
    if (!pair_eligible(ops, n, dtype, causal)) return false;
    const SetPlan u = plan_set(BH, N, 3, ops[0].di, ops[0].dj, causal, dtype);
    if (!(u.G == 1 && u.halves == 1 && 3 * BH <= target_workgroups())) return true;
    // ... unless the forward pass has left the states dQ starts from and the sequence is long: the pair's workgroups
    // (in two groups) then share every tile with dQ's, which the three separate problems cannot (B6 H8 D64 N8192:
    // 96 against 113 us, N16384: 179 against 225 us; N4096: 51 against 51 us, N2048: 34 against 28 us).
    return ops[0].ext != nullptr && (N + 63) / 64 >= 128;
}

int pad_key(const Op &o) { return cott::mfma_pad(o.di) * 1000 + cott::mfma_pad(o.dj); }

// How one set of ops with equal padded head dims (members[0..cnt) of ops[0..n)) is run.
struct SetLayout {
    SetPlan p;
    bool pair;        // dQ + (dK, dV) pair workgroups
    bool complement;  // the ops that sum over the past run in complement form (see ProblemT)
    int twin_of[8];   // >= 0: member whose state, transposed, is this member's state
};

SetLayout layout_set(const Op *ops, int n, const int *members, int cnt, long BH, int N, int dtype, bool causal) {
    SetLayout L;
    const Op &first = ops[members[0]];
    const bool half = dtype == COTT_BF16 || dtype == COTT_F16;
    L.pair = use_pair(ops, n, BH, N, dtype, causal);  // then all three ops are in this set
    bool has_ext = false;
    for (int c = 0; c < cnt; ++c) has_ext = has_ext || ops[members[c]].ext != nullptr;
    L.p = L.pair ? plan_set(BH, N, 2, first.di, first.dj, causal, dtype, true)
                 : plan_set(BH, N, cnt, first.di, first.dj, causal, dtype, false, has_ext);
    const SetPlan &p = L.p;
    // Gradient sets cut into sequence groups: the op that sums over the past (dQ) is put in complement form and
    // walks the sequence from the end like the two that sum over the future, so the three workgroups of a head
    // and group read the same tiles at the same time and the second and third reader find them in L2.
    // (Beside a (dK, dV) pair dQ does the same whenever the forward pass has left its states, also when a head is one
    // group: see run_ops.  Three separate problems of one group each gain nothing from it: 142 -> 157 us at B8 H16
    // N2048 D128, where the 384 workgroups do not run at the same time anyway.)
    bool any_rev = false;
    for (int c = 0; c < cnt; ++c) any_rev = any_rev || ops[members[c]].reversed;
    L.complement = causal && !L.pair && p.G > 1 && cnt > 1 && any_rev && p.halves == 1 && half;
    // ... and when two of them are X = G(.,B,C), Y = G(.,C,B) with square padded head dims (dK and dV), their
    // states are transposes of each other: the group-state pass computes X's only.
    for (int c = 0; c < 8; ++c) L.twin_of[c] = -1;
    if (causal && !L.pair && p.G > 1 && p.halves == 1 && half && cott::mfma_pad(first.di) == cott::mfma_pad(first.dj))
        for (int c = 1; c < cnt; ++c)
            for (int e = 0; e < c && L.twin_of[c] < 0; ++e) {
                const Op &x = ops[members[e]], &y = ops[members[c]];
                if (L.twin_of[e] < 0 && x.B == y.C && x.C == y.B && x.reversed == y.reversed && x.di == y.dj &&
                    x.dj == y.di && !x.sin && !x.sout && !y.sin && !y.sout && !x.lay[1] == !y.lay[2] &&
                    !x.lay[2] == !y.lay[1])
                    L.twin_of[c] = e;
            }
    // The group-state pass only streams two operands into MFMAs and two of its workgroups fit a CU: when its grid
    // does not fill the chip, every group is cut into up to four pieces (one workgroup and one slot each).  With k
    // workgroups on the fullest CU the pass takes about k * (1.15 if k == 2) / pieces of its one-piece time
    // (measured at B1 H16 N65536 D128: 144 workgroups 194 us, 288: 193, 432: 158, 576: 187; 240 -> 480: 84 -> 90).
    // (fp32 ops on split operands have a group-state pass of the same kind, one 80 KiB workgroup per CU)
    const bool split32 = dtype == COTT_F32 && causal && cott::mfma_pad(first.di) == 64 && cott::mfma_pad(first.dj) == 64 &&
                         exp_int("COTT_F32_SPLIT", 1) != 0;
    if (p.G > 1 && (half || split32)) {
        long wgs = 0;
        if (L.pair)
            wgs = (ops[members[0]].ext != nullptr ? 1L : 2L) * (p.G - 1);
        else
            for (int c = 0; c < cnt; ++c) {
                if (L.twin_of[c] >= 0 || ops[members[c]].ext != nullptr) continue;
                const bool comp = L.complement && !ops[members[c]].reversed && !ops[members[c]].sin && !ops[members[c]].sout;
                wgs += (long)p.halves * (causal && !comp ? p.G - 1 : p.G);
            }
        wgs *= BH;
        static const int force = exp_int("COTT_SUB", 0);
        const long cus = device_cus();
        int sub = 1;
        double best = 1e30;
        for (int s = 1; s <= 4; ++s) {
            if (s > 1 && (p.cpg + s - 1) / s < 4) break;
            const long k = (wgs * s + cus - 1) / cus;
            if (k > (split32 ? 1 : 2)) break;
            const double cost = (double)k * (k == 2 ? 1.15 : 1.0) / s;
            if (cost < best - 1e-9) {
                best = cost;
                sub = s;
            }
        }
        if (force > 0) sub = force;
        if (sub > 1) {
            L.p.sub = sub;
            L.p.ws_bytes *= (size_t)sub;
        }
    }
    return L;
}

// The launches of a call: ops with equal padded head dims form a set (sets[s][0 .. counts[s])).  One case is cut in
// two: the three gradients of heads that are one group each, whose 3 * BH workgroups (one per CU: the widest tiles)
// would run as one full round of the chip and a partly empty one.  dK and dV, which share their tiles, then form one
// launch of 2 * BH workgroups and dQ a second one, in column halves where that fills the chip (gradients at B8 H16
// N2048 D128: 140 -> 131 us, B6: 132 -> 114 us, B7 N4096: 282 -> 247 us).
int form_sets(const Op *ops, int n, long BH, int N, int dtype, bool causal, int sets[8][8], int *counts) {
    int nsets = 0;
    bool done[8] = {false};
    for (int i = 0; i < n; ++i) {
        if (done[i]) continue;
        int *members = sets[nsets], cnt = 0;
        for (int j = i; j < n; ++j)
            if (!done[j] && pad_key(ops[j]) == pad_key(ops[i])) { done[j] = true; members[cnt++] = j; }
        counts[nsets++] = cnt;
        static const int split_sets = exp_int("COTT_SPLIT_SETS", 1);
        const bool half = dtype == COTT_BF16 || dtype == COTT_F16;
        if (!(split_sets && causal && half && n == 3 && cnt == 3) || use_pair(ops, n, BH, N, dtype, causal)) continue;
        bool plain = true;
        for (int c = 0; c < 3; ++c) plain = plain && !ops[c].sin && !ops[c].sout && !ops[c].ext && !ops[c].save;
        const SetPlan u = plan_set(BH, N, 3, ops[members[0]].di, ops[members[0]].dj, causal, dtype);
        const long tgt = target_workgroups();
        if (!plain || u.G != 1 || u.halves != 1 || 3 * BH <= tgt || 2 * BH > tgt) continue;
        int rev[8], fwd[8], nr = 0, nf = 0;
        for (int c = 0; c < 3; ++c) (ops[members[c]].reversed ? rev[nr++] : fwd[nf++]) = members[c];
        if (nr != 2 || nf != 1) continue;
        members[0] = rev[0];
        members[1] = rev[1];
        counts[nsets - 1] = 2;
        sets[nsets][0] = fwd[0];
        counts[nsets++] = 1;
    }
    return nsets;
}

// Workspace needed by run_ops for the same arguments.
size_t ops_workspace(const Op *ops, int n, long BH, int N, int dtype, bool causal) {
    if (BH <= 0 || N <= 0) return 0;
    for (int i = 0; i < n; ++i)
        if (!use_mfma(dtype, ops[i].di, ops[i].dj, N)) return 0;
    size_t total = 0;
    int sets[8][8], counts[8];
    const int nsets = form_sets(ops, n, BH, N, dtype, causal, sets, counts);
    for (int s = 0; s < nsets; ++s) total += layout_set(ops, n, sets[s], counts[s], BH, N, dtype, causal).p.ws_bytes;
    return total;
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
    // one head is addressed through a 32-bit byte offset: its bytes must stay below 2^32 (fp32: N*D < 2^30)
    if ((long)N * dmax > (1L << 30) - (dtype == COTT_F32 ? 1 : 0))
        return fail(COTT_ERR_UNSUPPORTED, "%s: N*D = %ld exceeds 2^30", fn, (long)N * dmax);
    return COTT_OK;
}

// Runs n generic ops (n <= 3) over the same (BH, N) on the best available kernel family.
int run_ops(const char *fn, bool causal, const Op *ops, int n, long BH, int N, int dtype, void *ws, size_t ws_bytes,
            hipStream_t stream, const cott::SetArgs::Prep *prep = nullptr) {
    bool mfma = true;
    for (int i = 0; i < n; ++i) mfma = mfma && use_mfma(dtype, ops[i].di, ops[i].dj, N);
    const size_t esz = elem_size(dtype);
    bool interleaved = false;
    for (int i = 0; i < n; ++i) interleaved = interleaved || ops[i].lay[0] || ops[i].lay[1] || ops[i].lay[2] || ops[i].lay[3];
    if (interleaved && !(mfma && (dtype == COTT_BF16 || dtype == COTT_F16)))
        return fail(COTT_ERR_UNSUPPORTED, "%s: (B,N,H,D) operands need bf16 / fp16 and head dims 32..128 in steps of 16", fn);
    if (!mfma) {
        for (int i = 0; i < n; ++i) {
            if (!cott::generic_fits(dtype, ops[i].di))
                return fail(COTT_ERR_UNSUPPORTED, "%s: head dim %d too large for dtype %d on this build", fn, ops[i].di,
                            dtype);
            cott::OpDesc d{ops[i].A, ops[i].B, ops[i].C, ops[i].O, ops[i].di, ops[i].dj, ops[i].dj, ops[i].reversed,
                           ops[i].sin,  ops[i].sout, ops[i].dj};
            hipError_t e = cott::launch_generic(dtype, causal, d, (int)BH, N, stream);
            if (e != hipSuccess) return fail(COTT_ERR_HIP, "%s: HIP launch failed: %s", fn, hipGetErrorString(e));
        }
        return COTT_OK;
    }
    const size_t need = ops_workspace(ops, n, BH, N, dtype, causal);
    if (need > 0 && (ws == nullptr || ws_bytes < need || !aligned16(ws)))
        return fail(COTT_ERR_WORKSPACE, "%s: workspace of %zu bytes (16-byte aligned) required, got %zu", fn, need,
                    ws ? ws_bytes : (size_t)0);
    char *ws_cursor = static_cast<char *>(ws);
    int sets[8][8], counts[8];
    const int nsets = form_sets(ops, n, BH, N, dtype, causal, sets, counts);
    for (int si = 0; si < nsets; ++si) {
        cott::SetArgs a;
        a.count = 0;
        const int *members = sets[si], cnt = counts[si];
        const int i = members[0];
        const SetLayout L = layout_set(ops, n, members, cnt, BH, N, dtype, causal);
        const SetPlan &p = L.p;
        if (prep != nullptr) a.prep = *prep;
        const bool pair = L.pair, complement = L.complement;
        const int *twin_of = L.twin_of;
        a.pair = pair ? 1 : 0;
        // Non-temporal loads: tensors several times the last-level cache, and no operand read by two problems
        static const long stream_min_bytes = (long)exp_int("COTT_STREAM_MIN_MB", 128) << 20;
        const bool big = (long)BH * N * (ops[i].di > ops[i].dj ? ops[i].di : ops[i].dj) * (long)esz >= stream_min_bytes;
        a.stream_scan = causal && big && cnt == 1 && p.halves == 1 && (dtype == COTT_BF16 || dtype == COTT_F16);
        bool distinct = causal && p.halves == 1 && (dtype == COTT_BF16 || dtype == COTT_F16);
        for (int c = 0; c < cnt && distinct; ++c)
            for (int e = 0; e < c; ++e) {
                if (twin_of[c] >= 0 || twin_of[e] >= 0) continue;  // skipped by the group-state pass
                const Op &x = ops[members[e]], &y = ops[members[c]];
                if (x.B == y.B || x.B == y.C || x.C == y.B || x.C == y.C) distinct = false;
            }
        a.stream_state = distinct && big;
        for (int c = 0; c < cnt; ++c) {
            const Op &o = ops[members[c]];
            const int djh = o.dj / p.halves;
            for (int h = 0; h < p.halves; ++h) {
                cott::OpDesc &d = a.op[a.count++];
                d.A = o.A;
                d.B = o.B;
                d.C = static_cast<const char *>(o.C) + (size_t)h * djh * esz;
                d.O = static_cast<char *>(o.O) + (size_t)h * djh * esz;
                d.di = o.di;
                d.dj = djh;
                d.ldc = o.dj;
                d.reversed = o.reversed;
                // (... and so does dQ beside a (dK, dV) pair when the forward pass has left its states)
                d.comp = ((complement || (pair && o.ext != nullptr)) && !o.reversed && !o.sin && !o.sout) ? 1 : 0;
                d.seed_from = twin_of[c];  // (halves == 1 here: set index == member index)
                d.c0 = h * djh;
                const size_t ssz = dtype == COTT_F64 ? 8 : 4;
                d.sin = o.sin ? static_cast<const char *>(o.sin) + (size_t)h * djh * ssz : nullptr;
                d.sout = o.sout ? static_cast<char *>(o.sout) + (size_t)h * djh * ssz : nullptr;
                d.lds = o.dj;
                for (int x = 0; x < 4; ++x) d.lay[x] = o.lay[x];
                d.H = o.H;
                if (o.save != nullptr) {
                    if (!causal || o.reversed || dtype == COTT_F32)
                        return fail(COTT_ERR_UNSUPPORTED, "%s: states are saved by a forward-direction 16-bit causal op", fn);
                    d.save = o.save;  // (the column half is found from c0)
                    d.save_njt = cott::mfma_pad(o.dj) / 16;
                    d.save_slot = cott::mfma_pad(o.di) * cott::mfma_pad(o.dj);
                    d.save_cpg = o.save_cpg;
                    d.save_n = o.save_n;
                }
                if (o.ext != nullptr) {
                    if (!d.comp || p.G != o.save_n || p.cpg != o.save_cpg)
                        return fail(COTT_ERR_INVALID, "%s: the saved states were cut for another plan (%d cuts of %d chunks; "
                                    "this launch needs %d of %d, complement form %d)", fn, o.save_n, o.save_cpg, p.G, p.cpg, d.comp);
                    d.ext = o.ext;  // saved by an op with this op's dims swapped
                    d.save_njt = cott::mfma_pad(o.di) / 16;
                    d.save_slot = cott::mfma_pad(o.di) * cott::mfma_pad(o.dj);
                    d.save_cpg = o.save_cpg;
                    d.save_n = o.save_n;
                }
            }
        }
        a.ws = p.ws_bytes ? reinterpret_cast<float *>(ws_cursor) : nullptr;
        ws_cursor += p.ws_bytes;
        a.BH = (int)BH; a.N = N;
        a.nchunks = p.nchunks; a.cpg = p.cpg; a.G = p.G; a.sub = p.sub;
        a.cus = device_cus();
        a.xcds = device_xcds();
        a.scan_prof_id = n > 1 ? cott::K_SCAN_GRAD : cott::K_SCAN;
        a.stream = stream;
        hipError_t e;
        if (dtype == COTT_F32)
            e = causal ? cott::launch_causal_mfma_f32(a) : cott::launch_noncausal_mfma_f32(a);
        else if (dtype == COTT_BF16)
            e = causal ? cott::launch_causal_mfma_bf16(a) : cott::launch_noncausal_mfma_bf16(a);
        else
            e = causal ? cott::launch_causal_mfma_fp16(a) : cott::launch_noncausal_mfma_fp16(a);
        if (e != hipSuccess) return fail(COTT_ERR_HIP, "%s: HIP launch failed: %s", fn, hipGetErrorString(e));
    }
    return COTT_OK;
}

// The three gradients as generic ops with permuted operands (Cuda_Kernel/Custom_Kernel.py:106-108;
// for the non-causal form dq = d_o (v^T k), dk = v (d_o^T q), dv = k (q^T d_o), nothing reversed).
void grad_ops(Op *ops, const void *q, const void *k, const void *v, const void *d_o, void *dq, void *dk, void *dv, int Dk,
              int Dv, bool causal) {
    ops[0] = Op{d_o, v, k, dq, Dv, Dk, 0};
    ops[1] = Op{v, d_o, q, dk, Dv, Dk, causal ? 1 : 0};
    ops[2] = Op{k, q, d_o, dv, Dk, Dv, causal ? 1 : 0};
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
                                               "scan_kernel<apply>", "scan_kernel<causal> (dQ,dK,dV set)", "generic_scan_kernel",
                                               "decode_kernel", "prep_kernel", "stream_probe_kernel"};
    return (kernel_id >= 0 && kernel_id < cott::K_COUNT) ? names[kernel_id] : "";
}

const char *cott_last_error(void) { return g_err; }

size_t cott_causal_workspace_bytes(int B, int H, int N, int Dk, int Dv, int dtype) {
    const Op op{nullptr, nullptr, nullptr, nullptr, Dk, Dv, 0};
    return ops_workspace(&op, 1, (long)B * H, N, dtype, true);
}

int cott_causal_fwd(const void *q, const void *k, const void *v, void *o, int B, int H, int N, int Dk, int Dv,
                    int dtype, int reversed, void *workspace, size_t workspace_bytes, void *stream) {
    const char *fn = "cott_causal_fwd";
    if (int rc = check_common(fn, B, H, N, Dk, Dv, dtype)) return rc;
    if ((long)B * H * N == 0) return COTT_OK;
    if (!q || !k || !v || !o) return fail(COTT_ERR_INVALID, "%s: null tensor pointer", fn);
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o))
        return fail(COTT_ERR_INVALID, "%s: tensor pointers must be 16-byte aligned", fn);
    const Op op{q, k, v, o, Dk, Dv, reversed ? 1 : 0};
    return run_ops(fn, true, &op, 1, (long)B * H, N, dtype, workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}

int cott_causal_fwd_may_alias_v(int B, int H, int N, int Dk, int Dv, int dtype) {
    // The MFMA scan kernels load the v rows of a chunk before they store its outputs, every workgroup reads only the
    // rows (sequence group) and columns (column half) it writes, and the group-state pass has finished with v
    // before the scan starts.  The plain-FMA kernels declare their operands __restrict__.
    if (check_common("cott_causal_fwd_may_alias_v", B, H, N, Dk, Dv, dtype) != COTT_OK) return 0;
    return use_mfma(dtype, Dk, Dv, N) ? 1 : 0;
}

int cott_causal_fwd_prep_supported(int B, int H, int N, int Dk, int Dv, int dtype, int rotary_dim) {
    if (B < 0 || H < 0 || N < 0 || (dtype != COTT_BF16 && dtype != COTT_F16) || Dk % 16 != 0 || Dk < 32) return 0;
    if (!use_mfma(dtype, Dk, Dv, N)) return 0;
    if (rotary_dim != 0 && (rotary_dim < 8 || rotary_dim % 8 != 0 || rotary_dim > Dk)) return 0;
    const long dmax = Dk > Dv ? Dk : Dv;
    if ((long)N * H * dmax > (1L << 30) || (long)B * H > (1L << 22)) return 0;
    if ((long)B * H * N == 0) return 1;
    const SetPlan p = plan_set((long)B * H, N, 1, Dk, Dv, true, dtype);
    // q / k rows of up to 64 columns are prepared by scan_kernel's loader wavefronts, 128-wide rows by colscan_kernel's
    // (value tiles of 64 or 128 columns there); sequences cut into groups take a group-state pass that prepares k and v
    // the same way
    const int pk = cott::mfma_pad(Dk), pv = cott::mfma_pad(Dv / p.halves);
    return (pk <= 64 && pk * pv <= 128 * 64) || (pk == 128 && pv >= 64);
}

int cott_causal_fwd_prep_preferred(int B, int H, int N, int Dk, int Dv, int dtype, int rotary_dim) {
    if (!cott_causal_fwd_prep_supported(B, H, N, Dk, Dv, dtype, rotary_dim)) return 0;
    if ((long)B * H * N == 0) return 1;
    // Measured in a loop over one shape, rotary 32 with position ids, mask and value scaling, one launch against
    // cott_prep_ex_fwd + cott_causal_fwd.  Heads that are one group: B16 H16 N2048 D64 113 against 137 us, D128 210
    // against 275; B32 H16 N2048 D128 413 against 563; in column halves B8 H16 N2048 D64 61 against 60..67, N8192 282
    // against 306, D128 N2048 143 against 160, N8192 509 against 628.  Whole problems in sequence groups (the sums of
    // 64- and 128-wide rows by colsum_prep_kernel): B1 H16 N65536 D128 567 against 722, N32768 312 against 372, B4 H16
    // N8192 D128 305 against 338, B2 H12 N32768 D128 460 against 522; D64 even or a little ahead (B4 H16 N32768 598
    // against 650, N8192 166 against 161, B1 H16 N32768 170 against 169).  Column halves in groups are slower: both
    // halves of a head prepare its q and k rows and so does the group-state pass (B2 H12 N8192 D64 92 against 65, D128
    // 183 against 149; B1 H16 N8192 D128 112 against 92).
    const SetPlan p = plan_set((long)B * H, N, 1, Dk, Dv, true, dtype);
    return p.G == 1 || p.halves == 1;
}

namespace {
int fwd_prep_impl(const char *fn, const void *q, const void *k, const void *v, void *o, void *q_out, void *k_out,
                  void *v_out, const unsigned char *keep, const float *cnt, const float *sig, const float *rot_table,
                  const long long *pos_ids, long long pos0, int rotary_dim, int table_rows, int in_bnhd, int o_bnhd, float *saved, int chunks_per_cut,
                  int ncuts, int B, int H, int N, int Dk, int Dv, int dtype, void *workspace, size_t workspace_bytes,
                  void *stream) {
    if (int rc = check_common(fn, B, H, N, Dk, Dv, dtype)) return rc;
    if (dtype != COTT_BF16 && dtype != COTT_F16)
        return fail(COTT_ERR_UNSUPPORTED, "%s: needs bf16 / fp16 tensors", fn);
    if (!use_mfma(dtype, Dk, Dv, N))
        return fail(COTT_ERR_UNSUPPORTED, "%s: needs head dims 32..128 in steps of 16", fn);
    if ((cnt == nullptr) != (sig == nullptr)) return fail(COTT_ERR_INVALID, "%s: cnt and sig go together", fn);
    if (rot_table != nullptr) {
        if (rotary_dim < 8 || rotary_dim % 8 != 0 || rotary_dim > Dk)
            return fail(COTT_ERR_INVALID, "%s: rotary_dim must be a multiple of 8 in [8, Dk] (got %d)", fn, rotary_dim);
        if (table_rows < 1) return fail(COTT_ERR_INVALID, "%s: empty rotary table", fn);
    }
    if ((long)B * H * N == 0) return COTT_OK;
    if (!cott_causal_fwd_prep_supported(B, H, N, Dk, Dv, dtype, rot_table ? rotary_dim : 0))
        return fail(COTT_ERR_UNSUPPORTED, "%s: the fused preparation is not built for these head dims "
                    "(cott_causal_fwd_prep_supported); prepare the inputs with cott_prep_ex_fwd instead", fn);
    if (in_bnhd || o_bnhd) {
        const long dmax = Dk > Dv ? Dk : Dv;
        if ((long)N * H * dmax > (1L << 30))
            return fail(COTT_ERR_UNSUPPORTED, "%s: N*H*D = %ld exceeds 2^30", fn, (long)N * H * dmax);
    }
    if (!q || !k || !v || !o) return fail(COTT_ERR_INVALID, "%s: null tensor pointer", fn);
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o) || !aligned16(q_out) || !aligned16(k_out) ||
        !aligned16(v_out) || !aligned16(rot_table))
        return fail(COTT_ERR_INVALID, "%s: tensor pointers must be 16-byte aligned", fn);
    if (reinterpret_cast<uintptr_t>(pos_ids) & 7u) return fail(COTT_ERR_INVALID, "%s: position ids must be 8-byte aligned", fn);
    if ((long)N > (1L << 28)) return fail(COTT_ERR_UNSUPPORTED, "%s: N = %d exceeds 2^28", fn, N);
    Op op{q, k, v, o, Dk, Dv, 0};
    op.H = H;
    if (in_bnhd) op.lay[0] = op.lay[1] = op.lay[2] = 1;
    if (o_bnhd) op.lay[3] = 1;
    if (saved != nullptr) {
        if (chunks_per_cut < 1 || ncuts < 1 || (long)(ncuts - 1) * chunks_per_cut > (N + 63) / 64 - 1)
            return fail(COTT_ERR_INVALID, "%s: %d cuts of %d chunks do not fit %d positions (ask cott_causal_saved_plan)", fn,
                        ncuts, chunks_per_cut, N);
        if (!aligned16(saved)) return fail(COTT_ERR_INVALID, "%s: tensor pointers must be 16-byte aligned", fn);
        op.save = saved;
        op.save_cpg = chunks_per_cut;
        op.save_n = ncuts;
    }
    cott::SetArgs::Prep prep;
    prep.on = true;
    prep.keep = keep;
    prep.cnt = cnt;
    prep.sig = sig;
    prep.rot = rot_table;
    prep.pos = rot_table ? pos_ids : nullptr;
    prep.pos0 = pos0;
    prep.R = rot_table ? rotary_dim : 0;
    prep.table_rows = table_rows;
    prep.H = H;
    prep.dv = Dv;
    prep.qo = q_out;
    prep.ko = k_out;
    prep.vo = v_out;
    return run_ops(fn, true, &op, 1, (long)B * H, N, dtype, workspace, workspace_bytes, static_cast<hipStream_t>(stream), &prep);
}
}  // namespace

int cott_causal_fwd_prep(const void *q, const void *k, const void *v, void *o, void *q_out, void *k_out, void *v_out,
                         const unsigned char *keep, const float *cnt, const float *sig, const float *rot_table,
                         const long long *pos_ids, long long pos0, int rotary_dim, int table_rows, int in_bnhd, int o_bnhd, int B,
                         int H, int N, int Dk, int Dv, int dtype, void *workspace, size_t workspace_bytes, void *stream) {
    return fwd_prep_impl("cott_causal_fwd_prep", q, k, v, o, q_out, k_out, v_out, keep, cnt, sig, rot_table, pos_ids, pos0, rotary_dim,
                         table_rows, in_bnhd, o_bnhd, nullptr, 0, 0, B, H, N, Dk, Dv, dtype, workspace, workspace_bytes, stream);
}

int cott_causal_fwd_prep_save(const void *q, const void *k, const void *v, void *o, void *q_out, void *k_out, void *v_out,
                              const unsigned char *keep, const float *cnt, const float *sig, const float *rot_table,
                              const long long *pos_ids, long long pos0, int rotary_dim, int table_rows, int in_bnhd, int o_bnhd, float *saved,
                              int chunks_per_cut, int ncuts, int B, int H, int N, int Dk, int Dv, int dtype, void *workspace,
                              size_t workspace_bytes, void *stream) {
    const char *fn = "cott_causal_fwd_prep_save";
    if ((long)B * H * N != 0 && saved == nullptr) return fail(COTT_ERR_INVALID, "%s: null tensor pointer", fn);
    return fwd_prep_impl(fn, q, k, v, o, q_out, k_out, v_out, keep, cnt, sig, rot_table, pos_ids, pos0, rotary_dim, table_rows,
                         in_bnhd, o_bnhd, saved, chunks_per_cut, ncuts, B, H, N, Dk, Dv, dtype, workspace, workspace_bytes, stream);
}

int cott_noncausal_fwd_prep_supported(int B, int H, int N, int Dk, int Dv, int dtype) {
    if (B < 0 || H < 0 || N < 0 || (dtype != COTT_BF16 && dtype != COTT_F16) || Dk % 16 != 0 || Dk < 32) return 0;
    if (!use_mfma(dtype, Dk, Dv, N)) return 0;
    const long dmax = Dk > Dv ? Dk : Dv;
    if ((long)N * H * dmax > (1L << 30) || (long)B * H > (1L << 22)) return 0;
    if ((long)B * H * N == 0) return 1;
    // one workgroup (or two column halves) per head (B16 H16 N512 D128: 56 us against 60 us for the two kernels;
    // B32 H12 N512 D64: 40 against 47 us)
    return plan_set((long)B * H, N, 1, Dk, Dv, false, dtype).G == 1;
}

int cott_noncausal_fwd_prep(const void *q, const void *k, const void *v, void *o, void *q_out, void *k_out, void *v_out,
                            const unsigned char *keep, const float *cnt, const float *sig, int in_bnhd, int o_bnhd, int B,
                            int H, int N, int Dk, int Dv, int dtype, void *stream) {
    const char *fn = "cott_noncausal_fwd_prep";
    if (int rc = check_common(fn, B, H, N, Dk, Dv, dtype)) return rc;
    if (dtype != COTT_BF16 && dtype != COTT_F16) return fail(COTT_ERR_UNSUPPORTED, "%s: needs bf16 / fp16 tensors", fn);
    if (!use_mfma(dtype, Dk, Dv, N)) return fail(COTT_ERR_UNSUPPORTED, "%s: needs head dims 32..128 in steps of 16", fn);
    if ((cnt == nullptr) != (sig == nullptr)) return fail(COTT_ERR_INVALID, "%s: cnt and sig go together", fn);
    if ((long)B * H * N == 0) return COTT_OK;
    if (!cott_noncausal_fwd_prep_supported(B, H, N, Dk, Dv, dtype))
        return fail(COTT_ERR_UNSUPPORTED, "%s: the fused preparation needs bf16 / fp16 heads that fit one "
                    "workgroup (cott_noncausal_fwd_prep_supported); prepare the inputs with cott_prep_ex_fwd instead", fn);
    if (!q || !k || !v || !o) return fail(COTT_ERR_INVALID, "%s: null tensor pointer", fn);
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o) || !aligned16(q_out) || !aligned16(k_out) ||
        !aligned16(v_out))
        return fail(COTT_ERR_INVALID, "%s: tensor pointers must be 16-byte aligned", fn);
    Op op{q, k, v, o, Dk, Dv, 0};
    op.H = H;
    if (in_bnhd) op.lay[0] = op.lay[1] = op.lay[2] = 1;
    if (o_bnhd) op.lay[3] = 1;
    cott::SetArgs::Prep prep;
    prep.on = true;
    prep.keep = keep;
    prep.cnt = cnt;
    prep.sig = sig;
    prep.rot = nullptr;
    prep.pos0 = 0;
    prep.R = 0;
    prep.table_rows = 0;
    prep.H = H;
    prep.dv = Dv;
    prep.qo = q_out;
    prep.ko = k_out;
    prep.vo = v_out;
    return run_ops(fn, false, &op, 1, (long)B * H, N, dtype, nullptr, 0, static_cast<hipStream_t>(stream), &prep);
}

namespace {
// dst[i] = src ? src[i] : 0 over n 16-byte vectors: the state pass-through of an empty sequence.  A kernel rather than
// hipMemsetAsync / hipMemcpyAsync so that the call can be recorded into a HIP graph like every other launch here.
__global__ __launch_bounds__(256) void state_passthrough_kernel(uint4 *dst, const uint4 *src, size_t n) {
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) dst[i] = src ? src[i] : uint4{0u, 0u, 0u, 0u};
}

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
void *g_scratch_ptr[kMaxDevices] = {nullptr};

// Device address of `scratch` on the current device, looked up once per device.
int scratch_of_current_device(const char *fn, void **out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(COTT_ERR_HIP, "%s: hipGetDevice failed: %s", fn, hipGetErrorString(e));
    if (dev < 0 || dev >= kMaxDevices) return fail(COTT_ERR_UNSUPPORTED, "%s: device index %d not below %d", fn, dev, kMaxDevices);
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (g_scratch_ptr[dev] == nullptr) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || p == nullptr)
            return fail(COTT_ERR_HIP, "%s: hipGetSymbolAddress(scratch) failed on device %d: %s", fn, dev, hipGetErrorString(e));
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return COTT_OK;
}
}  // namespace

// Also resolves the scratch array's address on the current device (when there is one), so that a caller who asks for
// the size before recording cott_causal_fwd_noalloc into a HIP graph has the symbol lookup, and whatever code-object
// loading it triggers, behind it when the capture starts.
size_t cott_noalloc_scratch_bytes(void) {
    int count = 0;
    if (hipGetDeviceCount(&count) == hipSuccess && count > 0) {
        void *p = nullptr;
        (void)scratch_of_current_device("cott_noalloc_scratch_bytes", &p);
    } else {
        (void)hipGetLastError();  // no device: only the size is wanted (host-side checks)
    }
    return (size_t)COTT_SCRATCH_BYTES;
}

int cott_causal_fwd_noalloc(const void *q, const void *k, const void *v, void *o, int B, int H, int N, int Dk, int Dv,
                            int dtype, int reversed, void *stream) {
    const char *fn = "cott_causal_fwd_noalloc";
    if (int rc = check_common(fn, B, H, N, Dk, Dv, dtype)) return rc;
    if ((long)B * H * N == 0) return COTT_OK;
    if (!q || !k || !v || !o) return fail(COTT_ERR_INVALID, "%s: null tensor pointer", fn);
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o))
        return fail(COTT_ERR_INVALID, "%s: tensor pointers must be 16-byte aligned", fn);
    const Op op{q, k, v, o, Dk, Dv, reversed ? 1 : 0};
    const size_t need = ops_workspace(&op, 1, (long)B * H, N, dtype, true);
    if (need > (size_t)COTT_SCRATCH_BYTES)
        return fail(COTT_ERR_WORKSPACE, "%s: this shape needs %zu bytes of group-state slots, the built-in scratch holds %zu; "
                    "use cott_causal_fwd with a workspace", fn, need, (size_t)COTT_SCRATCH_BYTES);
    void *ws = nullptr;
    if (need > 0)
        if (int rc = scratch_of_current_device(fn, &ws)) return rc;
    return run_ops(fn, true, &op, 1, (long)B * H, N, dtype, ws, need, static_cast<hipStream_t>(stream));
}

int cott_causal_fwd_state(const void *q, const void *k, const void *v, void *o, const void *state_in, void *state_out,
                          int B, int H, int N, int Dk, int Dv, int dtype, void *workspace, size_t workspace_bytes,
                          void *stream) {
    const char *fn = "cott_causal_fwd_state";
    if (int rc = check_common(fn, B, H, N, Dk, Dv, dtype)) return rc;
    const long BH = (long)B * H;
    if (BH == 0) return COTT_OK;
    const size_t ssz = dtype == COTT_F64 ? 8 : 4;
    const uintptr_t smask = dtype == COTT_F64 ? 31u : 15u;
    if ((reinterpret_cast<uintptr_t>(state_in) & smask) || (reinterpret_cast<uintptr_t>(state_out) & smask))
        return fail(COTT_ERR_INVALID, "%s: state pointers must be 16-byte (fp64: 32-byte) aligned", fn);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (N == 0) {  // nothing to scan: the state passes through (or starts at zero)
        if (state_out && state_out != state_in) {
            const size_t bytes = (size_t)BH * Dk * Dv * ssz;
            if (bytes % 16 != 0) return fail(COTT_ERR_UNSUPPORTED, "%s: state size %zu is not a multiple of 16 bytes", fn, bytes);
            const size_t n16 = bytes / 16;
            const unsigned blocks = (unsigned)((n16 + 255) / 256 < 2048 ? (n16 + 255) / 256 : 2048);
            state_passthrough_kernel<<<dim3(blocks ? blocks : 1), dim3(256), 0, st>>>(
                static_cast<uint4 *>(state_out), static_cast<const uint4 *>(state_in), n16);
            hipError_t e = hipGetLastError();
            if (e != hipSuccess) return fail(COTT_ERR_HIP, "%s: state pass-through failed: %s", fn, hipGetErrorString(e));
        }
        return COTT_OK;
    }
    if (!q || !k || !v || !o) return fail(COTT_ERR_INVALID, "%s: null tensor pointer", fn);
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o))
        return fail(COTT_ERR_INVALID, "%s: tensor pointers must be 16-byte aligned", fn);
    Op op{q, k, v, o, Dk, Dv, 0};
    op.sin = state_in;
    op.sout = state_out;
    return run_ops(fn, true, &op, 1, BH, N, dtype, workspace, workspace_bytes, st);
}

size_t cott_causal_bwd_workspace_bytes(int B, int H, int N, int Dk, int Dv, int dtype) {
    Op ops[3];
    grad_ops(ops, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, Dk, Dv, true);
    return ops_workspace(ops, 3, (long)B * H, N, dtype, true);
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
    Op ops[3];
    grad_ops(ops, q, k, v, d_o, dq, dk, dv, Dk, Dv, true);
    return run_ops(fn, true, ops, 3, (long)B * H, N, dtype, workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}

namespace {
// Whether the backward pass of this shape takes states saved by the forward pass, and how they are cut: dQ must run
// in complement form in a set cut into G > 1 groups (16-bit MFMA kernels, no pair workgroups).
bool saved_states_plan(long BH, int N, int Dk, int Dv, int dtype, int *cpg, int *ncuts, size_t *bwd_ws) {
    *cpg = 0;
    *ncuts = 0;
    if (bwd_ws) *bwd_ws = 0;
    if ((dtype != COTT_BF16 && dtype != COTT_F16) || BH * N == 0) return false;
    if (!use_mfma(dtype, Dk, Dv, N) || !use_mfma(dtype, Dv, Dk, N)) return false;
    Op ops[3];
    char tag[8];  // distinct stand-in addresses: the layout only compares operands
    grad_ops(ops, tag + 0, tag + 1, tag + 2, tag + 3, tag + 4, tag + 5, tag + 6, Dk, Dv, true);
    ops[0].ext = tag + 7;  // plan as the backward pass would with the states at hand
    int members[8], cnt = 0;
    for (int j = 0; j < 3; ++j)
        if (pad_key(ops[j]) == pad_key(ops[0])) members[cnt++] = j;
    const SetLayout L = layout_set(ops, 3, members, cnt, BH, N, dtype, true);
    // dQ takes the states where it runs in complement form: in sets cut into groups, and beside a (dK, dV) pair
    // (there also when a head is one group: the one slot is then the sum over the whole sequence)
    if (!L.pair && !L.complement) return false;
    // Sequences of a few chunks gain nothing from it (at 8 chunks the extra tensor costs the host side of the call more
    // than the kernels gain), and their rows would lose precision: in complement form the rows of the first chunk are
    // a difference of two sums rounded to 16 bits instead of one short sum.
    if (L.p.nchunks < 16) return false;
    *cpg = L.p.cpg;
    *ncuts = L.p.G;
    if (bwd_ws) {
        ops[0].save_cpg = L.p.cpg;
        ops[0].save_n = L.p.G;
        *bwd_ws = ops_workspace(ops, 3, BH, N, dtype, true);
    }
    return true;
}
}  // namespace

int cott_causal_saved_plan(int B, int H, int N, int Dk, int Dv, int dtype, int *chunks_per_cut, int *ncuts,
                           int *slot_floats, size_t *bwd_workspace_bytes) {
    const char *fn = "cott_causal_saved_plan";
    if (!chunks_per_cut || !ncuts || !slot_floats) return fail(COTT_ERR_INVALID, "%s: null result pointer", fn);
    *chunks_per_cut = 0;
    *ncuts = 0;
    *slot_floats = 0;
    if (bwd_workspace_bytes) *bwd_workspace_bytes = 0;
    if (elem_size(dtype) == 0 || B < 0 || H < 0 || N < 0 || Dk < 1 || Dv < 1)
        return fail(COTT_ERR_INVALID, "%s: bad shape or dtype", fn);
    if (saved_states_plan((long)B * H, N, Dk, Dv, dtype, chunks_per_cut, ncuts, bwd_workspace_bytes))
        *slot_floats = cott::mfma_pad(Dk) * cott::mfma_pad(Dv);
    return COTT_OK;
}

int cott_plan_geometry(int cus, int xcds) {
    if (cus < 0 || xcds < 0 || (cus > 0 && xcds > 0 && cus % xcds != 0))
        return fail(COTT_ERR_INVALID, "cott_plan_geometry: %d CUs in %d XCDs", cus, xcds);
    g_cus_given.store(cus, std::memory_order_relaxed);
    g_xcds_given.store(xcds, std::memory_order_relaxed);
    return COTT_OK;
}

int cott_plan_describe(int which, int with_saved_states, int B, int H, int N, int Dk, int Dv, int dtype, int *sets,
                       int *nsets) {
    const char *fn = "cott_plan_describe";
    if (!sets || !nsets || which < 0 || which > 3) return fail(COTT_ERR_INVALID, "%s: bad argument", fn);
    *nsets = 0;
    if (elem_size(dtype) == 0 || B < 0 || H < 0 || N < 0 || Dk < 1 || Dv < 1)
        return fail(COTT_ERR_INVALID, "%s: bad shape or dtype", fn);
    const bool causal = which < 2, grads = (which & 1) != 0;
    if ((long)B * H * N == 0 || !use_mfma(dtype, Dk, Dv, N) || (grads && !use_mfma(dtype, Dv, Dk, N))) return COTT_OK;
    Op ops[3];
    int n = 1;
    char tag[8];  // distinct stand-in addresses, never dereferenced: the layout only compares operands
    if (grads) {
        grad_ops(ops, tag + 0, tag + 1, tag + 2, tag + 3, tag + 4, tag + 5, tag + 6, Dk, Dv, causal);
        n = 3;
        if (with_saved_states && causal) {
            int cpc = 0, cuts = 0;
            if (saved_states_plan((long)B * H, N, Dk, Dv, dtype, &cpc, &cuts, nullptr)) {
                ops[0].ext = tag + 7;
                ops[0].save_cpg = cpc;
                ops[0].save_n = cuts;
            }
        }
    } else {
        ops[0] = Op{tag + 0, tag + 1, tag + 2, tag + 3, Dk, Dv, 0};
    }
    int members[8][8], counts[8];
    const int ns = form_sets(ops, n, (long)B * H, N, dtype, causal, members, counts);
    for (int s = 0; s < ns; ++s) {
        const SetLayout L = layout_set(ops, n, members[s], counts[s], (long)B * H, N, dtype, causal);
        int *o = sets + 8 * s;
        const int per_unit = L.pair ? 2 : counts[s] * L.p.halves;
        o[0] = counts[s];
        o[1] = L.p.halves;
        o[2] = L.p.G;
        o[3] = L.p.cpg;
        o[4] = L.p.sub;
        o[5] = L.pair ? 1 : 0;
        o[6] = L.complement ? 1 : 0;
        const long x = device_xcds();  // (head, group) units rounded up to whole rounds of the XCDs, as the launchers do
        o[7] = (int)((((long)B * H * L.p.G + x - 1) / x) * x * per_unit);
    }
    *nsets = ns;
    return COTT_OK;
}

namespace {
int check_interleaved(const char *fn, int H, int N, int Dk, int Dv, int dtype);

int fwd_save_impl(const char *fn, bool o_bnhd, const void *q, const void *k, const void *v, void *o, float *saved,
                  int chunks_per_cut, int ncuts, int B, int H, int N, int Dk, int Dv, int dtype, void *workspace,
                  size_t workspace_bytes, void *stream) {
    if (int rc = check_common(fn, B, H, N, Dk, Dv, dtype)) return rc;
    if ((dtype != COTT_BF16 && dtype != COTT_F16) || !use_mfma(dtype, Dk, Dv, N))
        return fail(COTT_ERR_UNSUPPORTED, "%s: needs bf16 / fp16 tensors and head dims 32..128 in steps of 16", fn);
    if (chunks_per_cut < 1 || ncuts < 1 || (long)(ncuts - 1) * chunks_per_cut > (N + 63) / 64 - 1)
        return fail(COTT_ERR_INVALID, "%s: %d cuts of %d chunks do not fit %d positions (ask cott_causal_saved_plan)", fn,
                    ncuts, chunks_per_cut, N);
    if ((long)B * H * N == 0) return COTT_OK;
    if (!q || !k || !v || !o || !saved) return fail(COTT_ERR_INVALID, "%s: null tensor pointer", fn);
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o) || !aligned16(saved))
        return fail(COTT_ERR_INVALID, "%s: tensor pointers must be 16-byte aligned", fn);
    if (o_bnhd)
        if (int rc = check_interleaved(fn, H, N, Dk, Dv, dtype)) return rc;
    Op op{q, k, v, o, Dk, Dv, 0};
    op.save = saved;
    op.save_cpg = chunks_per_cut;
    op.save_n = ncuts;
    if (o_bnhd) op.lay[3] = 1;
    op.H = H;
    return run_ops(fn, true, &op, 1, (long)B * H, N, dtype, workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}

int bwd_saved_impl(const char *fn, bool do_bnhd, const void *q, const void *k, const void *v, const void *d_o, void *dq,
                   void *dk, void *dv, const float *saved, int chunks_per_cut, int ncuts, int B, int H, int N, int Dk, int Dv,
                   int dtype, void *workspace, size_t workspace_bytes, void *stream) {
    if (int rc = check_common(fn, B, H, N, Dk, Dv, dtype)) return rc;
    if (int rc = check_common(fn, B, H, N, Dv, Dk, dtype)) return rc;
    if ((long)B * H * N == 0) return COTT_OK;
    int cpg = 0, cuts = 0;
    if (!saved_states_plan((long)B * H, N, Dk, Dv, dtype, &cpg, &cuts, nullptr))
        return fail(COTT_ERR_UNSUPPORTED, "%s: the backward pass of this shape takes no saved states "
                    "(cott_causal_saved_plan gives 0 cuts); call cott_causal_bwd", fn);
    if (cpg != chunks_per_cut || cuts != ncuts)
        return fail(COTT_ERR_INVALID, "%s: states saved as %d cuts of %d chunks, this shape needs %d of %d", fn, ncuts,
                    chunks_per_cut, cuts, cpg);
    if (!q || !k || !v || !d_o || !dq || !dk || !dv || !saved) return fail(COTT_ERR_INVALID, "%s: null tensor pointer", fn);
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(d_o) || !aligned16(dq) || !aligned16(dk) ||
        !aligned16(dv) || !aligned16(saved))
        return fail(COTT_ERR_INVALID, "%s: tensor pointers must be 16-byte aligned", fn);
    if (do_bnhd)
        if (int rc = check_interleaved(fn, H, N, Dk, Dv, dtype)) return rc;
    Op ops[3];
    grad_ops(ops, q, k, v, d_o, dq, dk, dv, Dk, Dv, true);
    ops[0].ext = saved;
    ops[0].save_cpg = chunks_per_cut;
    ops[0].save_n = ncuts;
    if (do_bnhd) {
        ops[0].lay[0] = 1;  // d_o is A of dq, B of dk, C of dv (see cott_causal_bwd_bnhd)
        ops[1].lay[1] = 1;
        ops[2].lay[2] = 1;
    }
    for (int i = 0; i < 3; ++i) ops[i].H = H;
    return run_ops(fn, true, ops, 3, (long)B * H, N, dtype, workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}
}  // namespace

int cott_causal_fwd_save(const void *q, const void *k, const void *v, void *o, float *saved, int chunks_per_cut,
                         int ncuts, int B, int H, int N, int Dk, int Dv, int dtype, void *workspace,
                         size_t workspace_bytes, void *stream) {
    return fwd_save_impl("cott_causal_fwd_save", false, q, k, v, o, saved, chunks_per_cut, ncuts, B, H, N, Dk, Dv, dtype,
                         workspace, workspace_bytes, stream);
}
int cott_causal_fwd_save_bnhd(const void *q, const void *k, const void *v, void *o, float *saved, int chunks_per_cut,
                              int ncuts, int B, int H, int N, int Dk, int Dv, int dtype, void *workspace,
                              size_t workspace_bytes, void *stream) {
    return fwd_save_impl("cott_causal_fwd_save_bnhd", true, q, k, v, o, saved, chunks_per_cut, ncuts, B, H, N, Dk, Dv, dtype,
                         workspace, workspace_bytes, stream);
}
int cott_causal_bwd_saved(const void *q, const void *k, const void *v, const void *d_o, void *dq, void *dk, void *dv,
                          const float *saved, int chunks_per_cut, int ncuts, int B, int H, int N, int Dk, int Dv,
                          int dtype, void *workspace, size_t workspace_bytes, void *stream) {
    return bwd_saved_impl("cott_causal_bwd_saved", false, q, k, v, d_o, dq, dk, dv, saved, chunks_per_cut, ncuts, B, H, N, Dk,
                          Dv, dtype, workspace, workspace_bytes, stream);
}
int cott_causal_bwd_saved_bnhd(const void *q, const void *k, const void *v, const void *d_o, void *dq, void *dk, void *dv,
                               const float *saved, int chunks_per_cut, int ncuts, int B, int H, int N, int Dk, int Dv,
                               int dtype, void *workspace, size_t workspace_bytes, void *stream) {
    return bwd_saved_impl("cott_causal_bwd_saved_bnhd", true, q, k, v, d_o, dq, dk, dv, saved, chunks_per_cut, ncuts, B, H, N,
                          Dk, Dv, dtype, workspace, workspace_bytes, stream);
}

namespace {
// (B,N,H,D) operands are addressed with 32-bit byte offsets inside one batch element
int check_interleaved(const char *fn, int H, int N, int Dk, int Dv, int dtype) {
    if (dtype != COTT_BF16 && dtype != COTT_F16)
        return fail(COTT_ERR_UNSUPPORTED, "%s: (B,N,H,D) operands need bf16 / fp16 tensors", fn);
    if (!use_mfma(dtype, Dk, Dv, N) || !use_mfma(dtype, Dv, Dk, N))
        return fail(COTT_ERR_UNSUPPORTED, "%s: (B,N,H,D) operands need head dims 32..128 in steps of 16", fn);
    const long dmax = Dk > Dv ? Dk : Dv;
    if ((long)N * H * dmax > (1L << 30))
        return fail(COTT_ERR_UNSUPPORTED, "%s: N*H*D = %ld exceeds 2^30", fn, (long)N * H * dmax);
    return COTT_OK;
}
}  // namespace

int cott_causal_fwd_bnhd(const void *q, const void *k, const void *v, void *o, int B, int H, int N, int Dk, int Dv,
                         int dtype, void *workspace, size_t workspace_bytes, void *stream) {
    const char *fn = "cott_causal_fwd_bnhd";
    if (int rc = check_common(fn, B, H, N, Dk, Dv, dtype)) return rc;
    if ((long)B * H * N == 0) return COTT_OK;
    if (int rc = check_interleaved(fn, H, N, Dk, Dv, dtype)) return rc;
    if (!q || !k || !v || !o) return fail(COTT_ERR_INVALID, "%s: null tensor pointer", fn);
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o))
        return fail(COTT_ERR_INVALID, "%s: tensor pointers must be 16-byte aligned", fn);
    Op op{q, k, v, o, Dk, Dv, 0};
    op.lay[3] = 1;
    op.H = H;
    return run_ops(fn, true, &op, 1, (long)B * H, N, dtype, workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}

int cott_causal_bwd_bnhd(const void *q, const void *k, const void *v, const void *d_o, void *dq, void *dk, void *dv,
                         int B, int H, int N, int Dk, int Dv, int dtype, void *workspace, size_t workspace_bytes,
                         void *stream) {
    const char *fn = "cott_causal_bwd_bnhd";
    if (int rc = check_common(fn, B, H, N, Dk, Dv, dtype)) return rc;
    if (int rc = check_common(fn, B, H, N, Dv, Dk, dtype)) return rc;
    if ((long)B * H * N == 0) return COTT_OK;
    if (int rc = check_interleaved(fn, H, N, Dk, Dv, dtype)) return rc;
    if (!q || !k || !v || !d_o || !dq || !dk || !dv) return fail(COTT_ERR_INVALID, "%s: null tensor pointer", fn);
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(d_o) || !aligned16(dq) || !aligned16(dk) ||
        !aligned16(dv))
        return fail(COTT_ERR_INVALID, "%s: tensor pointers must be 16-byte aligned", fn);
    Op ops[3];
    grad_ops(ops, q, k, v, d_o, dq, dk, dv, Dk, Dv, true);
    ops[0].lay[0] = 1;  // dq = G(d_o, v, k):      d_o is A
    ops[1].lay[1] = 1;  // dk = G(v, d_o, q, rev): d_o is B
    ops[2].lay[2] = 1;  // dv = G(k, q, d_o, rev): d_o is C
    for (int i = 0; i < 3; ++i) ops[i].H = H;
    return run_ops(fn, true, ops, 3, (long)B * H, N, dtype, workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}

int cott_noncausal_fwd_bnhd(const void *q, const void *k, const void *v, void *o, int B, int H, int N, int Dk, int Dv,
                            int dtype, void *workspace, size_t workspace_bytes, void *stream) {
    const char *fn = "cott_noncausal_fwd_bnhd";
    if (int rc = check_common(fn, B, H, N, Dk, Dv, dtype)) return rc;
    if ((long)B * H * N == 0) return COTT_OK;
    if (int rc = check_interleaved(fn, H, N, Dk, Dv, dtype)) return rc;
    if (!q || !k || !v || !o) return fail(COTT_ERR_INVALID, "%s: null tensor pointer", fn);
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o))
        return fail(COTT_ERR_INVALID, "%s: tensor pointers must be 16-byte aligned", fn);
    Op op{q, k, v, o, Dk, Dv, 0};
    op.lay[3] = 1;
    op.H = H;
    return run_ops(fn, false, &op, 1, (long)B * H, N, dtype, workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}

int cott_noncausal_bwd_bnhd(const void *q, const void *k, const void *v, const void *d_o, void *dq, void *dk, void *dv,
                            int B, int H, int N, int Dk, int Dv, int dtype, void *workspace, size_t workspace_bytes,
                            void *stream) {
    const char *fn = "cott_noncausal_bwd_bnhd";
    if (int rc = check_common(fn, B, H, N, Dk, Dv, dtype)) return rc;
    if (int rc = check_common(fn, B, H, N, Dv, Dk, dtype)) return rc;
    if ((long)B * H * N == 0) return COTT_OK;
    if (int rc = check_interleaved(fn, H, N, Dk, Dv, dtype)) return rc;
    if (!q || !k || !v || !d_o || !dq || !dk || !dv) return fail(COTT_ERR_INVALID, "%s: null tensor pointer", fn);
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(d_o) || !aligned16(dq) || !aligned16(dk) ||
        !aligned16(dv))
        return fail(COTT_ERR_INVALID, "%s: tensor pointers must be 16-byte aligned", fn);
    Op ops[3];
    grad_ops(ops, q, k, v, d_o, dq, dk, dv, Dk, Dv, false);
    ops[0].lay[0] = 1;
    ops[1].lay[1] = 1;
    ops[2].lay[2] = 1;
    for (int i = 0; i < 3; ++i) ops[i].H = H;
    return run_ops(fn, false, ops, 3, (long)B * H, N, dtype, workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}

size_t cott_noncausal_workspace_bytes(int B, int H, int N, int Dk, int Dv, int dtype) {
    Op ops[3];
    grad_ops(ops, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, Dk, Dv, false);
    const size_t bwd = ops_workspace(ops, 3, (long)B * H, N, dtype, false);
    const Op op{nullptr, nullptr, nullptr, nullptr, Dk, Dv, 0};
    const size_t fwd = ops_workspace(&op, 1, (long)B * H, N, dtype, false);
    return fwd > bwd ? fwd : bwd;
}

int cott_noncausal_fwd(const void *q, const void *k, const void *v, void *o, int B, int H, int N, int Dk, int Dv,
                       int dtype, void *workspace, size_t workspace_bytes, void *stream) {
    const char *fn = "cott_noncausal_fwd";
    if (int rc = check_common(fn, B, H, N, Dk, Dv, dtype)) return rc;
    if ((long)B * H * N == 0) return COTT_OK;
    if (!q || !k || !v || !o) return fail(COTT_ERR_INVALID, "%s: null tensor pointer", fn);
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o))
        return fail(COTT_ERR_INVALID, "%s: tensor pointers must be 16-byte aligned", fn);
    const Op op{q, k, v, o, Dk, Dv, 0};
    return run_ops(fn, false, &op, 1, (long)B * H, N, dtype, workspace, workspace_bytes, static_cast<hipStream_t>(stream));
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
    Op ops[3];
    grad_ops(ops, q, k, v, d_o, dq, dk, dv, Dk, Dv, false);
    return run_ops(fn, false, ops, 3, (long)B * H, N, dtype, workspace, workspace_bytes, static_cast<hipStream_t>(stream));
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

int cott_decode_step_prep(void *state, const void *q, const void *k, const void *v, void *o, const float *sig, float cnt,
                          const float *rot_table, long long position, int rotary_dim, int table_rows, int B, int H,
                          int Dk, int Dv, int dtype, void *stream) {
    const char *fn = "cott_decode_step_prep";
    if (elem_size(dtype) == 0) return fail(COTT_ERR_INVALID, "%s: unknown dtype %d", fn, dtype);
    if (B < 0 || H < 0 || Dk < 1 || Dv < 1) return fail(COTT_ERR_INVALID, "%s: bad size", fn);
    const int nv = Dv / 4;
    if (Dv % 4 != 0 || !(nv == 8 || nv == 16 || nv == 32 || nv == 64) || Dk > 256)
        return fail(COTT_ERR_UNSUPPORTED, "%s: needs Dv in {32, 64, 128, 256} and Dk <= 256 (got Dk=%d Dv=%d)", fn, Dk, Dv);
    const long BH = (long)B * H;
    if (BH == 0) return COTT_OK;
    if (BH >= (1L << 31)) return fail(COTT_ERR_UNSUPPORTED, "%s: B*H too large", fn);
    if (!state || !q || !k || !v || !o) return fail(COTT_ERR_INVALID, "%s: null pointer", fn);
    if (!aligned16(state) || (dtype == COTT_F64 && (reinterpret_cast<uintptr_t>(state) & 31u)))
        return fail(COTT_ERR_INVALID, "%s: state must be 16-byte (fp64: 32-byte) aligned", fn);
    long long pos = 0;
    if (rot_table != nullptr) {
        if (rotary_dim < 2 || rotary_dim % 2 != 0 || rotary_dim > Dk)
            return fail(COTT_ERR_INVALID, "%s: rotary_dim must be even and in [2, Dk] (got %d)", fn, rotary_dim);
        if (table_rows < 1) return fail(COTT_ERR_INVALID, "%s: empty rotary table", fn);
        pos = position < 0 ? 0 : (position >= table_rows ? table_rows - 1 : position);  // clamped like the batched pass
    }
    hipError_t e = cott::launch_decode_prep(dtype, state, q, k, v, o, (int)BH, H, Dk, Dv, sig, cnt, rot_table, pos, rotary_dim,
                                            1e-12f, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return fail(COTT_ERR_HIP, "%s: HIP launch failed: %s", fn, hipGetErrorString(e));
    return COTT_OK;
}

namespace {
int check_prep(const char *fn, int B, int H, int N, int Dk, int Dv, int d0, int d1) {
    if (elem_size(d0) == 0 || elem_size(d1) == 0) return fail(COTT_ERR_INVALID, "%s: unknown dtype", fn);
    if (B < 0 || H < 0 || N < 0 || Dk < 1 || Dv < 1) return fail(COTT_ERR_INVALID, "%s: bad size", fn);
    if (Dk % 4 != 0 || Dv % 4 != 0) return fail(COTT_ERR_UNSUPPORTED, "%s: head dims must be multiples of 4", fn);
    if (Dk > 1024 || Dv > 1024) return fail(COTT_ERR_UNSUPPORTED, "%s: head dims above 1024", fn);
    if ((d0 == COTT_F64) != (d1 == COTT_F64)) return fail(COTT_ERR_UNSUPPORTED, "%s: fp64 only converts to fp64", fn);
    return COTT_OK;
}
int check_rotary(const char *fn, const float *table, const long long *pos, int R, int rows, int Dk) {
    if (table == nullptr && pos == nullptr) return COTT_OK;
    if (table == nullptr || pos == nullptr) return fail(COTT_ERR_INVALID, "%s: rotary table and positions go together", fn);
    if (R < 4 || R % 4 != 0 || R > Dk)
        return fail(COTT_ERR_INVALID, "%s: rotary_dim must be a multiple of 4 in [4, Dk] (got %d)", fn, R);
    if (rows < 1) return fail(COTT_ERR_INVALID, "%s: empty rotary table", fn);
    return COTT_OK;
}
}  // namespace

int cott_prep_ex_fwd(const void *q, const void *k, const void *v, void *q_out, void *k_out, void *v_out,
                     const unsigned char *keep, const float *cnt, const float *sig, const float *rot_table,
                     const long long *pos, int rotary_dim, int table_rows, int in_bnhd, int B, int H, int N, int Dk,
                     int Dv, int in_dtype, int out_dtype, void *stream) {
    const char *fn = "cott_prep_ex_fwd";
    if (int rc = check_prep(fn, B, H, N, Dk, Dv, in_dtype, out_dtype)) return rc;
    if (int rc = check_rotary(fn, rot_table, pos, rotary_dim, table_rows, Dk)) return rc;
    if ((long)B * H * N == 0) return COTT_OK;
    if (!q || !k || !v || !q_out || !k_out || !v_out) return fail(COTT_ERR_INVALID, "%s: null tensor pointer", fn);
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(q_out) || !aligned16(k_out) || !aligned16(v_out))
        return fail(COTT_ERR_INVALID, "%s: tensor pointers must be 16-byte aligned", fn);
    if ((cnt == nullptr) != (sig == nullptr)) return fail(COTT_ERR_INVALID, "%s: cnt and sig go together", fn);
    const void *x[3] = {q, k, v};
    void *y[3] = {q_out, k_out, v_out};
    hipError_t e = cott::launch_prep(false, x, nullptr, y, keep, cnt, sig, nullptr, B, H, N, Dk, Dv, in_dtype, out_dtype,
                                     out_dtype, 1e-12f, in_bnhd ? 1 : 0, rot_table, pos, rot_table ? rotary_dim : 0,
                                     table_rows, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return fail(COTT_ERR_HIP, "%s: HIP launch failed: %s", fn, hipGetErrorString(e));
    return COTT_OK;
}

int cott_prep_ex_bwd(const void *q, const void *k, const void *v, const void *gq, const void *gk, const void *gv,
                     void *dq, void *dk, void *dv, float *dsig_rows, const unsigned char *keep, const float *cnt,
                     const float *sig, const float *rot_table, const long long *pos, int rotary_dim, int table_rows,
                     int in_bnhd, int B, int H, int N, int Dk, int Dv, int in_dtype, int grad_dtype, void *stream) {
    const char *fn = "cott_prep_ex_bwd";
    if (int rc = check_prep(fn, B, H, N, Dk, Dv, in_dtype, grad_dtype)) return rc;
    if (int rc = check_rotary(fn, rot_table, pos, rotary_dim, table_rows, Dk)) return rc;
    if ((long)B * H * N == 0) return COTT_OK;
    if (!q || !k || !v || !gq || !gk || !gv || !dq || !dk || !dv) return fail(COTT_ERR_INVALID, "%s: null tensor pointer", fn);
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(gq) || !aligned16(gk) || !aligned16(gv) ||
        !aligned16(dq) || !aligned16(dk) || !aligned16(dv))
        return fail(COTT_ERR_INVALID, "%s: tensor pointers must be 16-byte aligned", fn);
    if ((cnt == nullptr) != (sig == nullptr)) return fail(COTT_ERR_INVALID, "%s: cnt and sig go together", fn);
    const void *x[3] = {q, k, v};
    const void *g[3] = {gq, gk, gv};
    void *y[3] = {dq, dk, dv};
    hipError_t e = cott::launch_prep(true, x, g, y, keep, cnt, sig, dsig_rows, B, H, N, Dk, Dv, in_dtype, in_dtype,
                                     grad_dtype, 1e-12f, in_bnhd ? 1 : 0, rot_table, pos, rot_table ? rotary_dim : 0,
                                     table_rows, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return fail(COTT_ERR_HIP, "%s: HIP launch failed: %s", fn, hipGetErrorString(e));
    return COTT_OK;
}

int cott_prep_fwd(const void *q, const void *k, const void *v, void *q_out, void *k_out, void *v_out,
                  const unsigned char *keep, const float *cnt, const float *sig, int B, int H, int N, int Dk, int Dv,
                  int in_dtype, int out_dtype, void *stream) {
    return cott_prep_ex_fwd(q, k, v, q_out, k_out, v_out, keep, cnt, sig, nullptr, nullptr, 0, 0, 0, B, H, N, Dk, Dv,
                            in_dtype, out_dtype, stream);
}

int cott_prep_bwd(const void *q, const void *k, const void *v, const void *gq, const void *gk, const void *gv, void *dq,
                  void *dk, void *dv, float *dsig_rows, const unsigned char *keep, const float *cnt, const float *sig,
                  int B, int H, int N, int Dk, int Dv, int in_dtype, int grad_dtype, void *stream) {
    return cott_prep_ex_bwd(q, k, v, gq, gk, gv, dq, dk, dv, dsig_rows, keep, cnt, sig, nullptr, nullptr, 0, 0, 0, B, H,
                            N, Dk, Dv, in_dtype, grad_dtype, stream);
}

}  // extern "C"
