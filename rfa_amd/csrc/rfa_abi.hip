// C ABI of librfa_hip.so: argument validation, launch planning and kernel
// launches.  See include/rfa_hip.h for the contract of every entry point.
#include "../../include/rfa_hip.h"

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "rfa_causal.h"
#include "rfa_sliced.h"
#include "rfa_project.h"
#include "rfa_decode.h"
#include "rfa_featuremap.h"
#include "rfa_masked.h"

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

#define RFA_HIP_TRY(expr)                                                                    \
    do {                                                                                     \
        hipError_t e_ = (expr);                                                              \
        if (e_ != hipSuccess)                                                                \
            return fail(RFA_ERR_HIP, "%s failed: %s", #expr, hipGetErrorString(e_));         \
    } while (0)


// ---- optional per-kernel timing with HIP events ------------------------------------
namespace prof {
enum Id { SEG_STATE, CAUSAL_FWD, CAUSAL_BWD_DQ, CAUSAL_BWD_DKDV, CROSS_READOUT, CROSS_READOUT_BWD,
          CROSS_STATE_BWD, DECODE_STEP, FEATURE_FWD, FEATURE_BWD, FEATURE_DW_REDUCE, MASKED_FWD, MASKED_PREP, MASKED_DQ, MASKED_DKDV, PROJECT_PHI, WGRAD_PARTIAL, WGRAD_REDUCE, TOTALS_SCAN, ZERO_FILL,
          SELFTEST, BUILD_W, DECODE_TOUCH, CAUSAL_BWD_SLICED, COPY_ROWS, COUNT };
const char* const kNames[COUNT] = {"k_segment_state", "k_causal_fwd", "k_causal_bwd_dq", "k_causal_bwd_dkdv",
                                   "k_cross_readout", "k_cross_readout_bwd", "k_cross_state_bwd", "k_decode_step",
                                   "k_feature_map_fwd", "k_feature_map_bwd", "k_feature_map_dw_reduce",
                                   "k_masked_fwd", "k_masked_bwd_prep", "k_masked_dq", "k_masked_dkdv", "k_project_phi",
                                   "k_weight_grad_partial", "k_weight_grad_reduce", "k_totals_scan",
                                   "k_zero_f32", "k_selftest", "k_build_random_matrices", "k_touch_rows",
                                   "k_sliced_bwd", "k_copy_rows_strided"};
struct Rec { int id; hipEvent_t a, b; };
std::mutex mu;
bool enabled = false;
std::vector<Rec> recs;
std::vector<hipEvent_t> pool;
double total_ms[COUNT] = {};
long long calls[COUNT] = {};

hipEvent_t take_event() {
    if (!pool.empty()) { hipEvent_t e = pool.back(); pool.pop_back(); return e; }
    hipEvent_t e = nullptr;
    (void)hipEventCreate(&e);
    return e;
}

// One kernel launch.  While profiling is on the launch carries a start/stop event pair
// that takes the kernel's own begin and end timestamps (hipExtLaunchKernelGGL), i.e. the
// same interval a kernel trace reports, without the launch latency around it.
template <typename F, typename... Args>
void launch(int id, F kern, dim3 grid, dim3 block, size_t lds, hipStream_t st, Args... args) {
    if (enabled) {
        std::lock_guard<std::mutex> lk(mu);
        hipEvent_t a = take_event(), b = take_event();
        if (a && b) {
            hipExtLaunchKernelGGL(kern, grid, block, (uint32_t)lds, st, a, b, 0, args...);
            recs.push_back({id, a, b});
            return;
        }
        if (a) pool.push_back(a);
        if (b) pool.push_back(b);
    }
    hipLaunchKernelGGL(kern, grid, block, lds, st, args...);
}
}  // namespace prof

#define RFA_LAUNCH(ID, ...) prof::launch(prof::ID, __VA_ARGS__)

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---- tuning knobs --------------------------------------------------------------------
// Process-wide overrides of the launch heuristics, for sweeps and for tests that must reach
// every code path at small sizes.  -1 = the heuristic.  The environment is read once, when the
// first knob is looked up, never on the launch path; rfa_tuning_set changes a knob afterwards.
namespace tune {
enum Key { NSEG, PREFIX, NSEG_SAME, FREE_WG, PROJECT_STREAMING, SLICED, RECOMPUTE, PREFIX_COST, FEATURE_WG, COUNT };
const char* const kNames[COUNT] = {"nseg", "prefix", "nseg_same", "free_wg", "project_streaming", "sliced", "recompute", "prefix_cost", "feature_wg"};
const char* const kEnv[COUNT] = {"RFA_HIP_NSEG", "RFA_HIP_PREFIX", "RFA_HIP_NSEG_SAME", "RFA_HIP_FREE_WG",
                                 "RFA_HIP_PROJECT_STREAMING", "RFA_HIP_SLICED", "RFA_HIP_RECOMPUTE",
                                 "RFA_HIP_PREFIX_COST", "RFA_HIP_FEATURE_WG"};
std::atomic<int> value[COUNT];
std::once_flag once;

void init() {
    for (int i = 0; i < COUNT; ++i) {
        int v = -1;
        if (const char* env = getenv(kEnv[i])) {
            char* end = nullptr;
            const long x = strtol(env, &end, 10);
            if (end != env && x >= 0 && x <= (1 << 20)) v = (int)x;
        }
        value[i].store(v, std::memory_order_relaxed);
    }
}

int get(Key k) {
    std::call_once(once, init);
    return value[k].load(std::memory_order_relaxed);
}

int find(const char* name) {
    if (!name) return -1;
    for (int i = 0; i < COUNT; ++i)
        if (strcmp(name, kNames[i]) == 0) return i;
    return -1;
}
}  // namespace tune

// Compute units of the current device (256 on an MI355X in its default partition mode);
// queried once per device.  Without a device (a host that only asks for buffer sizes) the
// MI355X figure is assumed.
int device_cus() {
    constexpr int kMaxDev = 64;
    static std::atomic<int> cache[kMaxDev];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDev) {
        (void)hipGetLastError();
        return 256;
    }
    int cus = cache[dev].load(std::memory_order_relaxed);
    if (cus <= 0) {
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) {
            (void)hipGetLastError();
            cus = 256;
        }
        cache[dev].store(cus, std::memory_order_relaxed);
    }
    return cus;
}

struct ScanPlan {
    int nseg;      // segments per sequence
    int seg_len;   // steps per segment (multiple of 64)
    int prefixed;  // the consumers read one pre-scanned state (k_totals_scan) instead of adding up the
                   // segment totals themselves
    int layout;    // what a saving forward leaves for the backward (SavedLayout)
};

// What rfa_causal_forward_save hands to the backward besides the raw denominators:
//   LAYOUT_SEGMENTS  the per-segment state totals; the backward runs the two segment sweeps
//   LAYOUT_FINAL     the state after the last step; the backward walks whole sequences backwards
//                    in state slices (rfa_sliced.h), one launch, every chunk read once
enum SavedLayout { LAYOUT_SEGMENTS = 0, LAYOUT_FINAL = 1 };

bool sliced_supported(int K, int d) { return (K == 64 || K == 128) && (d == 64 || d == 128); }

// The sliced backward has N * (K / 64 + d / 64) workgroups that never wait for each other, each
// walking a whole sequence.  Taken when they cover enough of the compute units ("sliced" knob: 0
// never, 1 whenever a kernel exists).  Measured against the two time-segmented sweeps at T = 1024:
// d = 64, K = 128 wins from 120 workgroups on (N = 40: 34.8 vs 37.3 us, N = 64: 34 vs 43, N = 512:
// 262 vs 285); d = 128 wins with K = 128 at 256 workgroups (60 vs 67 us) and loses with K = 64 at
// 192 (54 vs 50 us).
int choose_saved_layout(int64_t N, int K, int d) {
    if (!sliced_supported(K, d)) return LAYOUT_SEGMENTS;
    // its loader addresses the 64 rows of a chunk with 32-bit byte offsets
    if ((int64_t)rfa::kChunk * N * (K > d ? K : d) * 2 >= ((int64_t)1 << 32)) return LAYOUT_SEGMENTS;
    const int knob = tune::get(tune::SLICED);
    if (knob >= 0) return knob ? LAYOUT_FINAL : LAYOUT_SEGMENTS;
    const int64_t wgs = N * (K / rfa::kSliceWidth + d / rfa::kSliceWidth), cus = device_cus();
    if (d == 64) return wgs * 100 >= cus * 45 ? LAYOUT_FINAL : LAYOUT_SEGMENTS;
    return K == 128 && wgs * 10 >= cus * 9 ? LAYOUT_FINAL : LAYOUT_SEGMENTS;
}

// Whether the consumers read one pre-scanned state instead of adding up the segment totals
// themselves, (nseg - 1) / 2 states of K * d floats on average per workgroup: worth its pass over
// the totals from 128 KiB of such reads on.
bool use_scanned_totals(int nseg, int K, int d) {
    if (nseg < 2) return false;
    const int knob = tune::get(tune::PREFIX);
    if (knob >= 0) return knob != 0;
    return (int64_t)(nseg - 1) * K * d * 2 >= 128 * 1024;
}

// Enough (sequence, segment) workgroups to cover the compute units, at least two
// chunks per segment, at most 16 segments (the consumer sums the totals of all
// earlier segments).
ScanPlan make_plan(int64_t T, int64_t N, int K, int d) {
    ScanPlan p{1, rfa::kChunk, 0, LAYOUT_SEGMENTS};
    if (T <= 0 || N <= 0) return p;
    p.layout = choose_saved_layout(N, K, d);
    const int64_t nchunks = (T + rfa::kChunk - 1) / rfa::kChunk;
    int64_t want = (device_cus() + N - 1) / N;
    const int knob = tune::get(tune::NSEG);
    if (knob >= 1) {
        want = knob;
    } else {
        if (want > nchunks / 2) want = nchunks / 2;
    }
    if (want > rfa::kMaxSegments) want = rfa::kMaxSegments;
    if (want > nchunks) want = nchunks;
    if (want < 1) want = 1;
    const int64_t cps = (nchunks + want - 1) / want;
    p.nseg = (int)((nchunks + cps - 1) / cps);
    p.seg_len = (int)(cps * rfa::kChunk);
    p.prefixed = use_scanned_totals(p.nseg, K, d) ? 1 : 0;
    return p;
}

// ---- description of a saved-state buffer ---------------------------------------------
constexpr size_t kSavedHeaderBytes = 256;

rfa::PlanWords plan_words(int64_t T, int64_t N, int K, int d, const ScanPlan& p) {
    rfa::PlanWords w{};
    w.w[0] = rfa::kPlanMagic;
    w.w[1] = 1;
    w.w[2] = p.layout;
    w.w[3] = K;
    w.w[4] = d;
    w.w[5] = p.nseg;
    w.w[6] = p.seg_len;
    w.w[7] = p.prefixed;
    w.w[8] = (int)(T & 0xffffffff);
    w.w[9] = (int)(T >> 32);
    w.w[10] = (int)(N & 0xffffffff);
    w.w[11] = (int)(N >> 32);
    return w;
}

// What the last rfa_causal_forward_save wrote at each saved-buffer address, kept on the host so
// that the backward call runs with that forward's plan whatever the knobs say by then.  The table
// is a hint, never an authority: addresses come back from the caller's allocator for other
// buffers, so a record may describe a buffer that no longer exists.  The backward kernels always
// compare the header on the device with the plan they were launched for (NaN gradients on a
// mismatch); a record of another shape than the call's is dropped and the call falls back to the
// current plan, like a buffer the table does not know (copied by the caller, written by another
// process).  The table holds the most recent kRegistryEntries forwards; the oldest go first.
namespace registry {
constexpr size_t kRegistryEntries = 4096;
std::mutex mu;
std::unordered_map<const void*, rfa::PlanWords> table;
std::deque<const void*> order;       // addresses in the order they first entered the table

void put(const void* saved, const rfa::PlanWords& w) {
    std::lock_guard<std::mutex> lk(mu);
    auto it = table.find(saved);
    if (it != table.end()) {
        it->second = w;
        return;
    }
    while (table.size() >= kRegistryEntries && !order.empty()) {
        table.erase(order.front());
        order.pop_front();
    }
    table.emplace(saved, w);
    order.push_back(saved);
}

bool get(const void* saved, rfa::PlanWords* w) {
    std::lock_guard<std::mutex> lk(mu);
    auto it = table.find(saved);
    if (it == table.end()) return false;
    *w = it->second;
    return true;
}

// the address stays in `order`; put() tolerates entries whose record is already gone
void drop(const void* saved) {
    std::lock_guard<std::mutex> lk(mu);
    table.erase(saved);
}
}  // namespace registry

size_t align_up(size_t x) { return (x + 255) & ~size_t(255); }

struct Workspace {
    // all offsets in bytes from the workspace base
    size_t S, Z, R, r, den, gz, total;
};

Workspace layout_workspace(int64_t T, int64_t N, int K, int d, const ScanPlan& p, bool backward) {
    Workspace w{};
    size_t off = 0;
    const size_t seg_states = (size_t)N * p.nseg;
    w.S = off; off = align_up(off + (p.nseg > 1 ? seg_states * K * d * 4 : 0));
    w.Z = off; off = align_up(off + (p.nseg > 1 ? seg_states * K * 4 : 0));
    if (backward) {
        w.R = off; off = align_up(off + (p.nseg > 1 ? seg_states * K * d * 4 : 0));
        w.r = off; off = align_up(off + (p.nseg > 1 ? seg_states * K * 4 : 0));
        w.den = off; off = align_up(off + (size_t)T * N * 4);
        w.gz = off; off = align_up(off + (size_t)T * N * 4);
    }
    w.total = off;
    return w;
}

// wavefronts per workgroup of the scan kernels: 8 where the per-wave share of the fp32
// state would not fit the register file with 4 (K >= 128 with d = 128)
constexpr int causal_waves(int KD, int DH) { return (DH >= 128 && KD >= 128) ? 8 : 4; }
// the dQ sweep owns feature-row slices only, so it can run 8 waves (two per SIMD) whenever
// K >= 128
constexpr int dq_waves(int KD, int DH) { return KD >= 128 ? 8 : 4; }

// waves that own the forward state (value-column slices): 4 in the two-stage pipelined forward
template <int KD, int DH>
constexpr int fwd_state_waves_v = (rfa::FwdPipeCfg<KD, DH>::kLds <= 160 * 1024) ? 4 : causal_waves(KD, DH);

template <typename Kern>
int set_lds(Kern kern, size_t bytes) {
    RFA_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
    return RFA_OK;
}

template <bool REVERSE>
void launch_totals_scan(float* a, int64_t Ma, float* b, int64_t Mb, int N, int nseg, hipStream_t st) {
    const int64_t threads = (Ma + Mb) / 4;
    RFA_LAUNCH(TOTALS_SCAN, rfa::k_totals_scan<REVERSE>, dim3((unsigned)((threads + 255) / 256), (unsigned)N),
               dim3(rfa::kThreads), 0, st, a, Ma, b, Mb, nseg);
}

// The forward without segment totals (k_causal_fwd_pipe<.., RECOMPUTE>): every workgroup rebuilds
// the state at its segment's first step from the k, v rows before it.  A prefix chunk costs
// about an eighth of a scan chunk ("prefix_cost" knob, percent; measured at T = 1024, N = 64:
// 10 and 15 give 18.8 us, 20 to 30 give 19.0 to 19.2), so segment s gets
// u - cost * first[s] chunks, with u the smallest figure whose segments cover the sequence:
// prefix plus scan then take every workgroup about equally long.  Pays while a sequence has few
// segments (the last one streams nearly the whole sequence): up to 4 ("recompute" knob: 0 never,
// 1 whenever the kernel exists).  False if no such cut exists.
bool recompute_bounds(int64_t T, int nseg, rfa::SegBounds* b) {
    const int knob = tune::get(tune::RECOMPUTE);
    if (knob == 0 || nseg < 2 || nseg > rfa::kMaxSegments || (knob < 0 && nseg > 4)) return false;
    const int nch = (int)((T + rfa::kChunk - 1) / rfa::kChunk);
    const int cost_knob = tune::get(tune::PREFIX_COST);
    const double cost = (cost_knob >= 0 ? cost_knob : 12) / 100.0;
    for (double u = (double)nch / nseg; u <= nch; u += 0.25) {
        b->first[0] = 0;
        for (int s_ = 0; s_ < nseg; ++s_) {
            int len = (int)(u - cost * b->first[s_] + 1e-9);
            if (len < 1) len = 1;
            b->first[s_ + 1] = b->first[s_] + len;
        }
        if (b->first[nseg] < nch) continue;
        if (b->first[nseg - 1] >= nch) return false;        // the cut leaves a segment empty
        b->first[nseg] = nch;
        for (int s_ = nseg + 1; s_ <= rfa::kMaxSegments; ++s_) b->first[s_] = nch;
        return true;
    }
    return false;
}

template <int KD, int DH>
int launch_forward(const rfa::half_t* q, const rfa::half_t* k, const rfa::half_t* v, rfa::half_t* out,
                   int T, int N, const ScanPlan& p, char* ws, const Workspace& wl, int* savedHdr, float* savedS,
                   float* savedZ, float* savedDen, float* final_s, float* final_z, bool allow_recompute,
                   hipStream_t st) {
    // the two-stage pipelined forward needs both chunk buffers in LDS: K <= 128
    constexpr bool PIPE = rfa::FwdPipeCfg<KD, DH>::kLds <= 160 * 1024;
    constexpr int NW = PIPE ? 4 : causal_waves(KD, DH);
    static_assert(NW == fwd_state_waves_v<KD, DH>, "fragment layout of the segment totals");
    using Cfg = rfa::CausalCfg<KD, DH, NW>;
    // with a saved buffer the segment totals are written there directly (S in the forward's
    // fragment order, which the saved-pair backward reads as is)
    const rfa::PlanWords pw = plan_words(T, N, KD, DH, p);
    if constexpr (PIPE) {
        // nobody else reads the totals (the saved pair of this layout keeps only the final state):
        // one launch that needs none
        rfa::SegBounds bounds{};
        if (allow_recompute && !savedS && recompute_bounds(T, p.nseg, &bounds) &&
            (int64_t)rfa::kChunk * N * (KD > DH ? KD : DH) * 2 < ((int64_t)1 << 32)) {
            auto kern = rfa::k_causal_fwd_pipe<KD, DH, true>;
            if (int rc = set_lds(kern, rfa::FwdPipeCfg<KD, DH>::kLds)) return rc;
            RFA_LAUNCH(CAUSAL_FWD, kern, dim3(N * p.nseg), dim3(512), rfa::FwdPipeCfg<KD, DH>::kLds, st, q, k, v, out,
                       (const float*)nullptr, (const float*)nullptr, savedDen, final_s, final_z, T, N, p.nseg, p.seg_len, 0,
                       savedHdr, pw, bounds, 0);
            RFA_HIP_TRY(hipGetLastError());
            return RFA_OK;
        }
    }
    if (p.nseg > 1 && !ws && !savedS)
        return fail(RFA_ERR_WORKSPACE, "rfa_causal_forward: this shape needs a workspace for its segment totals");
    float* wsS = savedS ? savedS : reinterpret_cast<float*>(ws + wl.S);
    float* wsZ = savedZ ? savedZ : reinterpret_cast<float*>(ws + wl.Z);
    if (p.nseg > 1) {
        auto kern = rfa::k_segment_state<KD, DH, NW, true>;
        if (int rc = set_lds(kern, Cfg::kSegStateLds)) return rc;
        RFA_LAUNCH(SEG_STATE, kern, dim3(N * (p.nseg - 1)), dim3(64 * NW), Cfg::kSegStateLds, st,
                           k, v, (const uint8_t*)nullptr, 1, wsS, wsZ, (float*)nullptr, T, N, p.nseg, p.nseg - 1, p.seg_len);
    }
    if (p.prefixed) launch_totals_scan<false>(wsS, (int64_t)KD * DH, wsZ, KD, N, p.nseg, st);
    if constexpr (PIPE) {
        auto kern = rfa::k_causal_fwd_pipe<KD, DH, false>;
        if (int rc = set_lds(kern, rfa::FwdPipeCfg<KD, DH>::kLds)) return rc;
        RFA_LAUNCH(CAUSAL_FWD, kern, dim3(N * p.nseg), dim3(512), rfa::FwdPipeCfg<KD, DH>::kLds, st, q, k, v, out,
                           wsS, wsZ, savedDen, final_s, final_z, T, N, p.nseg, p.seg_len, p.prefixed, savedHdr, pw,
                           rfa::SegBounds{}, (int64_t)rfa::kChunk * N * (KD > DH ? KD : DH) * 2 >= ((int64_t)1 << 32) ? 1 : 0);
    } else {
        auto kern = rfa::k_causal_fwd<KD, DH, NW, true>;
        if (int rc = set_lds(kern, Cfg::kFwdLds)) return rc;
        RFA_LAUNCH(CAUSAL_FWD, kern, dim3(N * p.nseg), dim3(64 * NW), Cfg::kFwdLds, st, q, k, v, out,
                           wsS, wsZ, savedDen, final_s, final_z, T, N, p.nseg, p.seg_len, p.prefixed, savedHdr, pw);
    }
    RFA_HIP_TRY(hipGetLastError());
    return RFA_OK;
}

// The cut into segments the backward sweeps use for a forward plan pf.  Where both sweeps run as two
// workgroups per (sequence, segment) and the totals are scanned, the backward takes segments twice
// as long: half as many workgroups already cover the compute units, in one round instead of two.
ScanPlan backward_plan(const ScanPlan& pf, int K, int d, bool have_saved, int* s_ratio) {
    ScanPlan p = pf;
    *s_ratio = 1;
    if (K >= 256 && d >= 128 && have_saved && pf.prefixed && pf.nseg >= 4 && pf.nseg % 2 == 0 &&
        tune::get(tune::NSEG_SAME) <= 0) {
        p.nseg = pf.nseg / 2;
        p.seg_len = 2 * pf.seg_len;
        p.prefixed = use_scanned_totals(p.nseg, K, d) ? 1 : 0;      // of dR, dr
        *s_ratio = 2;
    }
    return p;
}

template <int KD, int DH>
int launch_backward(const rfa::half_t* q, const rfa::half_t* k, const rfa::half_t* v,
                    const rfa::half_t* g, const rfa::half_t* out, rfa::half_t* dq, rfa::half_t* dk,
                    rfa::half_t* dv, int T, int N, const ScanPlan& pf, char* ws, const Workspace& wl,
                    const int* savedHdr, const float* savedS, const float* savedZ, const float* savedDen,
                    hipStream_t st) {
    // pf is the forward's cut into segments (that of the saved totals)
    int s_ratio = 1;
    const ScanPlan p = backward_plan(pf, KD, DH, savedS != nullptr, &s_ratio);
    const int prefixed_s = pf.prefixed;
    const int prefixed = p.prefixed;   // of dR, dr
    const rfa::PlanWords pw = plan_words(T, N, KD, DH, pf);
    constexpr int NW = causal_waves(KD, DH);
    using Cfg = rfa::CausalCfg<KD, DH, NW>;
    float* wsS = reinterpret_cast<float*>(ws + wl.S);
    float* wsZ = reinterpret_cast<float*>(ws + wl.Z);
    float* wsR = reinterpret_cast<float*>(ws + wl.R);
    float* wsr = reinterpret_cast<float*>(ws + wl.r);
    float* den = reinterpret_cast<float*>(ws + wl.den);
    float* gz = reinterpret_cast<float*>(ws + wl.gz);
    const float* inS = wsS;
    const float* inZ = wsZ;
    if (savedS) {          // segment totals handed over by the forward pass (already scanned if prefixed_s)
        inS = savedS;
        inZ = savedZ;
    } else if (p.nseg > 1) {
        auto kern = rfa::k_segment_state<KD, DH, NW, false>;
        if (int rc = set_lds(kern, Cfg::kSegStateLds)) return rc;
        RFA_LAUNCH(SEG_STATE, kern, dim3(N * (p.nseg - 1)), dim3(64 * NW), Cfg::kSegStateLds, st,
                           k, v, (const uint8_t*)nullptr, 1, wsS, wsZ, (float*)nullptr, T, N, p.nseg, p.nseg - 1, p.seg_len);
        if (prefixed_s) launch_totals_scan<false>(wsS, (int64_t)KD * DH, wsZ, KD, N, p.nseg, st);
    }
    const float* den_in = den;
    if (savedDen) {
        // the forward's output and raw denominators are at hand: the sweep that needs no A = Q K^T
        if constexpr (KD >= 256 && DH >= 128) {
            // both carried states of one workgroup would not fit the register file: the feature
            // rows split over two workgroups (half of S^T and of R^T each)
            constexpr int KL = KD / 2;
            constexpr int NWQ = dq_waves(KL, DH);
            using CfgQ = rfa::CausalCfg<KL, DH, NWQ>;
            auto kern = rfa::k_causal_bwd_dq_saved<KL, DH, NWQ, fwd_state_waves_v<KD, DH>, KD>;
            if (int rc = set_lds(kern, CfgQ::kBwdDqSavedLds)) return rc;
            RFA_LAUNCH(CAUSAL_BWD_DQ, kern, dim3(2 * N * p.nseg), dim3(64 * NWQ), CfgQ::kBwdDqSavedLds, st, q, k, v, g,
                       out, savedDen, dq, inS, inZ, wsR, wsr, gz, T, N, p.nseg, p.seg_len, prefixed_s, pf.nseg, s_ratio,
                       savedHdr, pw);
        } else {
            constexpr int NWQ = dq_waves(KD, DH);
            using CfgQ = rfa::CausalCfg<KD, DH, NWQ>;
            auto kern = rfa::k_causal_bwd_dq_saved<KD, DH, NWQ, fwd_state_waves_v<KD, DH>>;
            if (int rc = set_lds(kern, CfgQ::kBwdDqSavedLds)) return rc;
            RFA_LAUNCH(CAUSAL_BWD_DQ, kern, dim3(N * p.nseg), dim3(64 * NWQ), CfgQ::kBwdDqSavedLds, st, q, k, v, g, out,
                       savedDen, dq, inS, inZ, wsR, wsr, gz, T, N, p.nseg, p.seg_len, prefixed_s, pf.nseg, s_ratio,
                       savedHdr, pw);
        }
        den_in = savedDen;
    } else {
        constexpr int NWQ = dq_waves(KD, DH);
        using CfgQ = rfa::CausalCfg<KD, DH, NWQ>;
        auto kern = rfa::k_causal_bwd_dq<KD, DH, NWQ, true>;
        if (int rc = set_lds(kern, CfgQ::kBwdDqLds)) return rc;
        RFA_LAUNCH(CAUSAL_BWD_DQ, kern, dim3(N * p.nseg), dim3(64 * NWQ), CfgQ::kBwdDqLds, st, q, k, v, g,
                           dq, inS, inZ, wsR, wsr, den, gz, T, N, p.nseg, p.seg_len, prefixed_s);
    }
    // the dQ sweep left the totals of dR, dr of segments 1 .. nseg - 1
    if (prefixed) launch_totals_scan<true>(wsR, (int64_t)KD * DH, wsr, KD, N, p.nseg, st);
    if constexpr (KD >= 256) {
        // two copies of R in one workgroup would not fit the register file: dK and dV in separate
        // workgroups (one copy each); measured 2.5x (d = 64) and 1.7x (d = 128) faster at K = 256,
        // slower than the shared tile phase below at K <= 128
        constexpr int NWR = (KD >= 128 && DH >= 128) ? 8 : 4;
        using CfgR = rfa::DkDvRoleCfg<KD, DH, NWR>;
        auto kern = rfa::k_causal_bwd_dkdv_roles<KD, DH, NWR>;
        if (int rc = set_lds(kern, CfgR::kLds)) return rc;
        RFA_LAUNCH(CAUSAL_BWD_DKDV, kern, dim3(2 * N * p.nseg), dim3(64 * NWR), CfgR::kLds, st, q, k, v, g, dk, dv,
                   (const float*)wsR, (const float*)wsr, den_in, (const float*)gz, T, N, p.nseg, p.seg_len, prefixed,
                   savedHdr, pw);
    } else
    if constexpr (NW == 4 && KD <= 128) {
        // 8 waves with the state phase split by role (dK waves / dV waves): two waves per SIMD
        // (K = 256 would spill at 256 registers per wave)
        using CfgK = rfa::CausalCfg<KD, DH, 8>;
        auto kern = rfa::k_causal_bwd_dkdv<KD, DH, 8, true, true>;
        if (int rc = set_lds(kern, CfgK::kBwdDkLds)) return rc;
        RFA_LAUNCH(CAUSAL_BWD_DKDV, kern, dim3(N * p.nseg), dim3(512), CfgK::kBwdDkLds, st, q, k, v, g,
                           dk, dv, wsR, wsr, den_in, gz, (const uint8_t*)nullptr, 1, T, N, p.nseg, p.seg_len, prefixed,
                           savedHdr, pw);
    } else {
        auto kern = rfa::k_causal_bwd_dkdv<KD, DH, NW, true>;
        if (int rc = set_lds(kern, Cfg::kBwdDkLds)) return rc;
        RFA_LAUNCH(CAUSAL_BWD_DKDV, kern, dim3(N * p.nseg), dim3(64 * NW), Cfg::kBwdDkLds, st, q, k, v, g,
                           dk, dv, wsR, wsr, den_in, gz, (const uint8_t*)nullptr, 1, T, N, p.nseg, p.seg_len, prefixed,
                           savedHdr, pw);
    }
    RFA_HIP_TRY(hipGetLastError());
    return RFA_OK;
}

// backward of a forward that left its final state (LAYOUT_FINAL): one launch, no workspace
template <int KD, int DH>
int launch_sliced_backward(const rfa::half_t* q, const rfa::half_t* k, const rfa::half_t* v, const rfa::half_t* g,
                           const rfa::half_t* out, rfa::half_t* dq, rfa::half_t* dk, rfa::half_t* dv, int T, int N,
                           const ScanPlan& pf, const int* savedHdr, const float* finalS, const float* finalZ,
                           const float* savedDen, hipStream_t st) {
    if constexpr (KD <= 128 && DH <= 128) {
        using Cfg = rfa::SlicedBwdCfg<KD, DH>;
        auto kern = rfa::k_sliced_bwd<KD, DH, rfa::kSliceWidth>;
        if (int rc = set_lds(kern, Cfg::kLds)) return rc;
        // the loader group addresses the 64 rows of a chunk with 32-bit byte offsets
        if ((int64_t)rfa::kChunk * N * (KD > DH ? KD : DH) * 2 >= ((int64_t)1 << 32))
            return fail(RFA_ERR_BAD_SHAPE, "sliced backward: 64 time steps of a tensor span 4 GiB or more (N=%d)", N);
        const int64_t grid = (int64_t)rfa::kXcds * ((N + rfa::kXcds - 1) / rfa::kXcds) * (Cfg::NA + Cfg::NB);
        RFA_LAUNCH(CAUSAL_BWD_SLICED, kern, dim3((unsigned)grid), dim3(Cfg::kThreads), Cfg::kLds, st, q, k, v, g, out,
                   savedDen, finalS, finalZ, dq, dk, dv, T, N, savedHdr, plan_words(T, N, KD, DH, pf));
        RFA_HIP_TRY(hipGetLastError());
        return RFA_OK;
    } else {
        return fail(RFA_ERR_UNSUPPORTED, "no sliced backward for K=%d d=%d", KD, DH);
    }
}

// ---- cross attention launchers ---------------------------------------------------
// time split for kernels whose workgroups do not depend on each other
ScanPlan make_free_plan(int64_t T, int64_t N) {
    ScanPlan p{1, rfa::kChunk, 0, LAYOUT_SEGMENTS};
    if (T <= 0 || N <= 0) return p;
    const int64_t nchunks = (T + rfa::kChunk - 1) / rfa::kChunk;
    int64_t target = 2 * device_cus();      // workgroups to aim for: two per compute unit
    if (tune::get(tune::FREE_WG) >= 1) target = tune::get(tune::FREE_WG);
    int64_t want = (target + N - 1) / N;
    if (want > nchunks) want = nchunks;
    if (want < 1) want = 1;
    const int64_t cps = (nchunks + want - 1) / want;
    p.nseg = (int)((nchunks + cps - 1) / cps);
    p.seg_len = (int)(cps * rfa::kChunk);
    return p;
}

template <int KD, int DH>
int launch_cross_state(const rfa::half_t* k, const rfa::half_t* v, const uint8_t* mask, int H, float* s,
                       float* z, int T, int N, hipStream_t st) {
    constexpr int NW = causal_waves(KD, DH);
    using Cfg = rfa::CausalCfg<KD, DH, NW>;
    const int seg_len = ((T + rfa::kChunk - 1) / rfa::kChunk) * rfa::kChunk;
    if (mask) {
        auto kern = rfa::k_segment_state<KD, DH, NW, false, true>;
        if (int rc = set_lds(kern, Cfg::kSegStateLds)) return rc;
        RFA_LAUNCH(SEG_STATE, kern, dim3(N), dim3(64 * NW), Cfg::kSegStateLds, st, k, v, mask, H, s, z,
                   (float*)nullptr, T, N, 1, 1, seg_len);
    } else {
        auto kern = rfa::k_segment_state<KD, DH, NW, false, false>;
        if (int rc = set_lds(kern, Cfg::kSegStateLds)) return rc;
        RFA_LAUNCH(SEG_STATE, kern, dim3(N), dim3(64 * NW), Cfg::kSegStateLds, st, k, v, mask, H, s, z,
                   (float*)nullptr, T, N, 1, 1, seg_len);
    }
    RFA_HIP_TRY(hipGetLastError());
    return RFA_OK;
}

template <int KD, int DH>
int launch_cross_readout(const rfa::half_t* q, const float* s, const float* z, rfa::half_t* out, int T, int N,
                         hipStream_t st) {
    constexpr int NW = causal_waves(KD, DH);
    using Cfg = rfa::CausalCfg<KD, DH, NW>;
    const ScanPlan p = make_free_plan(T, N);
    auto kern = rfa::k_causal_fwd<KD, DH, NW, false>;
    if (int rc = set_lds(kern, Cfg::kFwdLds)) return rc;
    RFA_LAUNCH(CROSS_READOUT, kern, dim3(N * p.nseg), dim3(64 * NW), Cfg::kFwdLds, st, q,
                       (const rfa::half_t*)nullptr, (const rfa::half_t*)nullptr, out, s, z, (float*)nullptr,
                       (float*)nullptr, (float*)nullptr, T, N, p.nseg, p.seg_len, 0, (int*)nullptr, rfa::PlanWords{});
    RFA_HIP_TRY(hipGetLastError());
    return RFA_OK;
}

template <int KD, int DH>
int launch_cross_readout_bwd(const rfa::half_t* q, const float* s, const float* z, const rfa::half_t* g,
                             rfa::half_t* dq, float* ds, float* dz, int T, int N, hipStream_t st) {
    constexpr int NW = dq_waves(KD, DH);
    using Cfg = rfa::CausalCfg<KD, DH, NW>;
    const int seg_len = ((T + rfa::kChunk - 1) / rfa::kChunk) * rfa::kChunk;
    auto kern = rfa::k_causal_bwd_dq<KD, DH, NW, false>;
    if (int rc = set_lds(kern, Cfg::kBwdDqLds)) return rc;
    RFA_LAUNCH(CROSS_READOUT_BWD, kern, dim3(N), dim3(64 * NW), Cfg::kBwdDqLds, st, q, (const rfa::half_t*)nullptr,
                       (const rfa::half_t*)nullptr, g, dq, s, z, ds, dz, (float*)nullptr, (float*)nullptr, T, N,
                       1, seg_len, 0);
    RFA_HIP_TRY(hipGetLastError());
    return RFA_OK;
}

template <int KD, int DH>
int launch_cross_state_bwd(const rfa::half_t* k, const rfa::half_t* v, const uint8_t* mask, int H,
                           const float* ds, const float* dz, rfa::half_t* dk, rfa::half_t* dv, int T, int N,
                           hipStream_t st) {
    constexpr int NW = causal_waves(KD, DH);    // the 8-wave role split of the causal sweep measured slower here
    using Cfg = rfa::CausalCfg<KD, DH, NW>;
    const ScanPlan p = make_free_plan(T, N);
    auto kern = rfa::k_causal_bwd_dkdv<KD, DH, NW, false>;
    if (int rc = set_lds(kern, Cfg::kBwdDkLds)) return rc;
    RFA_LAUNCH(CROSS_STATE_BWD, kern, dim3(N * p.nseg), dim3(64 * NW), Cfg::kBwdDkLds, st,
                       (const rfa::half_t*)nullptr, k, v, (const rfa::half_t*)nullptr, dk, dv, ds, dz,
                       (const float*)nullptr, (const float*)nullptr, mask, H, T, N, p.nseg, p.seg_len, 0,
                       (const int*)nullptr, rfa::PlanWords{});
    RFA_HIP_TRY(hipGetLastError());
    return RFA_OK;
}


// ---- quadratic form with explicit masks ---------------------------------------------------
template <int KD, int DH>
int launch_masked_fwd(const rfa::half_t* q, const rfa::half_t* k, const rfa::half_t* v, const uint8_t* pad,
                      const uint8_t* amask, rfa::half_t* out, float* rsum, int T, int Tp, int N, int H,
                      hipStream_t st) {
    using Cfg = rfa::MaskedCfg<KD, DH>;
    auto kern = rfa::k_masked_fwd<KD, DH>;
    if (int rc = set_lds(kern, Cfg::kLds)) return rc;
    const int nblk = (T + rfa::kChunk - 1) / rfa::kChunk;
    RFA_LAUNCH(MASKED_FWD, kern, dim3(N * (amask ? (nblk + 1) / 2 : nblk)), dim3(256), Cfg::kLds, st, q, k, v, pad, amask, out, rsum, T, Tp, N, H);
    RFA_HIP_TRY(hipGetLastError());
    return RFA_OK;
}

template <int KD, int DH>
int launch_masked_bwd(const rfa::half_t* q, const rfa::half_t* k, const rfa::half_t* v, const rfa::half_t* g,
                      const rfa::half_t* out, const float* rsum, const uint8_t* pad, const uint8_t* amask,
                      const uint8_t* amask_t, rfa::half_t* dq, rfa::half_t* dk, rfa::half_t* dv,
                      rfa::half_t* ghat, float* gz, int T, int Tp, int N, int H, hipStream_t st) {
    using Cfg = rfa::MaskedCfg<KD, DH>;
    const int nblk = (T + rfa::kChunk - 1) / rfa::kChunk;
    const int64_t rows = (int64_t)T * N;
    const int64_t pieces = rows * (DH / 8);
    RFA_LAUNCH(MASKED_PREP, rfa::k_masked_bwd_prep<DH>, dim3((unsigned)((pieces + 255) / 256)), dim3(256), 0, st, g, out,
               rsum, ghat, gz, rows);
    auto kq = rfa::k_masked_dq<KD, DH>;
    if (int rc = set_lds(kq, Cfg::kLds)) return rc;
    RFA_LAUNCH(MASKED_DQ, kq, dim3(N * (amask ? (nblk + 1) / 2 : nblk)), dim3(256), Cfg::kLds, st, (const rfa::half_t*)ghat, (const float*)gz, k,
               v, pad, amask, dq, T, Tp, N, H);
    auto kk = rfa::k_masked_dkdv<KD, DH>;
    if (int rc = set_lds(kk, Cfg::kLds)) return rc;
    RFA_LAUNCH(MASKED_DKDV, kk, dim3(N * (amask_t ? (nblk + 1) / 2 : nblk)), dim3(256), Cfg::kLds, st, q, k, v, (const rfa::half_t*)ghat,
               (const float*)gz, pad, amask_t, dk, dv, T, Tp, N, H);
    RFA_HIP_TRY(hipGetLastError());
    return RFA_OK;
}

// ---- decode launchers --------------------------------------------------------------
// packed: q, k, v are the three thirds of rows of width 3 * H * DH (the output of one projection
// whose weight stacks the three); otherwise separate contiguous tensors
template <int KD, int DH, bool FUSED>
int launch_decode(const rfa::half_t* q, const rfa::half_t* k, const rfa::half_t* v, const rfa::half_t* w,
                  float scale, int H, const float* s_in, const float* z_in, float* s, float* z, rfa::half_t* out,
                  int64_t steps, int64_t N, bool packed, hipStream_t st) {
    const int64_t B = N / H;
    const int64_t qk_bstride = packed ? (int64_t)3 * H * DH : (int64_t)H * (FUSED ? DH : KD);
    const int64_t v_bstride = packed ? (int64_t)3 * H * DH : (int64_t)H * DH;
    const int64_t qk_step = B * qk_bstride, v_step = B * v_bstride;
    // A step's q, k, v rows sit between its state loads and its state stores (the feature map
    // needs them first).  In a decoder they were written a moment ago; in a multi-step call they
    // are read for the first time, and that memory latency is then on every workgroup's critical
    // path at once (12.4 vs 10 us per step at 1024 heads).  So the rows of the next kTouchSteps
    // steps are streamed through once by a small kernel in front of them.
    constexpr int64_t kTouchSteps = 64;
    for (int64_t t = 0; t < steps; ++t) {
        if (steps > 1 && t % kTouchSteps == 0) {
            const int64_t m = (steps - t < kTouchSteps) ? steps - t : kTouchSteps;
            if (packed)
                RFA_LAUNCH(DECODE_TOUCH, rfa::k_touch_rows, dim3(256), dim3(rfa::kThreads), 0, st,
                           reinterpret_cast<const uint4*>(q + t * qk_step), (const uint4*)nullptr, (const uint4*)nullptr,
                           m * qk_step / 8, (int64_t)0, (int64_t)0);
            else
                RFA_LAUNCH(DECODE_TOUCH, rfa::k_touch_rows, dim3(256), dim3(rfa::kThreads), 0, st,
                           reinterpret_cast<const uint4*>(q + t * qk_step), reinterpret_cast<const uint4*>(k + t * qk_step),
                           reinterpret_cast<const uint4*>(v + t * v_step), m * qk_step / 8, m * qk_step / 8, m * v_step / 8);
        }
        RFA_LAUNCH(DECODE_STEP, (rfa::k_decode_step<KD, DH, FUSED>), dim3((unsigned)N), dim3(rfa::kThreads), 0, st,
                           q + t * qk_step, k + t * qk_step, v + t * v_step, w, scale, H, qk_bstride, v_bstride,
                           t == 0 ? s_in : (const float*)s, t == 0 ? z_in : (const float*)z, s, z, out + t * N * DH);
    }
    RFA_HIP_TRY(hipGetLastError());
    return RFA_OK;
}

// ---- projection launcher -----------------------------------------------------------
template <int D, int DH, int NKS>
int launch_project_rows(const rfa::half_t* x, const rfa::ProjectArgs& pa, const rfa::half_t* wf, int R, int H, int np,
                        float scale, hipStream_t st) {
    // rows of x in registers; split the H * np pairs of a row tile over enough groups to fill the CUs
    using Cfg = rfa::ProjectRowCfg<D, DH, NKS>;
    auto kern = rfa::k_project_phi_rows<D, DH, NKS>;
    if (int rc = set_lds(kern, Cfg::kLds)) return rc;
    const int nrt = (R + Cfg::BM - 1) / Cfg::BM;
    const int pairs = H * np;
    int ngroups = (device_cus() + nrt - 1) / nrt;
    if (ngroups > pairs) ngroups = pairs;
    const int ppg = (pairs + ngroups - 1) / ngroups;
    ngroups = (pairs + ppg - 1) / ppg;
    const int64_t grid = (int64_t)8 * ((nrt + 7) / 8) * ngroups;
    RFA_LAUNCH(PROJECT_PHI, kern, dim3((unsigned)grid), dim3(rfa::kThreads), Cfg::kLds, st, x, pa, wf, R, H, np, ngroups,
               ppg, scale);
    RFA_HIP_TRY(hipGetLastError());
    return RFA_OK;
}

template <int D, int DH>
int launch_project_phi(const rfa::half_t* x, const rfa::ProjectArgs& pa, const rfa::half_t* wf, int R, int E, int H,
                       int np, float scale, hipStream_t st) {
    if constexpr (DH == 64 && D <= 64) {
        if (tune::get(tune::PROJECT_STREAMING) <= 0) {
            if (E == 128) return launch_project_rows<D, DH, 4>(x, pa, wf, R, H, np, scale, st);
            if (E == 256) return launch_project_rows<D, DH, 8>(x, pa, wf, R, H, np, scale, st);
            if (E == 384) return launch_project_rows<D, DH, 12>(x, pa, wf, R, H, np, scale, st);
            if (E == 512) return launch_project_rows<D, DH, 16>(x, pa, wf, R, H, np, scale, st);
        }
    }
    using Cfg = rfa::ProjectCfg<D, DH>;
    auto kern = rfa::k_project_phi<D, DH>;
    if (int rc = set_lds(kern, Cfg::kLds)) return rc;
    const int nrt = (R + Cfg::BM - 1) / Cfg::BM;
    const int64_t grid = (int64_t)8 * ((nrt + 7) / 8) * H * np;
    RFA_LAUNCH(PROJECT_PHI, kern, dim3((unsigned)grid), dim3(rfa::kThreads), Cfg::kLds, st, x, pa, wf, R, E, H, np, scale);
    RFA_HIP_TRY(hipGetLastError());
    return RFA_OK;
}

// ---- weight-gradient plan -------------------------------------------------------------
struct WGradPlan {
    int nsplit;            // row splits (partials to add)
    int rows_per_split;    // multiple of 64
};

// About 256-512 workgroups: 8 splits (one per XCD) times as many as the tile count leaves room for.
WGradPlan make_wgrad_plan(int64_t R, int Eo, int Ei, int np) {
    const int64_t tiles = (int64_t)np * (Eo / 128) * (Ei / 128);
    const int64_t nchunks = (R + 63) / 64;
    int64_t want = 8 * ((32 + tiles - 1) / tiles);
    if (want > 64) want = 64;
    if (want > nchunks) want = nchunks;
    if (want < 1) want = 1;
    const int64_t cps = (nchunks + want - 1) / want;
    WGradPlan p;
    p.rows_per_split = (int)(cps * 64);
    p.nsplit = (int)((nchunks + cps - 1) / cps);
    if (p.nsplit < 1) p.nsplit = 1;
    return p;
}

// ---- feature map launchers ---------------------------------------------------------
int feature_bwd_blocks(int64_t R, int H, int ntens = 1) {
    const int64_t nrb = (R + 63) / 64;
    int64_t target = 512;               // about two workgroups per CU; few partial sums to reduce
    if (tune::get(tune::FEATURE_WG) >= 1) target = tune::get(tune::FEATURE_WG);
    int64_t nblk = (target + (int64_t)H * ntens - 1) / ((int64_t)H * ntens);
    if (nblk > nrb) nblk = nrb;
    if (nblk < 1) nblk = 1;
    return (int)nblk;
}

// Workgroups along x for the streaming feature-map kernels: eight waves each, a wave per group of
// 16 rows, one workgroup per CU in all (their registers leave room for one; a second round of
// workgroups would pay the staging of W' and, in the backward, the sum over the waves again);
// more rows make the waves walk further.  Never more than feature_bwd_blocks, which sizes the
// workspace of the backward's partial sums.
int feature_stream_blocks(int64_t R, int H, int ntens, int waves = rfa::kFeatureWaves) {
    const int64_t ngrp = (R + 15) / 16, full = (ngrp + waves - 1) / waves;
    int64_t target = std::min(device_cus(), 512);
    if (tune::get(tune::FEATURE_WG) >= 1) target = tune::get(tune::FEATURE_WG);
    int64_t nblk = (target + (int64_t)H * ntens - 1) / ((int64_t)H * ntens);
    if (nblk > full) nblk = full;
    if (nblk < 1) nblk = 1;
    return (int)nblk;
}

template <int D, int DH>
int launch_feature_fwd(const rfa::half_t* x, const rfa::half_t* w, rfa::half_t* phi, const rfa::half_t* x1,
                       rfa::half_t* phi1, int R, int H, float scale, hipStream_t st) {
    using Cfg = rfa::FeatureCfg<D, DH>;
    auto kern = rfa::k_feature_map_fwd<D, DH>;
    const int ntens = x1 ? 2 : 1;
    if (int rc = set_lds(kern, Cfg::kFwdLds)) return rc;
    RFA_LAUNCH(FEATURE_FWD, kern, dim3(feature_stream_blocks(R, H, ntens), H, ntens), dim3(rfa::kFeatureThreads), Cfg::kFwdLds,
               st, x, w, phi, x1, phi1, R, H, scale);
    RFA_HIP_TRY(hipGetLastError());
    return RFA_OK;
}

// dx_rs: halves between consecutive rows of dx / dx1 (H * DH for tensors of their own).  copy_src
// [R, H * DH] (or NULL) is copied to rows of copy_dst of the same pitch: the third block of a
// packed gradient, by a third set of workgroups of the same launch where the kernel has that job.
template <int D, int DH>
int launch_feature_bwd(const rfa::half_t* x, const rfa::half_t* w, const rfa::half_t* gphi, rfa::half_t* dx,
                       const rfa::half_t* x1, const rfa::half_t* gphi1, rfa::half_t* dx1,
                       float* dw, float* part, int R, int H, float scale, hipStream_t st,
                       int64_t dx_rs = 0, const rfa::half_t* copy_src = nullptr, rfa::half_t* copy_dst = nullptr) {
    const int ntens = x1 ? 2 : 1;       // two tensors through the same w: one launch, one reduction
    if (dx_rs == 0) dx_rs = (int64_t)H * DH;
    int nblk;
    if constexpr (rfa::FeatureStreamCfg<D, DH>::kFits) {
        using Cfg = rfa::FeatureStreamCfg<D, DH>;
        nblk = feature_stream_blocks(R, H, ntens, rfa::kFeatureBwdWaves);      // never more than feature_bwd_blocks, which sized the workspace
        auto kern = rfa::k_feature_map_bwd_stream<D, DH>;
        if (int rc = set_lds(kern, Cfg::kLds)) return rc;
        const bool copy_job = copy_src && ntens == 2;
        RFA_LAUNCH(FEATURE_BWD, kern, dim3(nblk, H, ntens + (copy_job ? 1 : 0)), dim3(rfa::kFeatureBwdThreads), Cfg::kLds, st,
                   x, w, gphi, dx, x1, gphi1, dx1, part, R, H, scale, dx_rs, copy_src, copy_dst);
        if (copy_job) copy_src = nullptr;
    } else {
        using Cfg = rfa::FeatureCfg<D, DH>;
        nblk = feature_bwd_blocks(R, H, ntens);
        auto kern = rfa::k_feature_map_bwd<D, DH>;
        if (int rc = set_lds(kern, Cfg::kBwdLds)) return rc;
        RFA_LAUNCH(FEATURE_BWD, kern, dim3(nblk, H, ntens), dim3(rfa::kThreads), Cfg::kBwdLds, st, x, w, gphi, dx, x1, gphi1,
                   dx1, part, R, H, scale, dx_rs);
    }
    if (copy_src) {
        const int64_t pieces = (int64_t)R * H * DH / 8;
        const unsigned blocks = (unsigned)std::min<int64_t>((pieces + rfa::kThreads - 1) / rfa::kThreads, 4 * (int64_t)device_cus());
        RFA_LAUNCH(COPY_ROWS, rfa::k_copy_rows_strided, dim3(blocks), dim3(rfa::kThreads), 0, st, copy_src, copy_dst, (int64_t)R,
                   H * DH, dx_rs);
    }
    if (!dw) {                  // dx only: the kernels got no place for partial sums and formed none
        RFA_HIP_TRY(hipGetLastError());
        return RFA_OK;
    }
    const int64_t elems = (int64_t)H * D * DH;
    static_assert((D * DH) % 256 == 0, "dw reduce works on blocks of 256 elements");
    RFA_LAUNCH(FEATURE_DW_REDUCE, rfa::k_feature_map_dw_reduce, dim3((unsigned)(elems / 256)), dim3(rfa::kThreads), 0, st,
                       part, dw, ntens * nblk, elems);
    RFA_HIP_TRY(hipGetLastError());
    return RFA_OK;
}

// zero fill by kernel (safe to record into a HIP graph, unlike a memset node)
__global__ void k_zero_f32(float* p, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0.f;
}

void zero_f32(float* p, int64_t n, hipStream_t st) {
    if (n > 0) RFA_LAUNCH(ZERO_FILL, k_zero_f32, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, p, n);
}

bool feature_shape_supported(int D, int d) { return (D == 32 || D == 64 || D == 128) && (d == 64 || d == 128); }

int check_causal_dims(int64_t T, int64_t N, int K, int d) {
    if (T < 0 || N < 0 || K <= 0 || d <= 0)
        return fail(RFA_ERR_BAD_SHAPE, "bad sizes T=%lld N=%lld K=%d d=%d", (long long)T, (long long)N, K, d);
    if (!rfa_shape_supported(K, d))
        return fail(RFA_ERR_UNSUPPORTED,
                    "no kernel for feature width K=%d, head dim d=%d (supported: K in {64,128,256}, d in {64,128})", K, d);
    if (T > (1 << 30) || N > (1 << 22) || T * N > (int64_t(1) << 31))
        return fail(RFA_ERR_BAD_SHAPE, "T=%lld N=%lld exceed the supported range", (long long)T, (long long)N);
    return RFA_OK;
}

// ---- static device memory --------------------------------------------------
// Memory the library owns without allocating: file-scope device variables, one copy per GPU, held
// until the process ends.  In host code such a name is a stand-in, not a device address: the
// address on the current device comes from hipGetSymbolAddress, once per device.
static __device__ int g_selftest_word;        // result word of rfa_selftest_layout
// workspace of rfa_causal_forward_noalloc: the segment totals of one forward call
constexpr size_t kStaticScratchBytes = (size_t)16 << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;

// address of a static device variable on the current device, looked up once per device
int cached_symbol_address(std::atomic<void*>* cache, hipError_t (*lookup)(void**), void** out) {
    int dev = 0;
    RFA_HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return fail(RFA_ERR_HIP, "device index %d not supported", dev);
    void* p = cache[dev].load(std::memory_order_acquire);
    if (!p) {
        RFA_HIP_TRY(lookup(&p));
        if (!p) return fail(RFA_ERR_HIP, "hipGetSymbolAddress returned a NULL address");
        cache[dev].store(p, std::memory_order_release);
    }
    *out = p;
    return RFA_OK;
}

// this device's copy of `scratch`: host code uses this pointer, never the array's name
int static_scratch_address(unsigned char** out) {
    static std::atomic<void*> cache[kMaxDevices];
    void* ptr = nullptr;
    if (int rc = cached_symbol_address(cache, [](void** q) { return hipGetSymbolAddress(q, HIP_SYMBOL(scratch)); }, &ptr))
        return rc;
    *out = static_cast<unsigned char*>(ptr);
    return RFA_OK;
}

int selftest_word_address(int** out) {
    static std::atomic<void*> cache[kMaxDevices];
    void* p = nullptr;
    if (int rc = cached_symbol_address(cache, [](void** q) { return hipGetSymbolAddress(q, HIP_SYMBOL(g_selftest_word)); }, &p))
        return rc;
    *out = static_cast<int*>(p);
    return RFA_OK;
}

// ---- layout self test ------------------------------------------------------
__global__ void k_selftest(int* bad) {
    using namespace rfa;
    __shared__ __align__(16) half_t A[16 * 40];
    __shared__ __align__(16) half_t B[16 * 40];
    __shared__ __align__(16) half_t X[32 * 24];
    const int lane = threadIdx.x, i = lane & 15, G = lane >> 4;
    for (int e = lane; e < 16 * 32; e += 64) {
        const int r = e / 32, c = e % 32;
        A[r * 40 + c] = (half_t)(float)((r * 7 + c * 3) % 11 - 5);
        B[r * 40 + c] = (half_t)(float)((r * 5 + c * 2) % 13 - 6);
    }
    for (int e = lane; e < 32 * 16; e += 64) X[(e / 16) * 24 + e % 16] = (half_t)(float)e;
    __syncthreads();
    f4 acc = mfma32(row8(A, 40, i, 0, G), row8(B, 40, i, 0, G), f4_zero());
    int nbad = 0;
    for (int e = 0; e < 4; ++e) {
        const int m = 4 * G + e, n = i;
        float want = 0.f;
        for (int r = 0; r < 32; ++r) want += (float)A[m * 40 + r] * (float)B[n * 40 + r];
        if (want != acc[e]) ++nbad;
    }
    h8 cf = col8(X, 24, 0, 0, lane);
    for (int e = 0; e < 8; ++e)
        if ((float)cf[e] != (float)((8 * G + e) * 16 + i)) ++nbad;
    if (nbad) atomicAdd(bad, nbad);
}

// ---- MFMA issue-rate probe ---------------------------------------------------
// Every wave runs `iters` rounds of 8 independent 16x16x32 fp16 MFMA accumulations on
// register operands: no memory traffic, so the time measures the matrix pipes alone.
__global__ __launch_bounds__(256) void k_mfma_rate(int iters, float* sink) {
    using namespace rfa;
    const int lane = threadIdx.x & 63;
    h8 a, b;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        a[e] = (half_t)(float)((lane + e) % 3 - 1);
        b[e] = (half_t)(float)((lane * 3 + e) % 5 - 2);
    }
    f4 acc[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) acc[t] = f4_zero();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int t = 0; t < 8; ++t) acc[t] = mfma32(a, b, acc[t]);
    }
    float s = 0.f;
#pragma unroll
    for (int t = 0; t < 8; ++t) s += acc[t][0] + acc[t][1] + acc[t][2] + acc[t][3];
    if (s == 12345.678f) sink[0] = s;      // keeps the loop alive without a store in practice
}

}  // namespace

extern "C" {

int rfa_version(void) { return 100; }

#ifdef RFA_PHASE_TIMING
// tuning builds only: out[32] receives the accumulated phase cycle counters; reset != 0 clears them
int rfa_debug_phase_ticks(unsigned long long* out, int reset) {
    if (reset) {
        unsigned long long z[32] = {};
        RFA_HIP_TRY(hipMemcpyToSymbol(HIP_SYMBOL(rfa::g_phase_ticks), z, sizeof(z)));
        return RFA_OK;
    }
    RFA_HIP_TRY(hipDeviceSynchronize());
    RFA_HIP_TRY(hipMemcpyFromSymbol(out, HIP_SYMBOL(rfa::g_phase_ticks), 32 * sizeof(unsigned long long)));
    return RFA_OK;
}
#endif

const char* rfa_last_error(void) { return g_err; }

int rfa_shape_supported(int K, int d) {
    return ((K == 64 || K == 128 || K == 256) && (d == 64 || d == 128)) ? 1 : 0;
}

int rfa_causal_num_segments(int64_t T, int64_t N, int K, int d) { return make_plan(T, N, K, d).nseg; }

int rfa_tuning_set(const char* name, int value) {
    const int k = tune::find(name);
    if (k < 0) return fail(RFA_ERR_BAD_SHAPE, "rfa_tuning_set: no knob named '%s'", name ? name : "(null)");
    if (value < -1 || value > (1 << 20)) return fail(RFA_ERR_BAD_SHAPE, "rfa_tuning_set: value %d out of range", value);
    (void)tune::get((tune::Key)k);      // the environment is read before the first store
    tune::value[k].store(value, std::memory_order_relaxed);
    return RFA_OK;
}

int rfa_tuning_get(const char* name, int* value) {
    const int k = tune::find(name);
    if (k < 0 || !value) return fail(RFA_ERR_BAD_SHAPE, "rfa_tuning_get: no knob named '%s'", name ? name : "(null)");
    *value = tune::get((tune::Key)k);
    return RFA_OK;
}

int rfa_selftest_layout(void* stream) {
    hipStream_t st = static_cast<hipStream_t>(stream);
    int* dbad = nullptr;      // a word of the library's static device memory: nothing is allocated
    if (int rc = selftest_word_address(&dbad)) return rc;
    int hbad = 0;
    RFA_HIP_TRY(hipMemcpyAsync(dbad, &hbad, sizeof(int), hipMemcpyHostToDevice, st));
    RFA_LAUNCH(SELFTEST, k_selftest, dim3(1), dim3(64), 0, st, dbad);
    RFA_HIP_TRY(hipMemcpyAsync(&hbad, dbad, sizeof(int), hipMemcpyDeviceToHost, st));
    RFA_HIP_TRY(hipStreamSynchronize(st));
    if (hbad) return fail(RFA_ERR_HIP, "selftest: %d lane values differ from the assumed MFMA / LDS layout", hbad);
    return RFA_OK;
}

int rfa_selftest_mfma_rate(int waves_per_simd, int iters, float* sink, double* flops, void* stream) {
    if (waves_per_simd < 1 || waves_per_simd > 8 || iters < 1 || !sink || !flops)
        return fail(RFA_ERR_BAD_SHAPE, "rfa_selftest_mfma_rate: waves_per_simd in 1..8, iters >= 1, non-NULL sink and flops");
    hipStream_t st = static_cast<hipStream_t>(stream);
    int dev = 0, cus = 0;
    RFA_HIP_TRY(hipGetDevice(&dev));
    RFA_HIP_TRY(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    const int blocks = cus * waves_per_simd;           // 4 waves per workgroup, one per SIMD
    RFA_LAUNCH(SELFTEST, k_mfma_rate, dim3(blocks), dim3(256), 0, st, iters, sink);
    RFA_HIP_TRY(hipGetLastError());
    *flops = (double)blocks * 4 * iters * 8 * (2.0 * 16 * 16 * 32);
    return RFA_OK;
}

size_t rfa_causal_forward_workspace_bytes(int64_t T, int64_t N, int K, int d) {
    if (T <= 0 || N <= 0 || !rfa_shape_supported(K, d)) return 0;
    return layout_workspace(T, N, K, d, make_plan(T, N, K, d), false).total;
}

size_t rfa_causal_backward_workspace_bytes(int64_t T, int64_t N, int K, int d) {
    if (T <= 0 || N <= 0 || !rfa_shape_supported(K, d)) return 0;
    return layout_workspace(T, N, K, d, make_plan(T, N, K, d), true).total;
}

// RFA_ONLY_KD=<K>,<d> (a development build: python -m rfa_amd.build --only K,d): kernels of one
// shape only, every other shape falls through to RFA_ERR_UNSUPPORTED; compiles in a fraction of
// the time.  Never defined in the library the package ships.
#ifdef RFA_ONLY_K
#define RFA_DISPATCH_KD(K, d, CALL) \
    if (K == RFA_ONLY_K && d == RFA_ONLY_D) { return CALL(RFA_ONLY_K, RFA_ONLY_D); }
#else
#define RFA_DISPATCH_KD(K, d, CALL)                                   \
    if (K == 64 && d == 64) { return CALL(64, 64); }                  \
    if (K == 128 && d == 64) { return CALL(128, 64); }                \
    if (K == 256 && d == 64) { return CALL(256, 64); }                \
    if (K == 64 && d == 128) { return CALL(64, 128); }                \
    if (K == 128 && d == 128) { return CALL(128, 128); }              \
    if (K == 256 && d == 128) { return CALL(256, 128); }
#endif

// The saved buffer: a 256-byte header (rfa::PlanWords: the plan of the forward that wrote the
// buffer), then S and z -- the segment totals (S in fragment order) or, with LAYOUT_FINAL, the
// state after the last step ([N][K][d], [N][K]) -- and the raw denominators.
struct SavedLayoutBytes { size_t S, Z, den, total; };

static SavedLayoutBytes saved_layout(int64_t T, int64_t N, int K, int d, const ScanPlan& p) {
    SavedLayoutBytes l{};
    size_t off = kSavedHeaderBytes;
    const size_t states = (size_t)N * (p.layout == LAYOUT_FINAL ? 1 : p.nseg);
    l.S = off; off += align_up(states * K * d * 4);
    l.Z = off; off += align_up(states * K * 4);
    l.den = off; off += align_up((size_t)T * N * 4);
    l.total = off;
    return l;
}

size_t rfa_causal_saved_state_bytes(int64_t T, int64_t N, int K, int d) {
    if (T <= 0 || N <= 0 || !rfa_shape_supported(K, d)) return 0;
    return saved_layout(T, N, K, d, make_plan(T, N, K, d)).total;
}

// The plan a backward call on `saved` runs with: the one recorded when a forward call of this
// process last wrote a buffer at that address, if that forward had this call's shape; else the
// current one.  Either way the kernels check the plan against the header in the buffer itself.
static int saved_plan(const void* saved, int64_t T, int64_t N, int K, int d, ScanPlan* p) {
    rfa::PlanWords w;
    if (saved && registry::get(saved, &w)) {
        const ScanPlan rec{w.w[5], w.w[6], w.w[7], w.w[2]};
        const rfa::PlanWords same = plan_words(T, N, K, d, rec);
        if (memcmp(&w, &same, sizeof(w)) == 0) {
            *p = rec;
            return RFA_OK;
        }
        registry::drop(saved);      // the address now holds something else
    }
    *p = make_plan(T, N, K, d);
    return RFA_OK;
}

size_t rfa_causal_backward_saved_workspace_bytes(const void* saved, int64_t T, int64_t N, int K, int d) {
    if (T <= 0 || N <= 0 || !rfa_shape_supported(K, d)) return 0;
    ScanPlan p;
    if (saved_plan(saved, T, N, K, d, &p) != RFA_OK) return 0;
    if (p.layout == LAYOUT_FINAL) return 0;
    return layout_workspace(T, N, K, d, p, true).total;
}

int rfa_causal_saved_describe(const void* saved, int32_t* words16, void* stream) {
    if (!saved || !words16) return fail(RFA_ERR_NULL_POINTER, "rfa_causal_saved_describe: NULL pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    RFA_HIP_TRY(hipMemcpyAsync(words16, saved, 16 * sizeof(int32_t), hipMemcpyDeviceToHost, st));
    RFA_HIP_TRY(hipStreamSynchronize(st));
    return RFA_OK;
}

static int causal_forward_impl(const void* q, const void* k, const void* v, void* out, int64_t T, int64_t N,
                               int K, int d, void* saved, size_t saved_bytes, bool want_saved, float* final_s,
                               float* final_z, void* workspace, size_t workspace_bytes, void* stream,
                               bool allow_recompute = true);

int rfa_causal_forward(const void* q, const void* k, const void* v, void* out, int64_t T, int64_t N,
                       int K, int d, void* workspace, size_t workspace_bytes, void* stream) {
    return causal_forward_impl(q, k, v, out, T, N, K, d, nullptr, 0, false, nullptr, nullptr, workspace,
                               workspace_bytes, stream);
}

size_t rfa_static_scratch_bytes(void) { return kStaticScratchBytes; }

int rfa_causal_forward_noalloc(const void* q, const void* k, const void* v, void* out, int64_t T, int64_t N,
                               int K, int d, void* stream) {
    if (int rc = check_causal_dims(T, N, K, d)) return rc;
    if (T == 0 || N == 0) return RFA_OK;
    const size_t need = rfa_causal_forward_workspace_bytes(T, N, K, d);
    if (need > kStaticScratchBytes)
        return fail(RFA_ERR_WORKSPACE,
                    "rfa_causal_forward_noalloc: this shape needs %zu bytes of segment totals, the static scratch "
                    "holds %zu; use rfa_causal_forward with a caller-owned workspace", need, kStaticScratchBytes);
    unsigned char* ptr = nullptr;       // this device's copy of the static array
    if (int rc = static_scratch_address(&ptr)) return rc;
    // every slot of the segment totals that the scan reads is written by the totals pass of the same
    // call first, so what an earlier call left in the array does not matter.  (This entry point
    // always takes the form with segment totals: the array is what it exists for.)
    return causal_forward_impl(q, k, v, out, T, N, K, d, nullptr, 0, false, nullptr, nullptr, ptr, kStaticScratchBytes,
                               stream, false);
}

int rfa_causal_prefill(const void* q, const void* k, const void* v, void* out, float* s, float* z, int64_t T,
                       int64_t N, int K, int d, void* workspace, size_t workspace_bytes, void* stream) {
    if (int rc = check_causal_dims(T, N, K, d)) return rc;
    if (N == 0) return RFA_OK;
    if (!s || !z) return fail(RFA_ERR_NULL_POINTER, "rfa_causal_prefill: NULL state pointer");
    if (!aligned16(s) || !aligned16(z)) return fail(RFA_ERR_ALIGNMENT, "rfa_causal_prefill: state must be 16-byte aligned");
    if (T == 0) {   // empty prompt: the state is zero
        hipStream_t st = static_cast<hipStream_t>(stream);
        zero_f32(s, (int64_t)N * K * d, st);
        zero_f32(z, (int64_t)N * K, st);
        return RFA_OK;
    }
    return causal_forward_impl(q, k, v, out, T, N, K, d, nullptr, 0, false, s, z, workspace, workspace_bytes, stream);
}

int rfa_causal_forward_save(const void* q, const void* k, const void* v, void* out, void* saved,
                            size_t saved_bytes, int64_t T, int64_t N, int K, int d, void* workspace,
                            size_t workspace_bytes, void* stream) {
    return causal_forward_impl(q, k, v, out, T, N, K, d, saved, saved_bytes, true, nullptr, nullptr, workspace,
                               workspace_bytes, stream);
}

static int causal_forward_impl(const void* q, const void* k, const void* v, void* out, int64_t T, int64_t N,
                               int K, int d, void* saved, size_t saved_bytes, bool want_saved, float* final_s,
                               float* final_z, void* workspace, size_t workspace_bytes, void* stream,
                               bool allow_recompute) {
    if (int rc = check_causal_dims(T, N, K, d)) return rc;
    if (T == 0 || N == 0) return RFA_OK;
    const ScanPlan p = make_plan(T, N, K, d);
    int* savedHdr = nullptr;
    float* savedS = nullptr;
    float* savedZ = nullptr;
    float* savedDen = nullptr;
    if (want_saved) {
        const SavedLayoutBytes sl = saved_layout(T, N, K, d, p);
        if (!saved || saved_bytes < sl.total || !aligned16(saved))
            return fail(RFA_ERR_WORKSPACE, "rfa_causal_forward_save: saved-state buffer of %zu bytes required, got %zu",
                        sl.total, saved ? saved_bytes : (size_t)0);
        char* sb = static_cast<char*>(saved);
        savedHdr = reinterpret_cast<int*>(sb);
        savedS = reinterpret_cast<float*>(sb + sl.S);
        savedZ = reinterpret_cast<float*>(sb + sl.Z);
        savedDen = reinterpret_cast<float*>(sb + sl.den);
    }
    if (!q || !k || !v || !out) return fail(RFA_ERR_NULL_POINTER, "rfa_causal_forward: NULL tensor pointer");
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(out))
        return fail(RFA_ERR_ALIGNMENT, "rfa_causal_forward: tensors must be 16-byte aligned");
    const Workspace wl = layout_workspace(T, N, K, d, p, false);
    if (want_saved && p.layout == LAYOUT_FINAL) {
        // the buffer gets the state after the last step; the segment totals stay in the workspace
        final_s = savedS;
        final_z = savedZ;
        savedS = nullptr;
        savedZ = nullptr;
    }
    // with the segment totals in the saved buffer the workspace is not touched
    if (!savedS && wl.total > 0 && (!workspace || workspace_bytes < wl.total || !aligned16(workspace)))
        return fail(RFA_ERR_WORKSPACE, "rfa_causal_forward: workspace of %zu bytes required, got %zu", wl.total,
                    workspace ? workspace_bytes : (size_t)0);
    hipStream_t st = static_cast<hipStream_t>(stream);
    auto* qh = static_cast<const rfa::half_t*>(q);
    auto* kh = static_cast<const rfa::half_t*>(k);
    auto* vh = static_cast<const rfa::half_t*>(v);
    auto* oh = static_cast<rfa::half_t*>(out);
    char* ws = static_cast<char*>(workspace);
    if (want_saved) registry::put(saved, plan_words(T, N, K, d, p));
#define RFA_CALL_FWD(KD, DH) launch_forward<KD, DH>(qh, kh, vh, oh, (int)T, (int)N, p, ws, wl, savedHdr, savedS, savedZ, savedDen, final_s, final_z, allow_recompute, st)
    RFA_DISPATCH_KD(K, d, RFA_CALL_FWD)
#undef RFA_CALL_FWD
    return fail(RFA_ERR_UNSUPPORTED, "unreachable");
}

static int causal_backward_impl(const void* q, const void* k, const void* v, const void* grad_attn,
                                const void* out, void* dq, void* dk, void* dv, int64_t T, int64_t N, int K, int d,
                                const void* saved, size_t saved_bytes, bool have_saved, void* workspace,
                                size_t workspace_bytes, void* stream);

int rfa_causal_backward(const void* q, const void* k, const void* v, const void* grad_attn, void* dq,
                        void* dk, void* dv, int64_t T, int64_t N, int K, int d, void* workspace,
                        size_t workspace_bytes, void* stream) {
    return causal_backward_impl(q, k, v, grad_attn, nullptr, dq, dk, dv, T, N, K, d, nullptr, 0, false, workspace,
                                workspace_bytes, stream);
}

int rfa_causal_backward_saved(const void* q, const void* k, const void* v, const void* grad_attn,
                              const void* out, const void* saved, size_t saved_bytes, void* dq, void* dk,
                              void* dv, int64_t T, int64_t N, int K, int d, void* workspace,
                              size_t workspace_bytes, void* stream) {
    if (T > 0 && N > 0) {
        if (!out) return fail(RFA_ERR_NULL_POINTER, "rfa_causal_backward_saved: NULL forward output");
        if (!aligned16(out)) return fail(RFA_ERR_ALIGNMENT, "rfa_causal_backward_saved: out must be 16-byte aligned");
    }
    return causal_backward_impl(q, k, v, grad_attn, out, dq, dk, dv, T, N, K, d, saved, saved_bytes, true, workspace,
                                workspace_bytes, stream);
}

static int causal_backward_impl(const void* q, const void* k, const void* v, const void* grad_attn,
                                const void* out, void* dq, void* dk, void* dv, int64_t T, int64_t N, int K, int d,
                                const void* saved, size_t saved_bytes, bool have_saved, void* workspace,
                                size_t workspace_bytes, void* stream) {
    if (int rc = check_causal_dims(T, N, K, d)) return rc;
    if (T == 0 || N == 0) return RFA_OK;
    ScanPlan p = make_plan(T, N, K, d);
    const int* savedHdr = nullptr;
    const float* savedS = nullptr;
    const float* savedZ = nullptr;
    const float* savedDen = nullptr;
    if (have_saved) {
        if (!saved || !aligned16(saved))
            return fail(RFA_ERR_WORKSPACE, "rfa_causal_backward_saved: NULL or misaligned saved-state buffer");
        if (int rc = saved_plan(saved, T, N, K, d, &p)) return rc;
        const SavedLayoutBytes sl = saved_layout(T, N, K, d, p);
        if (saved_bytes < sl.total)
            return fail(RFA_ERR_WORKSPACE, "rfa_causal_backward_saved: saved-state buffer of %zu bytes required, got %zu",
                        sl.total, saved_bytes);
        const char* sb = static_cast<const char*>(saved);
        savedHdr = reinterpret_cast<const int*>(sb);
        savedS = reinterpret_cast<const float*>(sb + sl.S);
        savedZ = reinterpret_cast<const float*>(sb + sl.Z);
        savedDen = reinterpret_cast<const float*>(sb + sl.den);
    }
    if (!q || !k || !v || !grad_attn || !dq || !dk || !dv)
        return fail(RFA_ERR_NULL_POINTER, "rfa_causal_backward: NULL tensor pointer");
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(grad_attn) || !aligned16(dq) ||
        !aligned16(dk) || !aligned16(dv))
        return fail(RFA_ERR_ALIGNMENT, "rfa_causal_backward: tensors must be 16-byte aligned");
    const bool sliced = have_saved && p.layout == LAYOUT_FINAL;
    const Workspace wl = layout_workspace(T, N, K, d, p, true);
    if (!sliced && (!workspace || workspace_bytes < wl.total || !aligned16(workspace)))
        return fail(RFA_ERR_WORKSPACE, "rfa_causal_backward: workspace of %zu bytes required, got %zu", wl.total,
                    workspace ? workspace_bytes : (size_t)0);
    hipStream_t st = static_cast<hipStream_t>(stream);
    auto* qh = static_cast<const rfa::half_t*>(q);
    auto* kh = static_cast<const rfa::half_t*>(k);
    auto* vh = static_cast<const rfa::half_t*>(v);
    auto* gh = static_cast<const rfa::half_t*>(grad_attn);
    auto* outh = static_cast<const rfa::half_t*>(out);
    auto* dqh = static_cast<rfa::half_t*>(dq);
    auto* dkh = static_cast<rfa::half_t*>(dk);
    auto* dvh = static_cast<rfa::half_t*>(dv);
    char* ws = static_cast<char*>(workspace);
    if (sliced) {
#define RFA_CALL_SL(KD, DH) launch_sliced_backward<KD, DH>(qh, kh, vh, gh, outh, dqh, dkh, dvh, (int)T, (int)N, p, savedHdr, savedS, savedZ, savedDen, st)
        RFA_DISPATCH_KD(K, d, RFA_CALL_SL)
#undef RFA_CALL_SL
    }
#define RFA_CALL_BWD(KD, DH) launch_backward<KD, DH>(qh, kh, vh, gh, outh, dqh, dkh, dvh, (int)T, (int)N, p, ws, wl, savedHdr, savedS, savedZ, savedDen, st)
    RFA_DISPATCH_KD(K, d, RFA_CALL_BWD)
#undef RFA_CALL_BWD
    return fail(RFA_ERR_UNSUPPORTED, "unreachable");
}

// ---- cross attention ---------------------------------------------------------------
static int check_cross_dims(const char* fn, int64_t L, int64_t B, int H, int K, int d) {
    if (L < 0 || B < 0 || H <= 0 || K <= 0 || d <= 0)
        return fail(RFA_ERR_BAD_SHAPE, "%s: bad sizes len=%lld B=%lld H=%d K=%d d=%d", fn, (long long)L, (long long)B, H, K, d);
    if (!rfa_shape_supported(K, d))
        return fail(RFA_ERR_UNSUPPORTED, "%s: no kernel for feature width K=%d, head dim d=%d", fn, K, d);
    if (L > (1 << 30) || B * H > (1 << 22) || L * B * H > (int64_t(1) << 31))
        return fail(RFA_ERR_BAD_SHAPE, "%s: sizes exceed the supported range", fn);
    return RFA_OK;
}

int rfa_cross_state(const void* phi_k, const void* v, const uint8_t* key_padding_mask, float* s, float* z,
                    int64_t S_len, int64_t B, int H, int K, int d, void* stream) {
    if (int rc = check_cross_dims("rfa_cross_state", S_len, B, H, K, d)) return rc;
    const int64_t N = B * H;
    if (N == 0) return RFA_OK;
    if (!s || !z) return fail(RFA_ERR_NULL_POINTER, "rfa_cross_state: NULL state pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (S_len == 0) {   // empty source: the state is zero
        zero_f32(s, (int64_t)N * K * d, st);
        zero_f32(z, (int64_t)N * K, st);
        return RFA_OK;
    }
    if (!phi_k || !v) return fail(RFA_ERR_NULL_POINTER, "rfa_cross_state: NULL tensor pointer");
    if (!aligned16(phi_k) || !aligned16(v) || !aligned16(s) || !aligned16(z))
        return fail(RFA_ERR_ALIGNMENT, "rfa_cross_state: tensors must be 16-byte aligned");
    auto* kh = static_cast<const rfa::half_t*>(phi_k);
    auto* vh = static_cast<const rfa::half_t*>(v);
#define RFA_CALL(KD, DH) launch_cross_state<KD, DH>(kh, vh, key_padding_mask, H, s, z, (int)S_len, (int)N, st)
    RFA_DISPATCH_KD(K, d, RFA_CALL)
#undef RFA_CALL
    return fail(RFA_ERR_UNSUPPORTED, "unreachable");
}

int rfa_cross_readout(const void* phi_q, const float* s, const float* z, void* out, int64_t T, int64_t N,
                      int K, int d, void* stream) {
    if (int rc = check_cross_dims("rfa_cross_readout", T, N, 1, K, d)) return rc;
    if (T == 0 || N == 0) return RFA_OK;
    if (!phi_q || !s || !z || !out) return fail(RFA_ERR_NULL_POINTER, "rfa_cross_readout: NULL tensor pointer");
    if (!aligned16(phi_q) || !aligned16(s) || !aligned16(z) || !aligned16(out))
        return fail(RFA_ERR_ALIGNMENT, "rfa_cross_readout: tensors must be 16-byte aligned");
    hipStream_t st = static_cast<hipStream_t>(stream);
    auto* qh = static_cast<const rfa::half_t*>(phi_q);
    auto* oh = static_cast<rfa::half_t*>(out);
#define RFA_CALL(KD, DH) launch_cross_readout<KD, DH>(qh, s, z, oh, (int)T, (int)N, st)
    RFA_DISPATCH_KD(K, d, RFA_CALL)
#undef RFA_CALL
    return fail(RFA_ERR_UNSUPPORTED, "unreachable");
}

int rfa_cross_readout_backward(const void* phi_q, const float* s, const float* z, const void* grad_attn,
                               void* dphi_q, float* ds, float* dz, int64_t T, int64_t N, int K, int d,
                               void* stream) {
    if (int rc = check_cross_dims("rfa_cross_readout_backward", T, N, 1, K, d)) return rc;
    if (N == 0) return RFA_OK;
    if (!ds || !dz) return fail(RFA_ERR_NULL_POINTER, "rfa_cross_readout_backward: NULL gradient pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (T == 0) {
        zero_f32(ds, (int64_t)N * K * d, st);
        zero_f32(dz, (int64_t)N * K, st);
        return RFA_OK;
    }
    if (!phi_q || !s || !z || !grad_attn || !dphi_q)
        return fail(RFA_ERR_NULL_POINTER, "rfa_cross_readout_backward: NULL tensor pointer");
    if (!aligned16(phi_q) || !aligned16(s) || !aligned16(z) || !aligned16(grad_attn) || !aligned16(dphi_q) ||
        !aligned16(ds) || !aligned16(dz))
        return fail(RFA_ERR_ALIGNMENT, "rfa_cross_readout_backward: tensors must be 16-byte aligned");
    auto* qh = static_cast<const rfa::half_t*>(phi_q);
    auto* gh = static_cast<const rfa::half_t*>(grad_attn);
    auto* dqh = static_cast<rfa::half_t*>(dphi_q);
#define RFA_CALL(KD, DH) launch_cross_readout_bwd<KD, DH>(qh, s, z, gh, dqh, ds, dz, (int)T, (int)N, st)
    RFA_DISPATCH_KD(K, d, RFA_CALL)
#undef RFA_CALL
    return fail(RFA_ERR_UNSUPPORTED, "unreachable");
}

int rfa_cross_state_backward(const void* phi_k, const void* v, const uint8_t* key_padding_mask, const float* ds,
                             const float* dz, void* dphi_k, void* dv, int64_t S_len, int64_t B, int H, int K,
                             int d, void* stream) {
    if (int rc = check_cross_dims("rfa_cross_state_backward", S_len, B, H, K, d)) return rc;
    const int64_t N = B * H;
    if (S_len == 0 || N == 0) return RFA_OK;
    if (!phi_k || !v || !ds || !dz || !dphi_k || !dv)
        return fail(RFA_ERR_NULL_POINTER, "rfa_cross_state_backward: NULL tensor pointer");
    if (!aligned16(phi_k) || !aligned16(v) || !aligned16(ds) || !aligned16(dz) || !aligned16(dphi_k) || !aligned16(dv))
        return fail(RFA_ERR_ALIGNMENT, "rfa_cross_state_backward: tensors must be 16-byte aligned");
    hipStream_t st = static_cast<hipStream_t>(stream);
    auto* kh = static_cast<const rfa::half_t*>(phi_k);
    auto* vh = static_cast<const rfa::half_t*>(v);
    auto* dkh = static_cast<rfa::half_t*>(dphi_k);
    auto* dvh = static_cast<rfa::half_t*>(dv);
#define RFA_CALL(KD, DH) launch_cross_state_bwd<KD, DH>(kh, vh, key_padding_mask, H, ds, dz, dkh, dvh, (int)S_len, (int)N, st)
    RFA_DISPATCH_KD(K, d, RFA_CALL)
#undef RFA_CALL
    return fail(RFA_ERR_UNSUPPORTED, "unreachable");
}


// ---- quadratic form with explicit masks ---------------------------------------------------
static int check_masked(const char* fn, int64_t T, int64_t Tp, int64_t B, int H, int K, int d, const void* amask) {
    if (int rc = check_cross_dims(fn, T, B, H, K, d)) return rc;
    if (T > (int64_t)64 * rfa::kMaxMaskBlocks)
        return fail(RFA_ERR_UNSUPPORTED, "%s: at most %d steps in the quadratic form (got %lld)", fn, 64 * rfa::kMaxMaskBlocks,
                    (long long)T);
    if (amask && (Tp < T || Tp % 64 != 0))
        return fail(RFA_ERR_BAD_SHAPE, "%s: the attn_mask row stride must be T rounded up to a multiple of 64 (got %lld for T=%lld)",
                    fn, (long long)Tp, (long long)T);
    return RFA_OK;
}

int rfa_masked_forward(const void* phi_q, const void* phi_k, const void* v, const uint8_t* key_padding_mask,
                       const uint8_t* attn_mask, void* out, float* rsum, int64_t T, int64_t Tp, int64_t B, int H,
                       int K, int d, void* stream) {
    if (int rc = check_masked("rfa_masked_forward", T, Tp, B, H, K, d, attn_mask)) return rc;
    const int64_t N = B * H;
    if (T == 0 || N == 0) return RFA_OK;
    if (!phi_q || !phi_k || !v || !out) return fail(RFA_ERR_NULL_POINTER, "rfa_masked_forward: NULL tensor pointer");
    if (!aligned16(phi_q) || !aligned16(phi_k) || !aligned16(v) || !aligned16(out) || (attn_mask && !aligned16(attn_mask)))
        return fail(RFA_ERR_ALIGNMENT, "rfa_masked_forward: tensors must be 16-byte aligned");
    hipStream_t st = static_cast<hipStream_t>(stream);
    auto* qh = static_cast<const rfa::half_t*>(phi_q);
    auto* kh = static_cast<const rfa::half_t*>(phi_k);
    auto* vh = static_cast<const rfa::half_t*>(v);
    auto* oh = static_cast<rfa::half_t*>(out);
#define RFA_CALL(KD, DH) launch_masked_fwd<KD, DH>(qh, kh, vh, key_padding_mask, attn_mask, oh, rsum, (int)T, (int)Tp, (int)N, H, st)
    RFA_DISPATCH_KD(K, d, RFA_CALL)
#undef RFA_CALL
    return fail(RFA_ERR_UNSUPPORTED, "unreachable");
}

size_t rfa_masked_backward_workspace_bytes(int64_t T, int64_t N, int d) {
    if (T <= 0 || N <= 0 || d <= 0) return 0;
    return align_up((size_t)T * N * d * 2) + align_up((size_t)T * N * 4);
}

int rfa_masked_backward(const void* phi_q, const void* phi_k, const void* v, const void* grad_attn, const void* out,
                        const float* rsum, const uint8_t* key_padding_mask, const uint8_t* attn_mask,
                        const uint8_t* attn_mask_t, void* dphi_q, void* dphi_k, void* dv, int64_t T, int64_t Tp,
                        int64_t B, int H, int K, int d, void* workspace, size_t workspace_bytes, void* stream) {
    if (int rc = check_masked("rfa_masked_backward", T, Tp, B, H, K, d, attn_mask)) return rc;
    const int64_t N = B * H;
    if (T == 0 || N == 0) return RFA_OK;
    if (!phi_q || !phi_k || !v || !grad_attn || !out || !rsum || !dphi_q || !dphi_k || !dv)
        return fail(RFA_ERR_NULL_POINTER, "rfa_masked_backward: NULL tensor pointer");
    if ((attn_mask == nullptr) != (attn_mask_t == nullptr))
        return fail(RFA_ERR_NULL_POINTER, "rfa_masked_backward: attn_mask and its transpose must be given together");
    if (!aligned16(phi_q) || !aligned16(phi_k) || !aligned16(v) || !aligned16(grad_attn) || !aligned16(out) ||
        !aligned16(dphi_q) || !aligned16(dphi_k) || !aligned16(dv) || (attn_mask && (!aligned16(attn_mask) || !aligned16(attn_mask_t))))
        return fail(RFA_ERR_ALIGNMENT, "rfa_masked_backward: tensors must be 16-byte aligned");
    const size_t need = rfa_masked_backward_workspace_bytes(T, N, d);
    if (!workspace || workspace_bytes < need || !aligned16(workspace))
        return fail(RFA_ERR_WORKSPACE, "rfa_masked_backward: workspace of %zu bytes required, got %zu", need,
                    workspace ? workspace_bytes : (size_t)0);
    hipStream_t st = static_cast<hipStream_t>(stream);
    auto* qh = static_cast<const rfa::half_t*>(phi_q);
    auto* kh = static_cast<const rfa::half_t*>(phi_k);
    auto* vh = static_cast<const rfa::half_t*>(v);
    auto* gh = static_cast<const rfa::half_t*>(grad_attn);
    auto* oh = static_cast<const rfa::half_t*>(out);
    auto* dqh = static_cast<rfa::half_t*>(dphi_q);
    auto* dkh = static_cast<rfa::half_t*>(dphi_k);
    auto* dvh = static_cast<rfa::half_t*>(dv);
    auto* ghat = static_cast<rfa::half_t*>(workspace);
    float* gz = reinterpret_cast<float*>(static_cast<char*>(workspace) + align_up((size_t)T * N * d * 2));
#define RFA_CALL(KD, DH) launch_masked_bwd<KD, DH>(qh, kh, vh, gh, oh, rsum, key_padding_mask, attn_mask, attn_mask_t, dqh, dkh, dvh, ghat, gz, (int)T, (int)Tp, (int)N, H, st)
    RFA_DISPATCH_KD(K, d, RFA_CALL)
#undef RFA_CALL
    return fail(RFA_ERR_UNSUPPORTED, "unreachable");
}

// ---- incremental decoding -----------------------------------------------------------
static int incremental_impl(const char* fn, const void* phi_q, const void* phi_k, const void* v, const float* s_in,
                            const float* z_in, float* s, float* z, void* out, int64_t steps, int64_t N, int K, int d,
                            void* stream) {
    if (int rc = check_cross_dims(fn, steps, N, 1, K, d)) return rc;
    if (steps == 0 || N == 0) return RFA_OK;
    if (!phi_q || !phi_k || !v || !s_in || !z_in || !s || !z || !out) return fail(RFA_ERR_NULL_POINTER, "%s: NULL tensor pointer", fn);
    if (!aligned16(phi_q) || !aligned16(phi_k) || !aligned16(v) || !aligned16(s_in) || !aligned16(z_in) || !aligned16(s) ||
        !aligned16(z) || !aligned16(out))
        return fail(RFA_ERR_ALIGNMENT, "%s: tensors must be 16-byte aligned", fn);
    hipStream_t st = static_cast<hipStream_t>(stream);
    auto* qh = static_cast<const rfa::half_t*>(phi_q);
    auto* kh = static_cast<const rfa::half_t*>(phi_k);
    auto* vh = static_cast<const rfa::half_t*>(v);
    auto* oh = static_cast<rfa::half_t*>(out);
#define RFA_CALL(KD, DH) launch_decode<KD, DH, false>(qh, kh, vh, nullptr, 0.f, 1, s_in, z_in, s, z, oh, steps, N, false, st)
    RFA_DISPATCH_KD(K, d, RFA_CALL)
#undef RFA_CALL
    return fail(RFA_ERR_UNSUPPORTED, "unreachable");
}

int rfa_incremental(const void* phi_q, const void* phi_k, const void* v, float* s, float* z, void* out,
                    int64_t steps, int64_t N, int K, int d, void* stream) {
    return incremental_impl("rfa_incremental", phi_q, phi_k, v, s, z, s, z, out, steps, N, K, d, stream);
}

int rfa_incremental_out(const void* phi_q, const void* phi_k, const void* v, const float* s_in, const float* z_in,
                        float* s_out, float* z_out, void* out, int64_t steps, int64_t N, int K, int d, void* stream) {
    return incremental_impl("rfa_incremental_out", phi_q, phi_k, v, s_in, z_in, s_out, z_out, out, steps, N, K, d, stream);
}

static int incremental_fused_impl(const char* fn, const void* q, const void* k, const void* v, const void* w, float scale,
                                  const float* s_in, const float* z_in, float* s, float* z, void* out, int64_t steps,
                                  int64_t B, int H, int D, int d, void* stream, bool packed = false) {
    if (int rc = check_cross_dims(fn, steps, B, H, 2 * D, d)) return rc;
    const int64_t N = B * H;
    if (steps == 0 || N == 0) return RFA_OK;
    if (!q || !k || !v || !w || !s_in || !z_in || !s || !z || !out) return fail(RFA_ERR_NULL_POINTER, "%s: NULL tensor pointer", fn);
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(w) || !aligned16(s_in) || !aligned16(z_in) ||
        !aligned16(s) || !aligned16(z) || !aligned16(out))
        return fail(RFA_ERR_ALIGNMENT, "%s: tensors must be 16-byte aligned", fn);
    hipStream_t st = static_cast<hipStream_t>(stream);
    auto* qh = static_cast<const rfa::half_t*>(q);
    auto* kh = static_cast<const rfa::half_t*>(k);
    auto* vh = static_cast<const rfa::half_t*>(v);
    auto* wh = static_cast<const rfa::half_t*>(w);
    auto* oh = static_cast<rfa::half_t*>(out);
    const int K = 2 * D;
#define RFA_CALL(KD, DH) launch_decode<KD, DH, true>(qh, kh, vh, wh, scale, H, s_in, z_in, s, z, oh, steps, N, packed, st)
    RFA_DISPATCH_KD(K, d, RFA_CALL)
#undef RFA_CALL
    return fail(RFA_ERR_UNSUPPORTED, "unreachable");
}

int rfa_incremental_fused(const void* q, const void* k, const void* v, const void* w, float scale, float* s,
                          float* z, void* out, int64_t steps, int64_t B, int H, int D, int d, void* stream) {
    return incremental_fused_impl("rfa_incremental_fused", q, k, v, w, scale, s, z, s, z, out, steps, B, H, D, d, stream);
}

int rfa_incremental_fused_out(const void* q, const void* k, const void* v, const void* w, float scale,
                              const float* s_in, const float* z_in, float* s_out, float* z_out, void* out,
                              int64_t steps, int64_t B, int H, int D, int d, void* stream) {
    return incremental_fused_impl("rfa_incremental_fused_out", q, k, v, w, scale, s_in, z_in, s_out, z_out, out, steps,
                                  B, H, D, d, stream);
}

int rfa_incremental_qkv(const void* qkv, const void* w, float scale, const float* s_in, const float* z_in,
                        float* s_out, float* z_out, void* out, int64_t steps, int64_t B, int H, int D, int d,
                        void* stream) {
    if (H <= 0 || d <= 0) return fail(RFA_ERR_BAD_SHAPE, "rfa_incremental_qkv: bad sizes H=%d d=%d", H, d);
    const rfa::half_t* base = static_cast<const rfa::half_t*>(qkv);
    const int64_t E = (int64_t)H * d;
    return incremental_fused_impl("rfa_incremental_qkv", base, base ? base + E : nullptr, base ? base + 2 * E : nullptr, w,
                                  scale, s_in, z_in, s_out, z_out, out, steps, B, H, D, d, stream, true);
}

// ---- random matrices ----------------------------------------------------------------
static int check_matrix_dims(const char* fn, int H, int D, int d, float tau) {
    if (H < 0 || D <= 0 || d <= 0 || H > (1 << 20) || D > (1 << 14) || d > (1 << 14))
        return fail(RFA_ERR_BAD_SHAPE, "%s: bad sizes H=%d D=%d d=%d", fn, H, D, d);
    if (!(tau != 0.f)) return fail(RFA_ERR_BAD_SHAPE, "%s: tau must be non-zero", fn);
    return RFA_OK;
}

int rfa_build_random_matrices(const void* w, const void* sigma, float tau, void* out, int H, int D, int d,
                              void* stream) {
    if (int rc = check_matrix_dims("rfa_build_random_matrices", H, D, d, tau)) return rc;
    if (H == 0) return RFA_OK;
    if (!w || !out) return fail(RFA_ERR_NULL_POINTER, "rfa_build_random_matrices: NULL tensor pointer");
    const int64_t total = (int64_t)H * D * d;
    RFA_LAUNCH(BUILD_W, rfa::k_build_random_matrices, dim3((unsigned)((total + rfa::kThreads - 1) / rfa::kThreads)),
               dim3(rfa::kThreads), 0, static_cast<hipStream_t>(stream), static_cast<const rfa::half_t*>(w),
               static_cast<const rfa::half_t*>(sigma), static_cast<rfa::half_t*>(out), tau, D, d, total);
    RFA_HIP_TRY(hipGetLastError());
    return RFA_OK;
}

int rfa_build_random_matrices_backward(const void* w, const void* sigma, const void* grad_out, float tau,
                                       void* dsigma, void* dw, int H, int D, int d, void* stream) {
    if (int rc = check_matrix_dims("rfa_build_random_matrices_backward", H, D, d, tau)) return rc;
    if (H == 0 || (!dsigma && !dw)) return RFA_OK;
    if (!w || !grad_out) return fail(RFA_ERR_NULL_POINTER, "rfa_build_random_matrices_backward: NULL tensor pointer");
    if (dsigma && !sigma)
        return fail(RFA_ERR_NULL_POINTER, "rfa_build_random_matrices_backward: dsigma asked for without sigma");
    hipStream_t st = static_cast<hipStream_t>(stream);
    auto* gh = static_cast<const rfa::half_t*>(grad_out);
    if (dsigma)
        RFA_LAUNCH(BUILD_W, rfa::k_build_random_matrices_dsigma, dim3((unsigned)H), dim3(rfa::kThreads), 0, st,
                   static_cast<const rfa::half_t*>(w), gh, static_cast<rfa::half_t*>(dsigma), tau, D, d);
    if (dw) {
        const int64_t total = (int64_t)H * D * d;
        RFA_LAUNCH(BUILD_W, rfa::k_build_random_matrices_dw, dim3((unsigned)((total + rfa::kThreads - 1) / rfa::kThreads)),
                   dim3(rfa::kThreads), 0, st, static_cast<const rfa::half_t*>(sigma), gh,
                   static_cast<rfa::half_t*>(dw), tau, D, d, total);
    }
    RFA_HIP_TRY(hipGetLastError());
    return RFA_OK;
}

// ---- feature map --------------------------------------------------------------------
int rfa_feature_map_supported(int D, int d) { return feature_shape_supported(D, d) ? 1 : 0; }

static int check_feature_dims(const char* fn, int64_t R, int H, int D, int d) {
    if (R < 0 || H <= 0 || D <= 0 || d <= 0)
        return fail(RFA_ERR_BAD_SHAPE, "%s: bad sizes rows=%lld H=%d D=%d d=%d", fn, (long long)R, H, D, d);
    if (!feature_shape_supported(D, d))
        return fail(RFA_ERR_UNSUPPORTED, "%s: no kernel for proj_dim D=%d, head dim d=%d (supported: D in {32,64,128}, d in {64,128})", fn, D, d);
    if (R * H > (int64_t(1) << 31) || R > (int64_t(1) << 30) || H > 65535)
        return fail(RFA_ERR_BAD_SHAPE, "%s: sizes exceed the supported range", fn);
    return RFA_OK;
}

#define RFA_DISPATCH_FEATURE(D, d, CALL)                  \
    if (D == 32 && d == 64) { return CALL(32, 64); }      \
    if (D == 64 && d == 64) { return CALL(64, 64); }      \
    if (D == 128 && d == 64) { return CALL(128, 64); }    \
    if (D == 32 && d == 128) { return CALL(32, 128); }    \
    if (D == 64 && d == 128) { return CALL(64, 128); }    \
    if (D == 128 && d == 128) { return CALL(128, 128); }

int rfa_feature_map_forward(const void* x, const void* w, void* phi, int64_t R, int H, int D, int d, float scale,
                            void* stream) {
    if (int rc = check_feature_dims("rfa_feature_map_forward", R, H, D, d)) return rc;
    if (R == 0) return RFA_OK;
    if (!x || !w || !phi) return fail(RFA_ERR_NULL_POINTER, "rfa_feature_map_forward: NULL tensor pointer");
    if (!aligned16(x) || !aligned16(w) || !aligned16(phi))
        return fail(RFA_ERR_ALIGNMENT, "rfa_feature_map_forward: tensors must be 16-byte aligned");
    hipStream_t st = static_cast<hipStream_t>(stream);
    auto* xh = static_cast<const rfa::half_t*>(x);
    auto* wh = static_cast<const rfa::half_t*>(w);
    auto* ph = static_cast<rfa::half_t*>(phi);
#define RFA_CALL(DD, DH) launch_feature_fwd<DD, DH>(xh, wh, ph, nullptr, nullptr, (int)R, H, scale, st)
    RFA_DISPATCH_FEATURE(D, d, RFA_CALL)
#undef RFA_CALL
    return fail(RFA_ERR_UNSUPPORTED, "unreachable");
}

int rfa_feature_map_forward_pair(const void* x0, const void* x1, const void* w, void* phi0, void* phi1, int64_t R,
                                 int H, int D, int d, float scale, void* stream) {
    if (int rc = check_feature_dims("rfa_feature_map_forward_pair", R, H, D, d)) return rc;
    if (R == 0) return RFA_OK;
    if (!x0 || !x1 || !w || !phi0 || !phi1)
        return fail(RFA_ERR_NULL_POINTER, "rfa_feature_map_forward_pair: NULL tensor pointer");
    if (!aligned16(x0) || !aligned16(x1) || !aligned16(w) || !aligned16(phi0) || !aligned16(phi1))
        return fail(RFA_ERR_ALIGNMENT, "rfa_feature_map_forward_pair: tensors must be 16-byte aligned");
    hipStream_t st = static_cast<hipStream_t>(stream);
#define RFA_CALL(DD, DH)                                                                                         \
    launch_feature_fwd<DD, DH>(static_cast<const rfa::half_t*>(x0), static_cast<const rfa::half_t*>(w),           \
                               static_cast<rfa::half_t*>(phi0), static_cast<const rfa::half_t*>(x1),              \
                               static_cast<rfa::half_t*>(phi1), (int)R, H, scale, st)
    RFA_DISPATCH_FEATURE(D, d, RFA_CALL)
#undef RFA_CALL
    return fail(RFA_ERR_UNSUPPORTED, "unreachable");
}

size_t rfa_feature_map_backward_workspace_bytes(int64_t R, int H, int D, int d) {
    if (R <= 0 || H <= 0 || !feature_shape_supported(D, d)) return 0;
    return (size_t)feature_bwd_blocks(R, H) * H * D * d * 4;
}

int rfa_feature_map_backward(const void* x, const void* w, const void* grad_phi, void* dx, float* dw, int64_t R,
                             int H, int D, int d, float scale, void* workspace, size_t workspace_bytes,
                             void* stream) {
    if (int rc = check_feature_dims("rfa_feature_map_backward", R, H, D, d)) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (R == 0) {
        if (dw) zero_f32(dw, (int64_t)H * D * d, st);
        return RFA_OK;
    }
    if (!x || !w || !grad_phi || !dx) return fail(RFA_ERR_NULL_POINTER, "rfa_feature_map_backward: NULL tensor pointer");
    if (!aligned16(x) || !aligned16(w) || !aligned16(grad_phi) || !aligned16(dx) || !aligned16(dw))
        return fail(RFA_ERR_ALIGNMENT, "rfa_feature_map_backward: tensors must be 16-byte aligned");
    const size_t need = dw ? rfa_feature_map_backward_workspace_bytes(R, H, D, d) : 0;
    if (dw && (!workspace || workspace_bytes < need || !aligned16(workspace)))
        return fail(RFA_ERR_WORKSPACE, "rfa_feature_map_backward: workspace of %zu bytes required, got %zu", need,
                    workspace ? workspace_bytes : (size_t)0);
    auto* xh = static_cast<const rfa::half_t*>(x);
    auto* wh = static_cast<const rfa::half_t*>(w);
    auto* gh = static_cast<const rfa::half_t*>(grad_phi);
    auto* dxh = static_cast<rfa::half_t*>(dx);
    float* part = dw ? static_cast<float*>(workspace) : nullptr;
#define RFA_CALL(DD, DH) launch_feature_bwd<DD, DH>(xh, wh, gh, dxh, nullptr, nullptr, nullptr, dw, part, (int)R, H, scale, st)
    RFA_DISPATCH_FEATURE(D, d, RFA_CALL)
#undef RFA_CALL
    return fail(RFA_ERR_UNSUPPORTED, "unreachable");
}

size_t rfa_feature_map_backward_pair_workspace_bytes(int64_t R, int H, int D, int d) {
    return 2 * rfa_feature_map_backward_workspace_bytes(R, H, D, d);
}

int rfa_feature_map_backward_pair(const void* x0, const void* x1, const void* w, const void* grad_phi0,
                                  const void* grad_phi1, void* dx0, void* dx1, float* dw, int64_t R, int H, int D,
                                  int d, float scale, void* workspace, size_t workspace_bytes, void* stream) {
    if (int rc = check_feature_dims("rfa_feature_map_backward_pair", R, H, D, d)) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (R == 0) {
        if (dw) zero_f32(dw, (int64_t)H * D * d, st);
        return RFA_OK;
    }
    if (!x0 || !x1 || !w || !grad_phi0 || !grad_phi1 || !dx0 || !dx1)
        return fail(RFA_ERR_NULL_POINTER, "rfa_feature_map_backward_pair: NULL tensor pointer");
    if (!aligned16(x0) || !aligned16(x1) || !aligned16(w) || !aligned16(grad_phi0) || !aligned16(grad_phi1) ||
        !aligned16(dx0) || !aligned16(dx1) || !aligned16(dw))
        return fail(RFA_ERR_ALIGNMENT, "rfa_feature_map_backward_pair: tensors must be 16-byte aligned");
    const size_t need = dw ? rfa_feature_map_backward_pair_workspace_bytes(R, H, D, d) : 0;
    if (dw && (!workspace || workspace_bytes < need || !aligned16(workspace)))
        return fail(RFA_ERR_WORKSPACE, "rfa_feature_map_backward_pair: workspace of %zu bytes required, got %zu", need,
                    workspace ? workspace_bytes : (size_t)0);
    float* part = dw ? static_cast<float*>(workspace) : nullptr;
#define RFA_CALL(DD, DH)                                                                                         \
    launch_feature_bwd<DD, DH>(static_cast<const rfa::half_t*>(x0), static_cast<const rfa::half_t*>(w),           \
                               static_cast<const rfa::half_t*>(grad_phi0), static_cast<rfa::half_t*>(dx0),        \
                               static_cast<const rfa::half_t*>(x1), static_cast<const rfa::half_t*>(grad_phi1),   \
                               static_cast<rfa::half_t*>(dx1), dw, part, (int)R, H, scale, st)
    RFA_DISPATCH_FEATURE(D, d, RFA_CALL)
#undef RFA_CALL
    return fail(RFA_ERR_UNSUPPORTED, "unreachable");
}

int rfa_feature_map_backward_pair_packed(const void* x0, const void* x1, const void* w, const void* grad_phi0,
                                         const void* grad_phi1, const void* third, void* packed, float* dw, int64_t R,
                                         int H, int D, int d, float scale, void* workspace, size_t workspace_bytes,
                                         void* stream) {
    if (int rc = check_feature_dims("rfa_feature_map_backward_pair_packed", R, H, D, d)) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (R == 0) {
        if (dw) zero_f32(dw, (int64_t)H * D * d, st);
        return RFA_OK;
    }
    if (!x0 || !x1 || !w || !grad_phi0 || !grad_phi1 || !packed)
        return fail(RFA_ERR_NULL_POINTER, "rfa_feature_map_backward_pair_packed: NULL tensor pointer");
    if (!aligned16(x0) || !aligned16(x1) || !aligned16(w) || !aligned16(grad_phi0) || !aligned16(grad_phi1) ||
        !aligned16(third) || !aligned16(packed) || !aligned16(dw))
        return fail(RFA_ERR_ALIGNMENT, "rfa_feature_map_backward_pair_packed: tensors must be 16-byte aligned");
    if ((int64_t)R * 3 * H * d >= ((int64_t)1 << 40))
        return fail(RFA_ERR_BAD_SHAPE, "rfa_feature_map_backward_pair_packed: sizes exceed the supported range");
    const size_t need = dw ? rfa_feature_map_backward_pair_workspace_bytes(R, H, D, d) : 0;
    if (dw && (!workspace || workspace_bytes < need || !aligned16(workspace)))
        return fail(RFA_ERR_WORKSPACE, "rfa_feature_map_backward_pair_packed: workspace of %zu bytes required, got %zu", need,
                    workspace ? workspace_bytes : (size_t)0);
    float* part = dw ? static_cast<float*>(workspace) : nullptr;
    const int64_t E = (int64_t)H * d;
    auto* pk = static_cast<rfa::half_t*>(packed);
#define RFA_CALL(DD, DH)                                                                                         \
    launch_feature_bwd<DD, DH>(static_cast<const rfa::half_t*>(x0), static_cast<const rfa::half_t*>(w),           \
                               static_cast<const rfa::half_t*>(grad_phi0), pk,                                    \
                               static_cast<const rfa::half_t*>(x1), static_cast<const rfa::half_t*>(grad_phi1),   \
                               pk + E, dw, part, (int)R, H, scale, st, 3 * E,                                     \
                               static_cast<const rfa::half_t*>(third), pk + 2 * E)
    RFA_DISPATCH_FEATURE(D, d, RFA_CALL)
#undef RFA_CALL
    return fail(RFA_ERR_UNSUPPORTED, "unreachable");
}

// ---- projection to heads with the feature map in the epilogue -------------------------
int rfa_project_feature_map(const void* x, const void* const* weights, const void* const* biases, void* const* y,
                            void* const* phi, int np, const void* w_feat, int64_t R, int E, int H, int D, int d,
                            float scale, void* stream) {
    if (int rc = check_feature_dims("rfa_project_feature_map", R, H, D, d)) return rc;
    if (np < 1 || np > rfa::kMaxProjections)
        return fail(RFA_ERR_BAD_SHAPE, "rfa_project_feature_map: %d projections (1..%d supported)", np, rfa::kMaxProjections);
    if (E < 64 || E % 64 != 0)
        return fail(RFA_ERR_BAD_SHAPE, "rfa_project_feature_map: input width E=%d must be a positive multiple of 64", E);
    if (R == 0) return RFA_OK;
    if (!x || !weights || !y) return fail(RFA_ERR_NULL_POINTER, "rfa_project_feature_map: NULL tensor pointer");
    if (!aligned16(x)) return fail(RFA_ERR_ALIGNMENT, "rfa_project_feature_map: tensors must be 16-byte aligned");
    if ((int64_t)8 * ((R + 127) / 128 + 7) / 8 * H * np > (int64_t(1) << 31) - 1)
        return fail(RFA_ERR_BAD_SHAPE, "rfa_project_feature_map: sizes exceed the supported range");
    rfa::ProjectArgs pa{};
    bool any_phi = false;
    for (int p = 0; p < np; ++p) {
        pa.w[p] = static_cast<const rfa::half_t*>(weights[p]);
        pa.b[p] = biases ? static_cast<const rfa::half_t*>(biases[p]) : nullptr;
        pa.y[p] = static_cast<rfa::half_t*>(y[p]);
        pa.phi[p] = phi ? static_cast<rfa::half_t*>(phi[p]) : nullptr;
        if (!pa.w[p] || (!pa.y[p] && !pa.phi[p]))
            return fail(RFA_ERR_NULL_POINTER, "rfa_project_feature_map: NULL weight %d, or neither y nor phi asked for", p);
        if (!aligned16(pa.w[p]) || !aligned16(pa.y[p]) || !aligned16(pa.phi[p]) ||
            (reinterpret_cast<uintptr_t>(pa.b[p]) & 7u))
            return fail(RFA_ERR_ALIGNMENT, "rfa_project_feature_map: tensors must be 16-byte aligned (bias: 8)");
        any_phi = any_phi || pa.phi[p];
    }
    if (any_phi && !w_feat) return fail(RFA_ERR_NULL_POINTER, "rfa_project_feature_map: NULL feature matrices");
    if (!aligned16(w_feat)) return fail(RFA_ERR_ALIGNMENT, "rfa_project_feature_map: tensors must be 16-byte aligned");
    hipStream_t st = static_cast<hipStream_t>(stream);
    auto* xh = static_cast<const rfa::half_t*>(x);
    auto* wfh = static_cast<const rfa::half_t*>(w_feat);
#define RFA_CALL(DD, DH) launch_project_phi<DD, DH>(xh, pa, wfh, (int)R, E, H, np, scale, st)
    RFA_DISPATCH_FEATURE(D, d, RFA_CALL)
#undef RFA_CALL
    return fail(RFA_ERR_UNSUPPORTED, "unreachable");
}

size_t rfa_linear_weight_grad_workspace_bytes(int64_t R, int E_out, int E_in, int np) {
    if (R <= 0 || E_out <= 0 || E_in <= 0 || E_out % 128 || E_in % 128 || np < 1 || np > rfa::kMaxProjections) return 0;
    const WGradPlan pl = make_wgrad_plan(R, E_out, E_in, np);
    return (size_t)pl.nsplit * np * ((size_t)E_out * E_in + E_out) * 4;
}

int rfa_linear_weight_grad(const void* x, const void* const* dy, void* const* dw, void* const* db, int np, int64_t R,
                           int E_out, int E_in, void* workspace, size_t workspace_bytes, void* stream) {
    if (R < 0 || E_out <= 0 || E_in <= 0 || R > (int64_t(1) << 30))
        return fail(RFA_ERR_BAD_SHAPE, "rfa_linear_weight_grad: bad sizes rows=%lld E_out=%d E_in=%d", (long long)R, E_out, E_in);
    if (E_out % 128 || E_in % 128)
        return fail(RFA_ERR_UNSUPPORTED, "rfa_linear_weight_grad: E_out=%d and E_in=%d must be multiples of 128", E_out, E_in);
    if (np < 1 || np > rfa::kMaxProjections)
        return fail(RFA_ERR_BAD_SHAPE, "rfa_linear_weight_grad: %d projections (1..%d supported)", np, rfa::kMaxProjections);
    if (!dy || !dw) return fail(RFA_ERR_NULL_POINTER, "rfa_linear_weight_grad: NULL pointer array");
    hipStream_t st = static_cast<hipStream_t>(stream);
    rfa::WeightGradArgs wa{};
    for (int p = 0; p < np; ++p) {
        wa.dy[p] = static_cast<const rfa::half_t*>(dy[p]);
        wa.dw[p] = static_cast<rfa::half_t*>(dw[p]);
        wa.db[p] = db ? static_cast<rfa::half_t*>(db[p]) : nullptr;
        if (!wa.dw[p] || (R > 0 && !wa.dy[p])) return fail(RFA_ERR_NULL_POINTER, "rfa_linear_weight_grad: NULL tensor %d", p);
        if (!aligned16(wa.dy[p]) || !aligned16(wa.dw[p]) || (reinterpret_cast<uintptr_t>(wa.db[p]) & 7u))
            return fail(RFA_ERR_ALIGNMENT, "rfa_linear_weight_grad: tensors must be 16-byte aligned (bias gradient: 8)");
    }
    if (R > 0 && !x) return fail(RFA_ERR_NULL_POINTER, "rfa_linear_weight_grad: NULL x");
    if (!aligned16(x)) return fail(RFA_ERR_ALIGNMENT, "rfa_linear_weight_grad: tensors must be 16-byte aligned");
    const WGradPlan pl = make_wgrad_plan(R > 0 ? R : 1, E_out, E_in, np);
    const size_t need = (size_t)pl.nsplit * np * ((size_t)E_out * E_in + E_out) * 4;
    if (!workspace || workspace_bytes < need || !aligned16(workspace))
        return fail(RFA_ERR_WORKSPACE, "rfa_linear_weight_grad: workspace of %zu bytes required, got %zu", need,
                    workspace ? workspace_bytes : (size_t)0);
    float* part = static_cast<float*>(workspace);
    float* bpart = part + (size_t)pl.nsplit * np * E_out * E_in;
    const int per_split = np * (E_out / 128) * (E_in / 128);
    const int64_t grid = (int64_t)8 * ((pl.nsplit + 7) / 8) * per_split;
    if (grid > (int64_t(1) << 30)) return fail(RFA_ERR_BAD_SHAPE, "rfa_linear_weight_grad: sizes exceed the supported range");
    auto kern = rfa::k_weight_grad_partial;
    if (int rc = set_lds(kern, rfa::WeightGradCfg::kLds)) return rc;
    // R = 0: every split is empty and the partials come out as zeros
    RFA_LAUNCH(WGRAD_PARTIAL, kern, dim3((unsigned)grid), dim3(rfa::kThreads), rfa::WeightGradCfg::kLds, st,
               static_cast<const rfa::half_t*>(x), wa, part, bpart, (int)R, E_out, E_in, np, pl.nsplit, pl.rows_per_split);
    const int64_t threads = (int64_t)np * ((int64_t)E_out * E_in + E_out) / 4;
    RFA_LAUNCH(WGRAD_REDUCE, rfa::k_weight_grad_reduce, dim3((unsigned)((threads + 255) / 256)), dim3(rfa::kThreads), 0, st,
               (const float*)part, (const float*)bpart, wa, E_out, E_in, np, pl.nsplit);
    RFA_HIP_TRY(hipGetLastError());
    return RFA_OK;
}

// ---- profiling ----------------------------------------------------------------------
int rfa_profile_enable(int on) {
    std::lock_guard<std::mutex> lk(prof::mu);
    prof::enabled = on != 0;
    return RFA_OK;
}

int rfa_profile_collect(void) {
    std::lock_guard<std::mutex> lk(prof::mu);
    for (auto& r : prof::recs) {
        hipError_t e = hipEventSynchronize(r.b);
        float ms = 0.f;
        if (e == hipSuccess) e = hipEventElapsedTime(&ms, r.a, r.b);
        if (e != hipSuccess) return fail(RFA_ERR_HIP, "rfa_profile_collect: %s", hipGetErrorString(e));
        prof::total_ms[r.id] += ms;
        prof::calls[r.id] += 1;
        prof::pool.push_back(r.a);
        prof::pool.push_back(r.b);
    }
    prof::recs.clear();
    return RFA_OK;
}

int rfa_profile_reset(void) {
    if (int rc = rfa_profile_collect()) return rc;
    std::lock_guard<std::mutex> lk(prof::mu);
    for (int i = 0; i < prof::COUNT; ++i) { prof::total_ms[i] = 0.0; prof::calls[i] = 0; }
    return RFA_OK;
}

int rfa_profile_kernel_count(void) { return prof::COUNT; }

int rfa_profile_get(int index, const char** name, double* total_ms, int64_t* calls) {
    if (index < 0 || index >= prof::COUNT) return fail(RFA_ERR_BAD_SHAPE, "rfa_profile_get: index %d out of range", index);
    std::lock_guard<std::mutex> lk(prof::mu);
    if (name) *name = prof::kNames[index];
    if (total_ms) *total_ms = prof::total_ms[index];
    if (calls) *calls = prof::calls[index];
    return RFA_OK;
}

}  // extern "C"
