// C ABI of librfa_hip.so: argument validation, launch planning and kernel
// launches.  See include/rfa_hip.h for the contract of every entry point.
#include "../../include/rfa_hip.h"

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "rfa_causal.h"

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

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

struct ScanPlan {
    int nseg;      // segments per sequence
    int seg_len;   // steps per segment (multiple of 64)
};

// Enough (sequence, segment) workgroups to cover the 256 CUs, at least two
// chunks per segment, at most 16 segments (the consumer sums the totals of all
// earlier segments).
ScanPlan make_plan(int64_t T, int64_t N) {
    ScanPlan p{1, rfa::kChunk};
    if (T <= 0 || N <= 0) return p;
    const int64_t nchunks = (T + rfa::kChunk - 1) / rfa::kChunk;
    int64_t want = (256 + N - 1) / N;
    if (const char* env = getenv("RFA_HIP_NSEG")) {
        const long v = strtol(env, nullptr, 10);
        if (v >= 1) want = v;
    } else {
        if (want > nchunks / 2) want = nchunks / 2;
    }
    if (want > 16) want = 16;
    if (want > nchunks) want = nchunks;
    if (want < 1) want = 1;
    const int64_t cps = (nchunks + want - 1) / want;
    p.nseg = (int)((nchunks + cps - 1) / cps);
    p.seg_len = (int)(cps * rfa::kChunk);
    return p;
}

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

template <typename Kern>
int set_lds(Kern kern, size_t bytes) {
    RFA_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
    return RFA_OK;
}

template <int KD, int DH>
int launch_forward(const rfa::half_t* q, const rfa::half_t* k, const rfa::half_t* v, rfa::half_t* out,
                   int T, int N, const ScanPlan& p, char* ws, const Workspace& wl, hipStream_t st) {
    using Cfg = rfa::CausalCfg<KD, DH>;
    float* wsS = reinterpret_cast<float*>(ws + wl.S);
    float* wsZ = reinterpret_cast<float*>(ws + wl.Z);
    if (p.nseg > 1) {
        auto kern = rfa::k_segment_state<KD, DH>;
        if (int rc = set_lds(kern, Cfg::kSegStateLds)) return rc;
        hipLaunchKernelGGL(kern, dim3(N * (p.nseg - 1)), dim3(rfa::kThreads), Cfg::kSegStateLds, st,
                           k, v, wsS, wsZ, T, N, p.nseg, p.seg_len);
    }
    auto kern = rfa::k_causal_fwd<KD, DH>;
    if (int rc = set_lds(kern, Cfg::kFwdLds)) return rc;
    hipLaunchKernelGGL(kern, dim3(N * p.nseg), dim3(rfa::kThreads), Cfg::kFwdLds, st, q, k, v, out,
                       wsS, wsZ, T, N, p.nseg, p.seg_len);
    RFA_HIP_TRY(hipGetLastError());
    return RFA_OK;
}

template <int KD, int DH>
int launch_backward(const rfa::half_t* q, const rfa::half_t* k, const rfa::half_t* v,
                    const rfa::half_t* g, rfa::half_t* dq, rfa::half_t* dk, rfa::half_t* dv, int T, int N,
                    const ScanPlan& p, char* ws, const Workspace& wl, hipStream_t st) {
    using Cfg = rfa::CausalCfg<KD, DH>;
    float* wsS = reinterpret_cast<float*>(ws + wl.S);
    float* wsZ = reinterpret_cast<float*>(ws + wl.Z);
    float* wsR = reinterpret_cast<float*>(ws + wl.R);
    float* wsr = reinterpret_cast<float*>(ws + wl.r);
    float* den = reinterpret_cast<float*>(ws + wl.den);
    float* gz = reinterpret_cast<float*>(ws + wl.gz);
    if (p.nseg > 1) {
        auto kern = rfa::k_segment_state<KD, DH>;
        if (int rc = set_lds(kern, Cfg::kSegStateLds)) return rc;
        hipLaunchKernelGGL(kern, dim3(N * (p.nseg - 1)), dim3(rfa::kThreads), Cfg::kSegStateLds, st,
                           k, v, wsS, wsZ, T, N, p.nseg, p.seg_len);
    }
    {
        auto kern = rfa::k_causal_bwd_dq<KD, DH>;
        if (int rc = set_lds(kern, Cfg::kBwdDqLds)) return rc;
        hipLaunchKernelGGL(kern, dim3(N * p.nseg), dim3(rfa::kThreads), Cfg::kBwdDqLds, st, q, k, v, g,
                           dq, wsS, wsZ, wsR, wsr, den, gz, T, N, p.nseg, p.seg_len);
    }
    {
        auto kern = rfa::k_causal_bwd_dkdv<KD, DH>;
        if (int rc = set_lds(kern, Cfg::kBwdDkLds)) return rc;
        hipLaunchKernelGGL(kern, dim3(N * p.nseg), dim3(rfa::kThreads), Cfg::kBwdDkLds, st, q, k, v, g,
                           dk, dv, wsR, wsr, den, gz, T, N, p.nseg, p.seg_len);
    }
    RFA_HIP_TRY(hipGetLastError());
    return RFA_OK;
}

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

}  // namespace

extern "C" {

int rfa_version(void) { return 100; }

const char* rfa_last_error(void) { return g_err; }

int rfa_shape_supported(int K, int d) {
    return ((K == 64 || K == 128 || K == 256) && (d == 64 || d == 128)) ? 1 : 0;
}

int rfa_causal_num_segments(int64_t T, int64_t N) { return make_plan(T, N).nseg; }

int rfa_selftest_layout(void* stream) {
    hipStream_t st = static_cast<hipStream_t>(stream);
    int* dbad = nullptr;
    RFA_HIP_TRY(hipMalloc(&dbad, sizeof(int)));
    int hbad = 0;
    hipError_t e = hipMemcpyAsync(dbad, &hbad, sizeof(int), hipMemcpyHostToDevice, st);
    if (e == hipSuccess) {
        hipLaunchKernelGGL(k_selftest, dim3(1), dim3(64), 0, st, dbad);
        e = hipMemcpyAsync(&hbad, dbad, sizeof(int), hipMemcpyDeviceToHost, st);
    }
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    (void)hipFree(dbad);
    if (e != hipSuccess) return fail(RFA_ERR_HIP, "selftest: %s", hipGetErrorString(e));
    if (hbad) return fail(RFA_ERR_HIP, "selftest: %d lane values differ from the assumed MFMA / LDS layout", hbad);
    return RFA_OK;
}

size_t rfa_causal_forward_workspace_bytes(int64_t T, int64_t N, int K, int d) {
    if (T <= 0 || N <= 0 || !rfa_shape_supported(K, d)) return 0;
    return layout_workspace(T, N, K, d, make_plan(T, N), false).total;
}

size_t rfa_causal_backward_workspace_bytes(int64_t T, int64_t N, int K, int d) {
    if (T <= 0 || N <= 0 || !rfa_shape_supported(K, d)) return 0;
    return layout_workspace(T, N, K, d, make_plan(T, N), true).total;
}

#define RFA_DISPATCH_KD(K, d, CALL)                                   \
    if (K == 64 && d == 64) { return CALL(64, 64); }                  \
    if (K == 128 && d == 64) { return CALL(128, 64); }                \
    if (K == 256 && d == 64) { return CALL(256, 64); }                \
    if (K == 64 && d == 128) { return CALL(64, 128); }                \
    if (K == 128 && d == 128) { return CALL(128, 128); }              \
    if (K == 256 && d == 128) { return CALL(256, 128); }

int rfa_causal_forward(const void* q, const void* k, const void* v, void* out, int64_t T, int64_t N,
                       int K, int d, void* workspace, size_t workspace_bytes, void* stream) {
    if (int rc = check_causal_dims(T, N, K, d)) return rc;
    if (T == 0 || N == 0) return RFA_OK;
    if (!q || !k || !v || !out) return fail(RFA_ERR_NULL_POINTER, "rfa_causal_forward: NULL tensor pointer");
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(out))
        return fail(RFA_ERR_ALIGNMENT, "rfa_causal_forward: tensors must be 16-byte aligned");
    const ScanPlan p = make_plan(T, N);
    const Workspace wl = layout_workspace(T, N, K, d, p, false);
    if (wl.total > 0 && (!workspace || workspace_bytes < wl.total || !aligned16(workspace)))
        return fail(RFA_ERR_WORKSPACE, "rfa_causal_forward: workspace of %zu bytes required, got %zu", wl.total,
                    workspace ? workspace_bytes : (size_t)0);
    hipStream_t st = static_cast<hipStream_t>(stream);
    auto* qh = static_cast<const rfa::half_t*>(q);
    auto* kh = static_cast<const rfa::half_t*>(k);
    auto* vh = static_cast<const rfa::half_t*>(v);
    auto* oh = static_cast<rfa::half_t*>(out);
    char* ws = static_cast<char*>(workspace);
#define RFA_CALL_FWD(KD, DH) launch_forward<KD, DH>(qh, kh, vh, oh, (int)T, (int)N, p, ws, wl, st)
    RFA_DISPATCH_KD(K, d, RFA_CALL_FWD)
#undef RFA_CALL_FWD
    return fail(RFA_ERR_UNSUPPORTED, "unreachable");
}

int rfa_causal_backward(const void* q, const void* k, const void* v, const void* grad_attn, void* dq,
                        void* dk, void* dv, int64_t T, int64_t N, int K, int d, void* workspace,
                        size_t workspace_bytes, void* stream) {
    if (int rc = check_causal_dims(T, N, K, d)) return rc;
    if (T == 0 || N == 0) return RFA_OK;
    if (!q || !k || !v || !grad_attn || !dq || !dk || !dv)
        return fail(RFA_ERR_NULL_POINTER, "rfa_causal_backward: NULL tensor pointer");
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(grad_attn) || !aligned16(dq) ||
        !aligned16(dk) || !aligned16(dv))
        return fail(RFA_ERR_ALIGNMENT, "rfa_causal_backward: tensors must be 16-byte aligned");
    const ScanPlan p = make_plan(T, N);
    const Workspace wl = layout_workspace(T, N, K, d, p, true);
    if (!workspace || workspace_bytes < wl.total || !aligned16(workspace))
        return fail(RFA_ERR_WORKSPACE, "rfa_causal_backward: workspace of %zu bytes required, got %zu", wl.total,
                    workspace ? workspace_bytes : (size_t)0);
    hipStream_t st = static_cast<hipStream_t>(stream);
    auto* qh = static_cast<const rfa::half_t*>(q);
    auto* kh = static_cast<const rfa::half_t*>(k);
    auto* vh = static_cast<const rfa::half_t*>(v);
    auto* gh = static_cast<const rfa::half_t*>(grad_attn);
    auto* dqh = static_cast<rfa::half_t*>(dq);
    auto* dkh = static_cast<rfa::half_t*>(dk);
    auto* dvh = static_cast<rfa::half_t*>(dv);
    char* ws = static_cast<char*>(workspace);
#define RFA_CALL_BWD(KD, DH) launch_backward<KD, DH>(qh, kh, vh, gh, dqh, dkh, dvh, (int)T, (int)N, p, ws, wl, st)
    RFA_DISPATCH_KD(K, d, RFA_CALL_BWD)
#undef RFA_CALL_BWD
    return fail(RFA_ERR_UNSUPPORTED, "unreachable");
}

}  // extern "C"
