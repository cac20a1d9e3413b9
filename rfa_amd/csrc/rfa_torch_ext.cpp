// PyTorch-ROCm C++ binding of librfa_hip.so: the module that stands where the reference's pybind
// extension rfa_cuda stood (random_feature_attention/cuda/rfa_cuda.cpp:22-42).  Same two entry
// points, forward(q, k, v) -> Tensor and backward(q, k, v, grad_attn) -> [grad_q, grad_k, grad_v],
// plus the entry points for the other parts of the path.  No kernels here: every function checks
// its tensors (TORCH_CHECK, where the reference checked nothing: cuda/forward.cu:156-159), makes
// the tensors' device current, allocates outputs and workspaces from torch's allocator and calls
// the C ABI (include/rfa_hip.h) with raw device pointers on torch's current HIP stream.
//
// Built as a plain host C++ file against torch's headers (see rfa_amd/build.py); the ctypes binding
// in rfa_amd/_lib.py stays as the torch-free way to reach the same library.
#include <torch/extension.h>

#include <c10/hip/HIPGuard.h>
#include <c10/hip/HIPStream.h>

#include <array>
#include <string>
#include <vector>

#include "../../include/rfa_hip.h"

namespace {

using torch::Tensor;

void check_rc(int rc) {
    // TORCH_CHECK raises RuntimeError in Python; the text carries the library's own message
    TORCH_CHECK(rc == RFA_OK, "librfa_hip error ", rc, ": ", rfa_last_error());
}

void check_half(const char* name, const Tensor& t, int64_t ndim) {
    TORCH_CHECK(t.is_cuda(), name, " must live on a HIP device (got ", t.device(), "); the kernels have no CPU path");
    TORCH_CHECK_TYPE(t.scalar_type() == torch::kFloat16, name, " must be float16 (got ", t.scalar_type(), ")");
    TORCH_CHECK_VALUE(t.dim() == ndim, name, " must have ", ndim, " dims (got ", t.sizes(), ")");
    TORCH_CHECK_VALUE(t.is_contiguous(), name, " must be contiguous");
}

void check_f32(const char* name, const Tensor& t, at::IntArrayRef shape) {
    TORCH_CHECK(t.is_cuda(), name, " must live on a HIP device");
    TORCH_CHECK_TYPE(t.scalar_type() == torch::kFloat32, name, " must be float32 (got ", t.scalar_type(), ")");
    TORCH_CHECK_VALUE(t.sizes() == shape, name, " must have shape ", shape, " (got ", t.sizes(), ")");
    TORCH_CHECK_VALUE(t.is_contiguous(), name, " must be contiguous");
}

void check_qkv(const Tensor& q, const Tensor& k, const Tensor& v) {
    check_half("q", q, 3);
    check_half("k", k, 3);
    check_half("v", v, 3);
    TORCH_CHECK_VALUE(q.sizes() == k.sizes(), "q ", q.sizes(), " and k ", k.sizes(), " differ");
    TORCH_CHECK_VALUE(v.size(0) == q.size(0) && v.size(1) == q.size(1), "v ", v.sizes(), " does not match q ", q.sizes(),
                      " in [tgt_len, bsz*heads]");
    TORCH_CHECK(q.device() == k.device() && q.device() == v.device(), "q, k, v must be on one device");
}

// device guard + current stream of the tensors' device
struct Launch {
    c10::hip::HIPGuard guard;
    void* stream;
    explicit Launch(const Tensor& t)
        : guard(t.get_device()), stream(c10::hip::getCurrentHIPStream(t.get_device()).stream()) {}
};

Tensor workspace(size_t nbytes, const Tensor& like) {
    // torch's caching allocator: no hipMalloc on the steady-state path
    return torch::empty({(int64_t)(nbytes ? nbytes : 1)}, like.options().dtype(torch::kUInt8));
}

void* ptr(const Tensor& t) { return t.data_ptr(); }
void* ptr(const c10::optional<Tensor>& t) { return t.has_value() ? t->data_ptr() : nullptr; }

// ---- causal -------------------------------------------------------------------------
Tensor forward(const Tensor& q, const Tensor& k, const Tensor& v) {
    check_qkv(q, k, v);
    const int64_t T = q.size(0), N = q.size(1);
    const int K = (int)q.size(2), d = (int)v.size(2);
    Tensor out = torch::empty_like(v);
    Launch l(q);
    const size_t nbytes = rfa_causal_forward_workspace_bytes(T, N, K, d);
    Tensor ws = workspace(nbytes, q);
    check_rc(rfa_causal_forward(ptr(q), ptr(k), ptr(v), ptr(out), T, N, K, d, ptr(ws), nbytes, l.stream));
    return out;
}

std::tuple<Tensor, Tensor, Tensor> prefill(const Tensor& q, const Tensor& k, const Tensor& v) {
    check_qkv(q, k, v);
    const int64_t T = q.size(0), N = q.size(1);
    const int K = (int)q.size(2), d = (int)v.size(2);
    Tensor out = torch::empty_like(v);
    Tensor s = torch::empty({N, K, d}, q.options().dtype(torch::kFloat32));
    Tensor z = torch::empty({N, K}, q.options().dtype(torch::kFloat32));
    Launch l(q);
    const size_t nbytes = rfa_causal_forward_workspace_bytes(T, N, K, d);
    Tensor ws = workspace(nbytes, q);
    check_rc(rfa_causal_prefill(ptr(q), ptr(k), ptr(v), ptr(out), s.data_ptr<float>(), z.data_ptr<float>(), T, N, K, d,
                                ptr(ws), nbytes, l.stream));
    return {out, s, z};
}

std::tuple<Tensor, Tensor> forward_save(const Tensor& q, const Tensor& k, const Tensor& v) {
    check_qkv(q, k, v);
    const int64_t T = q.size(0), N = q.size(1);
    const int K = (int)q.size(2), d = (int)v.size(2);
    Tensor out = torch::empty_like(v);
    Launch l(q);
    const size_t nbytes = rfa_causal_forward_workspace_bytes(T, N, K, d);
    const size_t sbytes = rfa_causal_saved_state_bytes(T, N, K, d);
    Tensor ws = workspace(nbytes, q);
    Tensor saved = workspace(sbytes, q);
    check_rc(rfa_causal_forward_save(ptr(q), ptr(k), ptr(v), ptr(out), ptr(saved), sbytes, T, N, K, d, ptr(ws), nbytes,
                                     l.stream));
    return {out, saved};
}

std::vector<Tensor> backward_saved(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& grad_attn,
                                   const Tensor& out, const Tensor& saved) {
    check_qkv(q, k, v);
    check_half("grad_attn", grad_attn, 3);
    check_half("out", out, 3);
    TORCH_CHECK_VALUE(grad_attn.sizes() == v.sizes(), "grad_attn ", grad_attn.sizes(), " must match v ", v.sizes());
    TORCH_CHECK_VALUE(out.sizes() == v.sizes(), "out ", out.sizes(), " must match v ", v.sizes());
    TORCH_CHECK_TYPE(saved.is_cuda() && saved.scalar_type() == torch::kUInt8 && saved.is_contiguous(),
                     "saved must be the byte buffer returned by forward_save");
    const int64_t T = q.size(0), N = q.size(1);
    const int K = (int)q.size(2), d = (int)v.size(2);
    Tensor dq = torch::empty_like(q), dk = torch::empty_like(k), dv = torch::empty_like(v);
    Launch l(q);
    // sized for the plan of the forward call that wrote `saved`
    const size_t nbytes = rfa_causal_backward_saved_workspace_bytes(ptr(saved), T, N, K, d);
    Tensor ws = workspace(nbytes, q);
    check_rc(rfa_causal_backward_saved(ptr(q), ptr(k), ptr(v), ptr(grad_attn), ptr(out), ptr(saved), (size_t)saved.numel(),
                                       ptr(dq), ptr(dk), ptr(dv), T, N, K, d, ptr(ws), nbytes, l.stream));
    return {dq, dk, dv};
}

std::vector<Tensor> backward(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& grad_attn) {
    check_qkv(q, k, v);
    check_half("grad_attn", grad_attn, 3);
    TORCH_CHECK_VALUE(grad_attn.sizes() == v.sizes(), "grad_attn ", grad_attn.sizes(), " must match v ", v.sizes());
    const int64_t T = q.size(0), N = q.size(1);
    const int K = (int)q.size(2), d = (int)v.size(2);
    Tensor dq = torch::empty_like(q), dk = torch::empty_like(k), dv = torch::empty_like(v);
    Launch l(q);
    const size_t nbytes = rfa_causal_backward_workspace_bytes(T, N, K, d);
    Tensor ws = workspace(nbytes, q);
    check_rc(rfa_causal_backward(ptr(q), ptr(k), ptr(v), ptr(grad_attn), ptr(dq), ptr(dk), ptr(dv), T, N, K, d, ptr(ws),
                                 nbytes, l.stream));
    return {dq, dk, dv};
}

// ---- feature map ----------------------------------------------------------------------
void check_feature_args(const Tensor& x, const Tensor& w) {
    check_half("x", x, 4);
    check_half("random_matrices", w, 3);
    TORCH_CHECK_VALUE(w.size(0) == x.size(2) && w.size(2) == x.size(3), "random_matrices ", w.sizes(),
                      " must be [num_heads, proj_dim, head_dim] for x ", x.sizes());
    TORCH_CHECK(x.device() == w.device(), "x and random_matrices must be on one device");
}

Tensor build_random_matrices(const Tensor& w, const c10::optional<Tensor>& sigma, double tau) {
    check_half("random_matrices", w, 3);
    const int H = (int)w.size(0), D = (int)w.size(1), d = (int)w.size(2);
    if (sigma.has_value()) {
        check_half("sigma", *sigma, 3);
        TORCH_CHECK_VALUE(sigma->size(0) == H && sigma->size(1) == 1 && sigma->size(2) == d, "sigma must be [", H, ", 1, ",
                          d, "] (got ", sigma->sizes(), ")");
    }
    Tensor out = torch::empty_like(w);
    Launch l(w);
    check_rc(rfa_build_random_matrices(ptr(w), ptr(sigma), (float)tau, ptr(out), H, D, d, l.stream));
    return out;
}

std::tuple<c10::optional<Tensor>, c10::optional<Tensor>> build_random_matrices_backward(
    const Tensor& w, const c10::optional<Tensor>& sigma, const Tensor& grad_out, double tau, bool want_dsigma, bool want_dw) {
    check_half("random_matrices", w, 3);
    check_half("grad_out", grad_out, 3);
    TORCH_CHECK_VALUE(grad_out.sizes() == w.sizes(), "grad_out must have the shape of random_matrices");
    const int H = (int)w.size(0), D = (int)w.size(1), d = (int)w.size(2);
    want_dsigma = want_dsigma && sigma.has_value();
    c10::optional<Tensor> dsigma, dw;
    if (want_dsigma) dsigma = torch::empty({H, 1, d}, w.options());
    if (want_dw) dw = torch::empty_like(w);
    Launch l(w);
    check_rc(rfa_build_random_matrices_backward(ptr(w), ptr(sigma), ptr(grad_out), (float)tau, ptr(dsigma), ptr(dw), H, D, d,
                                                l.stream));
    return {dsigma, dw};
}

Tensor feature_map_forward(const Tensor& x, const Tensor& w, double scale) {
    check_feature_args(x, w);
    const int64_t L = x.size(0), B = x.size(1);
    const int H = (int)x.size(2), d = (int)x.size(3), D = (int)w.size(1);
    Tensor phi = torch::empty({L, B, H, 2 * D}, x.options());
    Launch l(x);
    check_rc(rfa_feature_map_forward(ptr(x), ptr(w), ptr(phi), L * B, H, D, d, (float)scale, l.stream));
    return phi;
}

std::tuple<Tensor, Tensor> feature_map_forward_pair(const Tensor& x0, const Tensor& x1, const Tensor& w, double scale) {
    check_feature_args(x0, w);
    check_feature_args(x1, w);
    TORCH_CHECK(x0.sizes() == x1.sizes() && x0.device() == x1.device(), "x0 ", x0.sizes(), " and x1 ", x1.sizes(),
                " must have one shape and device");
    const int64_t L = x0.size(0), B = x0.size(1);
    const int H = (int)x0.size(2), d = (int)x0.size(3), D = (int)w.size(1);
    Tensor phi0 = torch::empty({L, B, H, 2 * D}, x0.options());
    Tensor phi1 = torch::empty_like(phi0);
    Launch l(x0);
    check_rc(rfa_feature_map_forward_pair(ptr(x0), ptr(x1), ptr(w), ptr(phi0), ptr(phi1), L * B, H, D, d, (float)scale,
                                          l.stream));
    return {phi0, phi1};
}

std::tuple<Tensor, c10::optional<Tensor>> feature_map_backward(const Tensor& x, const Tensor& w, const Tensor& grad_phi,
                                                               double scale, bool need_dw) {
    check_feature_args(x, w);
    const int64_t L = x.size(0), B = x.size(1);
    const int H = (int)x.size(2), d = (int)x.size(3), D = (int)w.size(1);
    check_half("grad_phi", grad_phi, 4);
    TORCH_CHECK_VALUE(grad_phi.size(0) == L && grad_phi.size(1) == B && grad_phi.size(2) == H && grad_phi.size(3) == 2 * D,
                      "grad_phi ", grad_phi.sizes(), " must be [", L, ", ", B, ", ", H, ", ", 2 * D, "]");
    Tensor dx = torch::empty_like(x);
    c10::optional<Tensor> dw;       // need_dw = false: w counts as a constant, no gradient formed
    if (need_dw) dw = torch::empty({H, D, d}, x.options().dtype(torch::kFloat32));
    Launch l(x);
    const size_t nbytes = need_dw ? rfa_feature_map_backward_workspace_bytes(L * B, H, D, d) : 0;
    Tensor ws = workspace(nbytes, x);
    check_rc(rfa_feature_map_backward(ptr(x), ptr(w), ptr(grad_phi), ptr(dx), need_dw ? dw->data_ptr<float>() : nullptr,
                                      L * B, H, D, d, (float)scale, need_dw ? ptr(ws) : nullptr, nbytes, l.stream));
    return {dx, dw};
}

std::tuple<Tensor, Tensor, c10::optional<Tensor>> feature_map_backward_pair(const Tensor& x0, const Tensor& x1,
                                                                            const Tensor& w, const Tensor& g0,
                                                                            const Tensor& g1, double scale, bool need_dw) {
    check_feature_args(x0, w);
    check_feature_args(x1, w);
    TORCH_CHECK_VALUE(x0.sizes() == x1.sizes(), "the two tensors must have one shape");
    const int64_t L = x0.size(0), B = x0.size(1);
    const int H = (int)x0.size(2), d = (int)x0.size(3), D = (int)w.size(1);
    for (const Tensor* g : {&g0, &g1}) {
        check_half("grad_phi", *g, 4);
        TORCH_CHECK_VALUE(g->size(0) == L && g->size(1) == B && g->size(2) == H && g->size(3) == 2 * D, "grad_phi ",
                          g->sizes(), " must be [", L, ", ", B, ", ", H, ", ", 2 * D, "]");
    }
    Tensor dx0 = torch::empty_like(x0), dx1 = torch::empty_like(x1);
    c10::optional<Tensor> dw;
    if (need_dw) dw = torch::empty({H, D, d}, x0.options().dtype(torch::kFloat32));
    Launch l(x0);
    const size_t nbytes = need_dw ? rfa_feature_map_backward_pair_workspace_bytes(L * B, H, D, d) : 0;
    Tensor ws = workspace(nbytes, x0);
    check_rc(rfa_feature_map_backward_pair(ptr(x0), ptr(x1), ptr(w), ptr(g0), ptr(g1), ptr(dx0), ptr(dx1),
                                           need_dw ? dw->data_ptr<float>() : nullptr, L * B, H, D, d, (float)scale,
                                           need_dw ? ptr(ws) : nullptr, nbytes, l.stream));
    return {dx0, dx1, dw};
}

std::tuple<Tensor, c10::optional<Tensor>> feature_map_backward_pair_packed(const Tensor& x0, const Tensor& x1,
                                                                           const Tensor& w, const Tensor& g0,
                                                                           const Tensor& g1,
                                                                           const c10::optional<Tensor>& third,
                                                                           double scale, bool need_dw) {
    check_feature_args(x0, w);
    check_feature_args(x1, w);
    TORCH_CHECK_VALUE(x0.sizes() == x1.sizes(), "the two tensors must have one shape");
    const int64_t L = x0.size(0), B = x0.size(1);
    const int H = (int)x0.size(2), d = (int)x0.size(3), D = (int)w.size(1);
    for (const Tensor* g : {&g0, &g1}) {
        check_half("grad_phi", *g, 4);
        TORCH_CHECK_VALUE(g->size(0) == L && g->size(1) == B && g->size(2) == H && g->size(3) == 2 * D, "grad_phi ",
                          g->sizes(), " must be [", L, ", ", B, ", ", H, ", ", 2 * D, "]");
    }
    if (third) {
        check_half("third", *third, third->dim());
        TORCH_CHECK_VALUE(third->numel() == x0.numel(), "third ", third->sizes(), " must hold ", L * B, " rows of ", H * d);
    }
    Tensor packed = torch::empty({L * B, 3 * (int64_t)H * d}, x0.options());
    c10::optional<Tensor> dw;
    if (need_dw) dw = torch::empty({H, D, d}, x0.options().dtype(torch::kFloat32));
    Launch l(x0);
    const size_t nbytes = need_dw ? rfa_feature_map_backward_pair_workspace_bytes(L * B, H, D, d) : 0;
    Tensor ws = workspace(nbytes, x0);
    check_rc(rfa_feature_map_backward_pair_packed(ptr(x0), ptr(x1), ptr(w), ptr(g0), ptr(g1), third ? ptr(*third) : nullptr,
                                                  ptr(packed), need_dw ? dw->data_ptr<float>() : nullptr, L * B, H, D, d,
                                                  (float)scale, need_dw ? ptr(ws) : nullptr, nbytes, l.stream));
    return {packed, dw};
}

// ---- projections ----------------------------------------------------------------------
// keep_y = false: a projection whose phi is asked for returns None in place of y (nothing will
// differentiate through it)
std::tuple<std::vector<c10::optional<Tensor>>, std::vector<c10::optional<Tensor>>> project_feature_map(
    const Tensor& x, const std::vector<Tensor>& weights, const std::vector<c10::optional<Tensor>>& biases,
    const std::vector<bool>& want_phi, const c10::optional<Tensor>& w, int64_t heads, double scale, bool keep_y) {
    check_half("x", x, 3);
    const int64_t L = x.size(0), B = x.size(1), E = x.size(2);
    const size_t n = weights.size();
    TORCH_CHECK_VALUE(n >= 1 && n <= 3 && biases.size() == n && want_phi.size() == n,
                      "1..3 projections with one bias entry and one want_phi flag each");
    const int64_t out_dim = weights[0].size(0);
    TORCH_CHECK_VALUE(out_dim % heads == 0, "output width ", out_dim, " is not a multiple of heads=", heads);
    const int64_t d = out_dim / heads;
    bool any_phi = false;
    for (size_t p = 0; p < n; ++p) {
        check_half("weight", weights[p], 2);
        TORCH_CHECK_VALUE(weights[p].size(0) == out_dim && weights[p].size(1) == E, "weight ", weights[p].sizes(),
                          " must be [", out_dim, ", ", E, "]");
        TORCH_CHECK(weights[p].device() == x.device(), "x and weights must be on one device");
        if (biases[p].has_value()) {
            check_half("bias", *biases[p], 1);
            TORCH_CHECK_VALUE(biases[p]->size(0) == out_dim && biases[p]->device() == x.device(), "bias must be [", out_dim,
                              "] on x's device");
        }
        any_phi = any_phi || want_phi[p];
    }
    int64_t D = 32;
    if (any_phi) {
        TORCH_CHECK_VALUE(w.has_value(), "feature matrices are needed when a phi is wanted");
        check_half("random_matrices", *w, 3);
        TORCH_CHECK_VALUE(w->size(0) == heads && w->size(2) == d && w->device() == x.device(), "random_matrices ",
                          w->sizes(), " must be [", heads, ", D, ", d, "] on x's device");
        D = w->size(1);
    }
    std::vector<c10::optional<Tensor>> ys, phis;
    std::array<const void*, 3> wp{}, bp{};
    std::array<void*, 3> yp{}, pp{};
    for (size_t p = 0; p < n; ++p) {
        ys.push_back(keep_y || !want_phi[p] ? c10::optional<Tensor>(torch::empty({L, B, heads, d}, x.options())) : c10::nullopt);
        phis.push_back(want_phi[p] ? c10::optional<Tensor>(torch::empty({L, B, heads, 2 * D}, x.options())) : c10::nullopt);
        wp[p] = ptr(weights[p]);
        bp[p] = ptr(biases[p]);
        yp[p] = ptr(ys[p]);
        pp[p] = ptr(phis[p]);
    }
    Launch l(x);
    check_rc(rfa_project_feature_map(ptr(x), wp.data(), bp.data(), yp.data(), pp.data(), (int)n, any_phi ? ptr(w) : nullptr,
                                     L * B, (int)E, (int)heads, (int)D, (int)d, (float)scale, l.stream));
    return {ys, phis};
}

std::tuple<std::vector<Tensor>, std::vector<c10::optional<Tensor>>> linear_weight_grad(
    const Tensor& x, const std::vector<Tensor>& dys, const std::vector<bool>& want_bias) {
    check_half("x", x, 2);
    const int64_t R = x.size(0), e_in = x.size(1);
    const size_t n = dys.size();
    TORCH_CHECK_VALUE(n >= 1 && n <= 3 && want_bias.size() == n, "1..3 layers with one want_bias flag each");
    const int64_t e_out = dys[0].size(1);
    TORCH_CHECK_VALUE(e_out % 128 == 0 && e_in % 128 == 0, "E_out=", e_out, " and E_in=", e_in, " must be multiples of 128");
    std::vector<Tensor> dws;
    std::vector<c10::optional<Tensor>> dbs;
    std::array<const void*, 3> dyp{};
    std::array<void*, 3> dwp{}, dbp{};
    for (size_t p = 0; p < n; ++p) {
        check_half("dy", dys[p], 2);
        TORCH_CHECK_VALUE(dys[p].size(0) == R && dys[p].size(1) == e_out && dys[p].device() == x.device(), "dy ",
                          dys[p].sizes(), " must be [", R, ", ", e_out, "] on x's device");
        dws.push_back(torch::empty({e_out, e_in}, x.options()));
        dbs.push_back(want_bias[p] ? c10::optional<Tensor>(torch::empty({e_out}, x.options())) : c10::nullopt);
        dyp[p] = ptr(dys[p]);
        dwp[p] = ptr(dws[p]);
        dbp[p] = ptr(dbs[p]);
    }
    Launch l(x);
    const size_t nbytes = rfa_linear_weight_grad_workspace_bytes(R > 0 ? R : 1, (int)e_out, (int)e_in, (int)n);
    Tensor ws = workspace(nbytes, x);
    check_rc(rfa_linear_weight_grad(ptr(x), dyp.data(), dwp.data(), dbp.data(), (int)n, R, (int)e_out, (int)e_in, ptr(ws),
                                    nbytes, l.stream));
    return {dws, dbs};
}

// ---- cross attention --------------------------------------------------------------------
// key_padding_mask [B, S] (non-zero = pad) -> a byte tensor the kernels can read.  The kernels test
// the bytes for non-zero: a contiguous one-byte mask goes in as it is (no conversion kernels in
// front of the launch), anything else is reduced to 0/1 bytes first.
c10::optional<Tensor> mask_bytes(const c10::optional<Tensor>& mask, int64_t B, int64_t S, const Tensor& like) {
    if (!mask.has_value()) return c10::nullopt;
    TORCH_CHECK_VALUE(mask->dim() == 2 && mask->size(0) == B && mask->size(1) == S, "key_padding_mask must be [", B, ", ", S,
                      "] (got ", mask->sizes(), ")");
    TORCH_CHECK(mask->device() == like.device(), "key_padding_mask must be on the tensors' device");
    if ((mask->scalar_type() == torch::kBool || mask->scalar_type() == torch::kUInt8) && mask->is_contiguous())
        return mask->scalar_type() == torch::kBool ? mask->view(torch::kUInt8) : *mask;
    return mask->ne(0).to(torch::kUInt8).contiguous();
}

std::tuple<Tensor, Tensor> cross_state(const Tensor& phi_k, const Tensor& v, const c10::optional<Tensor>& pad) {
    check_half("phi_k", phi_k, 4);
    check_half("v", v, 4);
    TORCH_CHECK_VALUE(phi_k.size(0) == v.size(0) && phi_k.size(1) == v.size(1) && phi_k.size(2) == v.size(2),
                      "phi_k and v must agree in [src_len, bsz, heads]");
    const int64_t S = phi_k.size(0), B = phi_k.size(1);
    const int H = (int)phi_k.size(2), K = (int)phi_k.size(3), d = (int)v.size(3);
    Tensor s = torch::empty({B, H, K, d}, v.options().dtype(torch::kFloat32));
    Tensor z = torch::empty({B, H, K}, v.options().dtype(torch::kFloat32));
    auto m = mask_bytes(pad, B, S, v);
    Launch l(v);
    check_rc(rfa_cross_state(ptr(phi_k), ptr(v), static_cast<const uint8_t*>(ptr(m)), s.data_ptr<float>(),
                             z.data_ptr<float>(), S, B, H, K, d, l.stream));
    return {s, z};
}

std::tuple<Tensor, Tensor> cross_state_backward(const Tensor& phi_k, const Tensor& v, const Tensor& ds, const Tensor& dz,
                                                const c10::optional<Tensor>& pad) {
    check_half("phi_k", phi_k, 4);
    check_half("v", v, 4);
    const int64_t S = phi_k.size(0), B = phi_k.size(1);
    const int H = (int)phi_k.size(2), K = (int)phi_k.size(3), d = (int)v.size(3);
    check_f32("ds", ds, {B, H, K, d});
    check_f32("dz", dz, {B, H, K});
    Tensor dk = torch::empty_like(phi_k), dv = torch::empty_like(v);
    auto m = mask_bytes(pad, B, S, v);
    Launch l(v);
    check_rc(rfa_cross_state_backward(ptr(phi_k), ptr(v), static_cast<const uint8_t*>(ptr(m)), ds.data_ptr<float>(),
                                      dz.data_ptr<float>(), ptr(dk), ptr(dv), S, B, H, K, d, l.stream));
    return {dk, dv};
}

Tensor cross_readout(const Tensor& phi_q, const Tensor& s, const Tensor& z) {
    check_half("phi_q", phi_q, 4);
    const int64_t T = phi_q.size(0), B = phi_q.size(1);
    const int64_t H = phi_q.size(2), K = phi_q.size(3);
    TORCH_CHECK_VALUE(s.dim() == 4, "s must be [bsz, heads, 2*proj_dim, head_dim]");
    const int64_t d = s.size(3);
    check_f32("s", s, {B, H, K, d});
    check_f32("z", z, {B, H, K});
    Tensor out = torch::empty({T, B, H, d}, phi_q.options());
    Launch l(phi_q);
    check_rc(rfa_cross_readout(ptr(phi_q), s.data_ptr<float>(), z.data_ptr<float>(), ptr(out), T, B * H, (int)K, (int)d,
                               l.stream));
    return out;
}

std::tuple<Tensor, Tensor, Tensor> cross_readout_backward(const Tensor& phi_q, const Tensor& s, const Tensor& z,
                                                          const Tensor& grad_attn) {
    check_half("phi_q", phi_q, 4);
    const int64_t T = phi_q.size(0), B = phi_q.size(1);
    const int64_t H = phi_q.size(2), K = phi_q.size(3);
    TORCH_CHECK_VALUE(s.dim() == 4, "s must be [bsz, heads, 2*proj_dim, head_dim]");
    const int64_t d = s.size(3);
    check_f32("s", s, {B, H, K, d});
    check_f32("z", z, {B, H, K});
    check_half("grad_attn", grad_attn, 4);
    TORCH_CHECK_VALUE(grad_attn.size(0) == T && grad_attn.size(1) == B && grad_attn.size(2) == H && grad_attn.size(3) == d,
                      "grad_attn must be [tgt_len, bsz, heads, head_dim]");
    Tensor dq = torch::empty_like(phi_q), ds = torch::empty_like(s), dz = torch::empty_like(z);
    Launch l(phi_q);
    check_rc(rfa_cross_readout_backward(ptr(phi_q), s.data_ptr<float>(), z.data_ptr<float>(), ptr(grad_attn), ptr(dq),
                                        ds.data_ptr<float>(), dz.data_ptr<float>(), T, B * H, (int)K, (int)d, l.stream));
    return {dq, ds, dz};
}

// ---- incremental decoding -----------------------------------------------------------------
Tensor incremental(const Tensor& phi_q, const Tensor& phi_k, const Tensor& v, const Tensor& s, const Tensor& z,
                   const c10::optional<Tensor>& s_out, const c10::optional<Tensor>& z_out) {
    check_qkv(phi_q, phi_k, v);
    const int64_t steps = phi_q.size(0), N = phi_q.size(1);
    const int64_t K = phi_q.size(2), d = v.size(2);
    check_f32("s", s, {N, K, d});
    check_f32("z", z, {N, K});
    TORCH_CHECK_VALUE(s_out.has_value() == z_out.has_value(), "s_out and z_out go together");
    if (s_out.has_value()) {
        check_f32("s_out", *s_out, {N, K, d});
        check_f32("z_out", *z_out, {N, K});
    }
    Tensor out = torch::empty_like(v);
    Launch l(v);
    check_rc(rfa_incremental_out(ptr(phi_q), ptr(phi_k), ptr(v), s.data_ptr<float>(), z.data_ptr<float>(),
                                 s_out.has_value() ? s_out->data_ptr<float>() : s.data_ptr<float>(),
                                 z_out.has_value() ? z_out->data_ptr<float>() : z.data_ptr<float>(), ptr(out), steps, N,
                                 (int)K, (int)d, l.stream));
    return out;
}

Tensor incremental_fused(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& w, double scale, const Tensor& s,
                         const Tensor& z, const c10::optional<Tensor>& s_out, const c10::optional<Tensor>& z_out) {
    check_half("q", q, 4);
    check_half("k", k, 4);
    check_half("v", v, 4);
    TORCH_CHECK_VALUE(q.sizes() == k.sizes() && q.sizes() == v.sizes(),
                      "q, k, v must have one shape [steps, bsz, heads, head_dim]");
    check_half("random_matrices", w, 3);
    const int64_t steps = q.size(0), B = q.size(1), H = q.size(2), d = q.size(3), D = w.size(1);
    TORCH_CHECK_VALUE(w.size(0) == H && w.size(2) == d, "random_matrices must be [heads, proj_dim, head_dim]");
    check_f32("s", s, {B, H, 2 * D, d});
    check_f32("z", z, {B, H, 2 * D});
    TORCH_CHECK_VALUE(s_out.has_value() == z_out.has_value(), "s_out and z_out go together");
    if (s_out.has_value()) {
        check_f32("s_out", *s_out, {B, H, 2 * D, d});
        check_f32("z_out", *z_out, {B, H, 2 * D});
    }
    Tensor out = torch::empty_like(v);
    Launch l(v);
    check_rc(rfa_incremental_fused_out(ptr(q), ptr(k), ptr(v), ptr(w), (float)scale, s.data_ptr<float>(), z.data_ptr<float>(),
                                       s_out.has_value() ? s_out->data_ptr<float>() : s.data_ptr<float>(),
                                       z_out.has_value() ? z_out->data_ptr<float>() : z.data_ptr<float>(), ptr(out), steps,
                                       B, (int)H, (int)D, (int)d, l.stream));
    return out;
}

Tensor incremental_qkv(const Tensor& qkv, const Tensor& w, double scale, const Tensor& s, const Tensor& z,
                       const c10::optional<Tensor>& s_out, const c10::optional<Tensor>& z_out) {
    check_half("qkv", qkv, 5);
    check_half("random_matrices", w, 3);
    const int64_t steps = qkv.size(0), B = qkv.size(1), H = qkv.size(3), d = qkv.size(4), D = w.size(1);
    TORCH_CHECK_VALUE(qkv.size(2) == 3, "qkv must be [steps, bsz, 3, heads, head_dim]");
    TORCH_CHECK_VALUE(w.size(0) == H && w.size(2) == d, "random_matrices must be [heads, proj_dim, head_dim]");
    check_f32("s", s, {B, H, 2 * D, d});
    check_f32("z", z, {B, H, 2 * D});
    TORCH_CHECK_VALUE(s_out.has_value() == z_out.has_value(), "s_out and z_out go together");
    if (s_out.has_value()) {
        check_f32("s_out", *s_out, {B, H, 2 * D, d});
        check_f32("z_out", *z_out, {B, H, 2 * D});
    }
    Tensor out = torch::empty({steps, B, H, d}, qkv.options());
    Launch l(qkv);
    check_rc(rfa_incremental_qkv(ptr(qkv), ptr(w), (float)scale, s.data_ptr<float>(), z.data_ptr<float>(),
                                 s_out.has_value() ? s_out->data_ptr<float>() : s.data_ptr<float>(),
                                 z_out.has_value() ? z_out->data_ptr<float>() : z.data_ptr<float>(), ptr(out), steps, B,
                                 (int)H, (int)D, (int)d, l.stream));
    return out;
}

// ---- quadratic form with explicit masks -------------------------------------------------------
std::tuple<Tensor, Tensor> masked_forward(const Tensor& phi_q, const Tensor& phi_k, const Tensor& v, int64_t H,
                                          const c10::optional<Tensor>& pad, const c10::optional<Tensor>& attn_mask_bytes) {
    check_qkv(phi_q, phi_k, v);
    const int64_t T = phi_q.size(0), N = phi_q.size(1), K = phi_q.size(2), d = v.size(2);
    TORCH_CHECK_VALUE(H > 0 && N % H == 0, "N=", N, " is not a multiple of heads=", H);
    const int64_t B = N / H, Tp = (T + 63) / 64 * 64;
    Tensor out = torch::empty_like(v);
    Tensor rsum = torch::empty({T, N}, v.options().dtype(torch::kFloat32));
    auto m = mask_bytes(pad, B, T, v);
    if (attn_mask_bytes.has_value())
        TORCH_CHECK_VALUE(attn_mask_bytes->is_cuda() && attn_mask_bytes->scalar_type() == torch::kUInt8 &&
                              attn_mask_bytes->is_contiguous() && attn_mask_bytes->dim() == 2 &&
                              attn_mask_bytes->size(0) == T && attn_mask_bytes->size(1) == Tp,
                          "attn_mask_bytes must come from pack_attn_mask");
    Launch l(v);
    check_rc(rfa_masked_forward(ptr(phi_q), ptr(phi_k), ptr(v), static_cast<const uint8_t*>(ptr(m)),
                                static_cast<const uint8_t*>(ptr(attn_mask_bytes)), ptr(out), rsum.data_ptr<float>(), T, Tp,
                                B, (int)H, (int)K, (int)d, l.stream));
    return {out, rsum};
}

std::vector<Tensor> masked_backward(const Tensor& phi_q, const Tensor& phi_k, const Tensor& v, const Tensor& grad_attn,
                                    const Tensor& out, const Tensor& rsum, int64_t H, const c10::optional<Tensor>& pad,
                                    const c10::optional<Tensor>& attn_mask_bytes,
                                    const c10::optional<Tensor>& attn_mask_t_bytes) {
    check_qkv(phi_q, phi_k, v);
    check_half("grad_attn", grad_attn, 3);
    check_half("out", out, 3);
    const int64_t T = phi_q.size(0), N = phi_q.size(1), K = phi_q.size(2), d = v.size(2);
    TORCH_CHECK_VALUE(H > 0 && N % H == 0, "N=", N, " is not a multiple of heads=", H);
    const int64_t B = N / H, Tp = (T + 63) / 64 * 64;
    TORCH_CHECK_VALUE(grad_attn.sizes() == v.sizes() && out.sizes() == v.sizes(), "grad_attn and out must match v");
    check_f32("rsum", rsum, {T, N});
    Tensor dq = torch::empty_like(phi_q), dk = torch::empty_like(phi_k), dv = torch::empty_like(v);
    auto m = mask_bytes(pad, B, T, v);
    Launch l(v);
    const size_t nbytes = rfa_masked_backward_workspace_bytes(T, N, (int)d);
    Tensor ws = workspace(nbytes, v);
    check_rc(rfa_masked_backward(ptr(phi_q), ptr(phi_k), ptr(v), ptr(grad_attn), ptr(out), rsum.data_ptr<float>(),
                                 static_cast<const uint8_t*>(ptr(m)), static_cast<const uint8_t*>(ptr(attn_mask_bytes)),
                                 static_cast<const uint8_t*>(ptr(attn_mask_t_bytes)), ptr(dq), ptr(dk), ptr(dv), T, Tp, B,
                                 (int)H, (int)K, (int)d, ptr(ws), nbytes, l.stream));
    return {dq, dk, dv};
}

void selftest_layout() {
    c10::hip::HIPGuard guard(c10::hip::current_device());
    check_rc(rfa_selftest_layout(c10::hip::getCurrentHIPStream().stream()));
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.doc() = "PyTorch-ROCm binding of librfa_hip.so (Random Feature Attention kernels for MI355X)";
    namespace py = pybind11;
    m.def("supported", [](int K, int d) { return rfa_shape_supported(K, d) != 0; });
    m.def("feature_map_supported", [](int D, int d) { return rfa_feature_map_supported(D, d) != 0; });
    m.def("selftest_layout", &selftest_layout);
    m.def("forward", &forward, "attn[T, N, d] of causal RFA (rfa_cuda.forward)", py::arg("q"), py::arg("k"), py::arg("v"));
    m.def("backward", &backward, "[grad_q, grad_k, grad_v] of causal RFA (rfa_cuda.backward)", py::arg("q"), py::arg("k"),
          py::arg("v"), py::arg("grad_attn"));
    m.def("prefill", &prefill, py::arg("q"), py::arg("k"), py::arg("v"));
    m.def("forward_save", &forward_save, py::arg("q"), py::arg("k"), py::arg("v"));
    m.def("backward_saved", &backward_saved, py::arg("q"), py::arg("k"), py::arg("v"), py::arg("grad_attn"), py::arg("out"),
          py::arg("saved"));
    m.def("build_random_matrices", &build_random_matrices, py::arg("w"), py::arg("sigma"), py::arg("tau"));
    m.def("build_random_matrices_backward", &build_random_matrices_backward, py::arg("w"), py::arg("sigma"),
          py::arg("grad_out"), py::arg("tau"), py::arg("want_dsigma"), py::arg("want_dw"));
    m.def("feature_map_forward", &feature_map_forward, py::arg("x"), py::arg("w"), py::arg("scale"));
    m.def("feature_map_forward_pair", &feature_map_forward_pair, py::arg("x0"), py::arg("x1"), py::arg("w"), py::arg("scale"));
    m.def("feature_map_backward", &feature_map_backward, py::arg("x"), py::arg("w"), py::arg("grad_phi"), py::arg("scale"),
          py::arg("need_dw") = true);
    m.def("feature_map_backward_pair", &feature_map_backward_pair, py::arg("x0"), py::arg("x1"), py::arg("w"),
          py::arg("grad_phi0"), py::arg("grad_phi1"), py::arg("scale"), py::arg("need_dw") = true);
    m.def("feature_map_backward_pair_packed", &feature_map_backward_pair_packed, py::arg("x0"), py::arg("x1"), py::arg("w"),
          py::arg("grad_phi0"), py::arg("grad_phi1"), py::arg("third"), py::arg("scale"), py::arg("need_dw") = true);
    m.def("project_feature_map", &project_feature_map, py::arg("x"), py::arg("weights"), py::arg("biases"),
          py::arg("want_phi"), py::arg("w"), py::arg("heads"), py::arg("scale"), py::arg("keep_y") = true);
    m.def("linear_weight_grad", &linear_weight_grad, py::arg("x"), py::arg("dys"), py::arg("want_bias"));
    m.def("cross_state", &cross_state, py::arg("phi_k"), py::arg("v"), py::arg("key_padding_mask") = py::none());
    m.def("cross_state_backward", &cross_state_backward, py::arg("phi_k"), py::arg("v"), py::arg("ds"), py::arg("dz"),
          py::arg("key_padding_mask") = py::none());
    m.def("cross_readout", &cross_readout, py::arg("phi_q"), py::arg("s"), py::arg("z"));
    m.def("cross_readout_backward", &cross_readout_backward, py::arg("phi_q"), py::arg("s"), py::arg("z"),
          py::arg("grad_attn"));
    m.def("incremental", &incremental, py::arg("phi_q"), py::arg("phi_k"), py::arg("v"), py::arg("s"), py::arg("z"),
          py::arg("s_out") = py::none(), py::arg("z_out") = py::none());
    m.def("incremental_fused", &incremental_fused, py::arg("q"), py::arg("k"), py::arg("v"), py::arg("w"), py::arg("scale"),
          py::arg("s"), py::arg("z"), py::arg("s_out") = py::none(), py::arg("z_out") = py::none());
    m.def("incremental_qkv", &incremental_qkv, py::arg("qkv"), py::arg("w"), py::arg("scale"), py::arg("s"), py::arg("z"),
          py::arg("s_out") = py::none(), py::arg("z_out") = py::none());
    m.def("masked_forward", &masked_forward, py::arg("phi_q"), py::arg("phi_k"), py::arg("v"), py::arg("H"),
          py::arg("key_padding_mask") = py::none(), py::arg("attn_mask_bytes") = py::none());
    m.def("masked_backward", &masked_backward, py::arg("phi_q"), py::arg("phi_k"), py::arg("v"), py::arg("grad_attn"),
          py::arg("out"), py::arg("rsum"), py::arg("H"), py::arg("key_padding_mask") = py::none(),
          py::arg("attn_mask_bytes") = py::none(), py::arg("attn_mask_t_bytes") = py::none());
}
