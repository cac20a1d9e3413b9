// Fused random-feature map  phi(x) = scale * [sin(W x^), cos(W x^)],  x^ = x / (||x|| + 1e-3)
// and its backward, for gfx950.
//
// Replaces the chain of ATen kernels in random_project / _normalize
// (random_feature_attention/utils.py:100-120: norm, add, div, einsum, sin, cos,
// cat, mul) by one kernel per direction.  The projection W' of one head stays
// resident in LDS while a workgroup streams rows of x through the MFMA.
//
// Layouts:  x   [R, H, DH] fp16   (R = seq_len * bsz rows, row-major)
//           w   [H, D, DH] fp16   (already sigma * W / tau, utils.py:90-97)
//           phi [R, H, 2D] fp16   (sin block in columns [0, D), cos block in [D, 2D))
#pragma once
#include "rfa_common.h"

namespace rfa {

template <int D, int DH>
struct FeatureCfg {
    static_assert(D % 32 == 0 && DH % 64 == 0, "D multiple of 32, DH multiple of 64");
    static constexpr int LDW = DH + lds_pad(DH);
    static constexpr int LDU = D + lds_pad(D);
    // staging rows of phi / grad_phi (2D halves): a stride of 32 bytes mod 256 spreads the
    // 8-byte fragment writes of 16 rows over all banks
    static constexpr int LDP = 2 * D + 16;
    static constexpr int LDG = (2 * D > DH ? 2 * D : DH) + 16;   // backward: grad_phi rows in, dx rows out
    static constexpr size_t kFwdLds = (size_t)(D * LDW + 64 * LDP) * 2;
    static constexpr size_t kBwdLds = (size_t)(D * LDW + 64 * LDW + 64 * LDU + 64 * LDG) * 2;
};

// Orders this wave's earlier LDS writes before its later LDS reads of other lanes' data.  One
// wave executes its LDS instructions in order, so only the compiler has to be stopped from
// moving them; a memory fence here would also wait for every global load and store in flight
// (the next block's prefetch, the previous rows' stores).
__device__ __forceinline__ void wave_lds_order() {
    __builtin_amdgcn_wave_barrier();
    asm volatile("" ::: "memory");
}

// Copy this wave's 16 staged rows (F halves each, row stride ld in LDS) to global rows
// r0 .. r0+15 of a [R, H, F] tensor at head h: every store instruction writes whole rows,
// 16 bytes per lane.
template <int F>
__device__ __forceinline__ void wave_rows_s2g(const half_t* Ss, int ld, half_t* __restrict__ dst, int r0, int R,
                                              int H, int h, int lane) {
    constexpr int PPR = F / 8;        // 16-byte pieces per row
    constexpr int RPI = 64 / PPR;     // rows per instruction
    static_assert(PPR <= 64 && 64 % PPR == 0, "row too long for one wave");
#pragma unroll
    for (int k = 0; k < 16 / RPI; ++k) {
        const int lr = k * RPI + lane / PPR, pc = lane % PPR;
        const uint4 val = *reinterpret_cast<const uint4*>(Ss + lr * ld + pc * 8);
        if (r0 + lr < R) *reinterpret_cast<uint4*>(dst + ((int64_t)(r0 + lr) * H + h) * F + pc * 8) = val;
    }
}

// The reverse, split so that the loads can be issued one row block ahead: global rows
// -> registers (zero beyond R) -> this wave's staging rows.
template <int F>
struct WaveRows {
    static constexpr int PPR = F / 8;
    static constexpr int RPI = 64 / PPR;
    static_assert(PPR <= 64 && 64 % PPR == 0, "row too long for one wave");
    uint4 v[16 / RPI];
};

template <int F>
__device__ __forceinline__ void wave_rows_g2r(WaveRows<F>& rr, const half_t* __restrict__ src, int r0, int R, int H,
                                              int h, int lane) {
    constexpr int PPR = WaveRows<F>::PPR, RPI = WaveRows<F>::RPI;
#pragma unroll
    for (int k = 0; k < 16 / RPI; ++k) {
        const int lr = k * RPI + lane / PPR, pc = lane % PPR;
        // no branch around the load: a row past the end reads the last row and is zeroed afterwards
        const int rc = min(r0 + lr, R - 1);
        rr.v[k] = *reinterpret_cast<const uint4*>(src + ((int64_t)rc * H + h) * F + pc * 8);
        if (r0 + lr >= R) rr.v[k] = make_uint4(0, 0, 0, 0);
    }
}

template <int F>
__device__ __forceinline__ void wave_rows_r2s(const WaveRows<F>& rr, half_t* Ss, int ld, int lane) {
    constexpr int PPR = WaveRows<F>::PPR, RPI = WaveRows<F>::RPI;
#pragma unroll
    for (int k = 0; k < 16 / RPI; ++k) {
        const int lr = k * RPI + lane / PPR, pc = lane % PPR;
        *reinterpret_cast<uint4*>(Ss + lr * ld + pc * 8) = rr.v[k];
    }
}

template <int D, int DH>
__device__ __forceinline__ void load_w_to_lds(half_t* Ws, const half_t* __restrict__ wh, int tid) {
    constexpr int LDW = FeatureCfg<D, DH>::LDW;
    constexpr int PPR = DH / 8;
    for (int p = tid; p < D * PPR; p += kThreads) {
        const int r = p / PPR, c8 = p % PPR;
        *reinterpret_cast<uint4*>(Ws + r * LDW + c8 * 8) = *reinterpret_cast<const uint4*>(wh + r * DH + c8 * 8);
    }
}

// grid = (ceil(R / 64), H, 1 or 2); wave w handles rows [64*bx + 16w, +16).  gridDim.z = 2 maps two
// tensors through the same W' in one launch (q and k of a module): workgroups with
// blockIdx.z = 1 take x1 / phi1.
template <int D, int DH>
__global__ __launch_bounds__(kThreads) void k_feature_map_fwd(
    const half_t* __restrict__ x0, const half_t* __restrict__ w, half_t* __restrict__ phi0,
    const half_t* __restrict__ x1, half_t* __restrict__ phi1, int R, int H, float scale) {
    const bool second = blockIdx.z != 0;
    const half_t* __restrict__ x = second ? x1 : x0;
    half_t* __restrict__ phi = second ? phi1 : phi0;
    using Cfg = FeatureCfg<D, DH>;
    constexpr int LDW = Cfg::LDW, LDP = Cfg::LDP;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    half_t* Ws = reinterpret_cast<half_t*>(smem_raw);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    half_t* Ps = Ws + D * LDW + wv * 16 * LDP;     // this wave's 16 output rows
    const int i = lane & 15, G = lane >> 4;
    const int h = blockIdx.y;
    const int r = blockIdx.x * 64 + 16 * wv + i;

    load_w_to_lds<D, DH>(Ws, w + (int64_t)h * D * DH, tid);

    h8 xb[DH / 32];
    float ss = 0.f;
#pragma unroll
    for (int cs = 0; cs < DH / 32; ++cs) {
        if (r < R) {
            xb[cs] = *reinterpret_cast<const h8*>(x + ((int64_t)r * H + h) * DH + cs * 32 + 8 * G);
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) xb[cs][e] = (half_t)0.f;
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) ss += (float)xb[cs][e] * (float)xb[cs][e];
    }
    ss = sum_over_groups(ss);
    const float inv = rcp_nr(sqrtf(ss) + 1e-3f);
    __syncthreads();

#pragma unroll
    for (int jt = 0; jt < D / 16; ++jt) {
        f4 acc = f4_zero();   // u^T tile (m = feature j, n = row)
#pragma unroll
        for (int cs = 0; cs < DH / 32; ++cs) acc = mfma32(row8(Ws, LDW, 16 * jt + i, cs * 32, G), xb[cs], acc);
        h4 sv, cv;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            float s_, c_;
            fast_sincos(acc[e] * inv, s_, c_);
            sv[e] = (half_t)(scale * s_);
            cv[e] = (half_t)(scale * c_);
        }
        *reinterpret_cast<h4*>(Ps + i * LDP + 16 * jt + 4 * G) = sv;
        *reinterpret_cast<h4*>(Ps + i * LDP + D + 16 * jt + 4 * G) = cv;
    }
    // the fragment layout holds 8 bytes per lane and row: stage through LDS so that the
    // stores to HBM cover whole 4D-byte rows
    wave_lds_order();
    wave_rows_s2g<2 * D>(Ps, LDP, phi, blockIdx.x * 64 + 16 * wv, R, H, h, lane);
}

// Backward.  grid = (nblk, H); workgroup (b, h) walks row blocks b, b+nblk, ...
// of 64 rows, writes dx for them and accumulates its share of
//     dW'[h][j][c] = sum_rows du[row][j] * x^[row][c]
// into dw_part[b][h][j][c] (fp32); k_feature_map_dw_reduce sums the nblk shares.
// With n = ||x||, inv = 1/(n + 1e-3), dus = du * inv, y = dus W':
//     dx = y - x * (x . y) / (n * (n + 1e-3))          (0 where n = 0)
// gridDim.z = 2 differentiates two tensors that went through the same W' in one launch (phi(q) and
// phi(k) of a module): workgroups with blockIdx.z = 1 take x1 / gphi1 / dx1 and the partial
// sums nblk .. 2 nblk - 1, so that the reduction over 2 nblk shares yields the sum of both dW'.
template <int D, int DH>
__global__ __launch_bounds__(kThreads) void k_feature_map_bwd(
    const half_t* __restrict__ x0, const half_t* __restrict__ w, const half_t* __restrict__ gphi0,
    half_t* __restrict__ dx0, const half_t* __restrict__ x1, const half_t* __restrict__ gphi1,
    half_t* __restrict__ dx1, float* __restrict__ dw_part, int R, int H, float scale) {
    const bool second = blockIdx.z != 0;
    const half_t* __restrict__ x = second ? x1 : x0;
    const half_t* __restrict__ gphi = second ? gphi1 : gphi0;
    half_t* __restrict__ dx = second ? dx1 : dx0;
    using Cfg = FeatureCfg<D, DH>;
    constexpr int LDW = Cfg::LDW, LDU = Cfg::LDU, LDG = Cfg::LDG;
    constexpr int NCTW = DH / 64;   // c-tiles of dW owned by one wave
    extern __shared__ __align__(16) unsigned char smem_raw[];
    half_t* Ws = reinterpret_cast<half_t*>(smem_raw);
    half_t* Xs = Ws + D * LDW;
    half_t* Us = Xs + 64 * LDW;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    half_t* Gs = Us + 64 * LDU + wv * 16 * LDG;   // this wave's 16 rows: grad_phi in, dx out
    const int i = lane & 15, G = lane >> 4;
    const int h = blockIdx.y;
    const int lr = 16 * wv + i;          // this lane's row inside a block

    load_w_to_lds<D, DH>(Ws, w + (int64_t)h * D * DH, tid);

    f4 dwacc[NCTW][D / 16];   // (m = c, n = j)
#pragma unroll
    for (int a = 0; a < NCTW; ++a)
#pragma unroll
        for (int b = 0; b < D / 16; ++b) dwacc[a][b] = f4_zero();

    // x rows are loaded straight into MFMA operand form (16 bytes per lane, 64-byte runs);
    // grad_phi rows are loaded whole and re-read from LDS in fragment form
    h8 xn[DH / 32];
    WaveRows<2 * D> gn;
    auto issue_loads = [&](int rb) {
        const int r = rb * 64 + lr;
#pragma unroll
        for (int cs = 0; cs < DH / 32; ++cs) {
            xn[cs] = *reinterpret_cast<const h8*>(x + ((int64_t)min(r, R - 1) * H + h) * DH + cs * 32 + 8 * G);
            if (r >= R) {
#pragma unroll
                for (int e = 0; e < 8; ++e) xn[cs][e] = (half_t)0.f;
            }
        }
        wave_rows_g2r<2 * D>(gn, gphi, rb * 64 + 16 * wv, R, H, h, lane);
    };

    const int nrb = (R + 63) / 64;
    if ((int)blockIdx.x < nrb) issue_loads(blockIdx.x);
    for (int rb = blockIdx.x; rb < nrb; rb += gridDim.x) {
        const int r0 = rb * 64 + 16 * wv;    // first row of this wave
        h8 xb[DH / 32];
        float ss = 0.f;
#pragma unroll
        for (int cs = 0; cs < DH / 32; ++cs) {
            xb[cs] = xn[cs];
            *reinterpret_cast<h8*>(Xs + lr * LDW + cs * 32 + 8 * G) = xb[cs];
#pragma unroll
            for (int e = 0; e < 8; ++e) ss += (float)xb[cs][e] * (float)xb[cs][e];
        }
        wave_rows_r2s<2 * D>(gn, Gs, LDG, lane);
        ss = sum_over_groups(ss);
        const float nrm = sqrtf(ss);
        const float inv = 1.0f / (nrm + 1e-3f);
        const float coef = nrm > 0.f ? inv / nrm : 0.f;
        __syncthreads();   // Ws (first pass), Xs, Gs visible; previous block's dW reads done
        if (rb + (int)gridDim.x < nrb) issue_loads(rb + gridDim.x);

#pragma unroll
        for (int jt = 0; jt < D / 16; ++jt) {
            f4 acc = f4_zero();
#pragma unroll
            for (int cs = 0; cs < DH / 32; ++cs) acc = mfma32(row8(Ws, LDW, 16 * jt + i, cs * 32, G), xb[cs], acc);
            const h4 gs = *reinterpret_cast<const h4*>(Gs + i * LDG + 16 * jt + 4 * G);
            const h4 gc = *reinterpret_cast<const h4*>(Gs + i * LDG + D + 16 * jt + 4 * G);
            h4 du;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float s_, c_;
                fast_sincos(acc[e] * inv, s_, c_);
                du[e] = (half_t)(scale * (c_ * (float)gs[e] - s_ * (float)gc[e]) * inv);
            }
            *reinterpret_cast<h4*>(Us + lr * LDU + 16 * jt + 4 * G) = du;
        }
        __syncthreads();   // Us complete

        // y^T tiles (m = c, n = row) for this wave's 16 rows
        f4 y[DH / 16];
        float xdot = 0.f;
#pragma unroll
        for (int ct = 0; ct < DH / 16; ++ct) {
            f4 acc = f4_zero();
#pragma unroll
            for (int js = 0; js < D / 32; ++js)
                acc = mfma32(col8(Ws, LDW, js * 32, 16 * ct, lane), row8(Us, LDU, lr, js * 32, G), acc);
            y[ct] = acc;
            h4 xv = *reinterpret_cast<const h4*>(Xs + lr * LDW + 16 * ct + 4 * G);
#pragma unroll
            for (int e = 0; e < 4; ++e) xdot += acc[e] * (float)xv[e];
        }
        xdot = sum_over_groups(xdot) * coef;
        // dx rows: fragment layout -> this wave's staging rows -> whole-row stores
#pragma unroll
        for (int ct = 0; ct < DH / 16; ++ct) {
            h4 xv = *reinterpret_cast<const h4*>(Xs + lr * LDW + 16 * ct + 4 * G);
            h4 o;
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = (half_t)(y[ct][e] - (float)xv[e] * xdot);
            *reinterpret_cast<h4*>(Gs + i * LDG + 16 * ct + 4 * G) = o;
        }
        wave_lds_order();
        wave_rows_s2g<DH>(Gs, LDG, dx, r0, R, H, h, lane);

        // dW (m = c, n = j) += X^T Us over the 64 rows of the block
#pragma unroll
        for (int rs = 0; rs < 2; ++rs) {
            h8 xa[NCTW];
#pragma unroll
            for (int a = 0; a < NCTW; ++a) xa[a] = col8(Xs, LDW, rs * 32, 16 * (wv * NCTW + a), lane);
#pragma unroll
            for (int jt = 0; jt < D / 16; ++jt) {
                h8 ub = col8(Us, LDU, rs * 32, 16 * jt, lane);
#pragma unroll
                for (int a = 0; a < NCTW; ++a) dwacc[a][jt] = mfma32(xa[a], ub, dwacc[a][jt]);
            }
        }
        __syncthreads();   // all reads of Xs / Us / Gs done before the next block overwrites them
    }

    float* po = dw_part + ((int64_t)(blockIdx.z * gridDim.x + blockIdx.x) * H + h) * D * DH;
#pragma unroll
    for (int a = 0; a < NCTW; ++a)
#pragma unroll
        for (int jt = 0; jt < D / 16; ++jt)
            *reinterpret_cast<f4*>(po + (16 * jt + i) * DH + 16 * (wv * NCTW + a) + 4 * G) = dwacc[a][jt];
}

// dw[e] = sum_b dw_part[b][e].  One workgroup of 4 waves per 256 consecutive elements
// (64 lanes x 16 bytes); wave p sums the shares b = p, p+4, ... with all its loads in
// flight at once, then the 4 waves are added through LDS.  elems % 256 == 0.
__global__ __launch_bounds__(kThreads) void k_feature_map_dw_reduce(const float* __restrict__ part,
                                                                    float* __restrict__ dw, int nblk,
                                                                    int64_t elems) {
    __shared__ f4 red[3][64];
    const int lane = threadIdx.x & 63, p = threadIdx.x >> 6;
    const int64_t e = ((int64_t)blockIdx.x * 64 + lane) * 4;
    f4 acc = f4_zero();
    int b = p;
    for (; b + 28 < nblk; b += 32) {
        f4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = *reinterpret_cast<const f4*>(part + (int64_t)(b + 4 * u) * elems + e);
#pragma unroll
        for (int u = 0; u < 8; ++u) acc += v[u];
    }
    for (; b < nblk; b += 4) acc += *reinterpret_cast<const f4*>(part + (int64_t)b * elems + e);
    if (p > 0) red[p - 1][lane] = acc;
    __syncthreads();
    if (p == 0) {
        acc += red[0][lane];
        acc += red[1][lane];
        acc += red[2][lane];
        *reinterpret_cast<f4*>(dw + e) = acc;
    }
}

// W' = (sigma * W if sigma) / tau, one element per thread, in the reference's own arithmetic
// (utils.py:90-97 on fp16 tensors: the product is rounded to fp16, then divided by tau in
// fp32 and rounded again).  w, out: [H, D, d]; sigma: [H, d] (broadcast over D) or NULL.
__global__ __launch_bounds__(kThreads) void k_build_random_matrices(const half_t* __restrict__ w,
                                                                    const half_t* __restrict__ sigma,
                                                                    half_t* __restrict__ out, float tau, int D,
                                                                    int d, int64_t total) {
    const int64_t e = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (e >= total) return;
    half_t t = w[e];
    if (sigma) t = (half_t)((float)sigma[(e / ((int64_t)D * d)) * d + e % d] * (float)t);
    out[e] = (half_t)((float)t / tau);
}

// Gradient of k_build_random_matrices as autograd forms it from the same fp16 operations, with
// t = fp16(g / tau):  dw = fp16(t * sigma) (t itself without sigma), one element per thread.
__global__ __launch_bounds__(kThreads) void k_build_random_matrices_dw(const half_t* __restrict__ sigma,
                                                                       const half_t* __restrict__ g,
                                                                       half_t* __restrict__ dw, float tau, int D,
                                                                       int d, int64_t total) {
    const int64_t e = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (e >= total) return;
    const half_t t = (half_t)((float)g[e] / tau);
    dw[e] = sigma ? (half_t)((float)t * (float)sigma[(e / ((int64_t)D * d)) * d + e % d]) : t;
}

// dsigma[h][c] = fp16(sum_j fp16(t[h][j][c] * w[h][j][c])), fp32 sum.  One workgroup per head:
// 64 columns at a time, the D rows dealt to the 4 waves, the 4 partial sums added in wave order.
__global__ __launch_bounds__(kThreads) void k_build_random_matrices_dsigma(const half_t* __restrict__ w,
                                                                           const half_t* __restrict__ g,
                                                                           half_t* __restrict__ dsigma, float tau,
                                                                           int D, int d) {
    __shared__ float red[4][64];
    const int h = blockIdx.x, lane = threadIdx.x & 63, slice = threadIdx.x >> 6;
    const half_t* wh = w + (int64_t)h * D * d;
    const half_t* gh = g + (int64_t)h * D * d;
    for (int c0 = 0; c0 < d; c0 += 64) {
        const int c = c0 + lane;
        float acc = 0.f;
        if (c < d) {
            // the kernel is one memory round trip after another: request the rows of a whole group (16 rows
            // of g and of w per thread) before the first is used, so that D = 64 takes one trip
            for (int j0 = slice; j0 < D; j0 += 64) {
                half_t gv[16], wv[16];
#pragma unroll
                for (int u = 0; u < 16; ++u) {
                    const int j = min(j0 + 4 * u, D - 1);
                    gv[u] = gh[j * d + c];
                    wv[u] = wh[j * d + c];
                }
#pragma unroll
                for (int u = 0; u < 16; ++u) {
                    if (j0 + 4 * u < D) {
                        const half_t t = (half_t)((float)gv[u] / tau);
                        acc += (float)(half_t)((float)t * (float)wv[u]);
                    }
                }
            }
        }
        red[slice][lane] = acc;
        __syncthreads();
        if (slice == 0 && c < d)
            dsigma[(int64_t)h * d + c] = (half_t)(((red[0][lane] + red[1][lane]) + red[2][lane]) + red[3][lane]);
        __syncthreads();
    }
}

}  // namespace rfa
