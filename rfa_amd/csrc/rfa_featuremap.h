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
    static constexpr size_t kFwdLds = (size_t)D * LDW * 2;
    static constexpr size_t kBwdLds = (size_t)(D * LDW + 64 * LDW + 64 * LDU) * 2;
};

template <int D, int DH>
__device__ __forceinline__ void load_w_to_lds(half_t* Ws, const half_t* __restrict__ wh, int tid) {
    constexpr int LDW = FeatureCfg<D, DH>::LDW;
    constexpr int PPR = DH / 8;
    for (int p = tid; p < D * PPR; p += kThreads) {
        const int r = p / PPR, c8 = p % PPR;
        *reinterpret_cast<uint4*>(Ws + r * LDW + c8 * 8) = *reinterpret_cast<const uint4*>(wh + r * DH + c8 * 8);
    }
}

// grid = (ceil(R / 64), H); wave w handles rows [64*bx + 16w, +16).
template <int D, int DH>
__global__ __launch_bounds__(kThreads) void k_feature_map_fwd(
    const half_t* __restrict__ x, const half_t* __restrict__ w, half_t* __restrict__ phi, int R, int H,
    float scale) {
    using Cfg = FeatureCfg<D, DH>;
    constexpr int LDW = Cfg::LDW;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    half_t* Ws = reinterpret_cast<half_t*>(smem_raw);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
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
    const float inv = 1.0f / (sqrtf(ss) + 1e-3f);
    __syncthreads();

    half_t* po = phi + ((int64_t)r * H + h) * (2 * D);
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
        if (r < R) {
            *reinterpret_cast<h4*>(po + 16 * jt + 4 * G) = sv;
            *reinterpret_cast<h4*>(po + D + 16 * jt + 4 * G) = cv;
        }
    }
}

// Backward.  grid = (nblk, H); workgroup (b, h) walks row blocks b, b+nblk, ...
// of 64 rows, writes dx for them and accumulates its share of
//     dW'[h][j][c] = sum_rows du[row][j] * x^[row][c]
// into dw_part[b][h][j][c] (fp32); k_feature_map_dw_reduce sums the nblk shares.
// With n = ||x||, inv = 1/(n + 1e-3), dus = du * inv, y = dus W':
//     dx = y - x * (x . y) / (n * (n + 1e-3))          (0 where n = 0)
template <int D, int DH>
__global__ __launch_bounds__(kThreads) void k_feature_map_bwd(
    const half_t* __restrict__ x, const half_t* __restrict__ w, const half_t* __restrict__ gphi,
    half_t* __restrict__ dx, float* __restrict__ dw_part, int R, int H, float scale) {
    using Cfg = FeatureCfg<D, DH>;
    constexpr int LDW = Cfg::LDW, LDU = Cfg::LDU;
    constexpr int NCTW = DH / 64;   // c-tiles of dW owned by one wave
    extern __shared__ __align__(16) unsigned char smem_raw[];
    half_t* Ws = reinterpret_cast<half_t*>(smem_raw);
    half_t* Xs = Ws + D * LDW;
    half_t* Us = Xs + 64 * LDW;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int i = lane & 15, G = lane >> 4;
    const int h = blockIdx.y;

    load_w_to_lds<D, DH>(Ws, w + (int64_t)h * D * DH, tid);

    f4 dwacc[NCTW][D / 16];   // (m = c, n = j)
#pragma unroll
    for (int a = 0; a < NCTW; ++a)
#pragma unroll
        for (int b = 0; b < D / 16; ++b) dwacc[a][b] = f4_zero();

    const int nrb = (R + 63) / 64;
    for (int rb = blockIdx.x; rb < nrb; rb += gridDim.x) {
        const int lr = 16 * wv + i;          // row inside the block
        const int r = rb * 64 + lr;
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
            *reinterpret_cast<h8*>(Xs + lr * LDW + cs * 32 + 8 * G) = xb[cs];
#pragma unroll
            for (int e = 0; e < 8; ++e) ss += (float)xb[cs][e] * (float)xb[cs][e];
        }
        ss = sum_over_groups(ss);
        const float nrm = sqrtf(ss);
        const float inv = 1.0f / (nrm + 1e-3f);
        const float coef = nrm > 0.f ? inv / nrm : 0.f;
        __syncthreads();   // Ws (first pass), Xs visible; previous block's dW reads done

        const half_t* gp = gphi + ((int64_t)r * H + h) * (2 * D);
#pragma unroll
        for (int jt = 0; jt < D / 16; ++jt) {
            f4 acc = f4_zero();
#pragma unroll
            for (int cs = 0; cs < DH / 32; ++cs) acc = mfma32(row8(Ws, LDW, 16 * jt + i, cs * 32, G), xb[cs], acc);
            h4 gs = h4_zero(), gc = h4_zero();
            if (r < R) {
                gs = *reinterpret_cast<const h4*>(gp + 16 * jt + 4 * G);
                gc = *reinterpret_cast<const h4*>(gp + D + 16 * jt + 4 * G);
            }
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
        if (r < R) {
            half_t* dxo = dx + ((int64_t)r * H + h) * DH;
#pragma unroll
            for (int ct = 0; ct < DH / 16; ++ct) {
                h4 xv = *reinterpret_cast<const h4*>(Xs + lr * LDW + 16 * ct + 4 * G);
                h4 o;
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = (half_t)(y[ct][e] - (float)xv[e] * xdot);
                *reinterpret_cast<h4*>(dxo + 16 * ct + 4 * G) = o;
            }
        }

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
        __syncthreads();   // all reads of Xs / Us done before the next block overwrites them
    }

    float* po = dw_part + ((int64_t)blockIdx.x * H + h) * D * DH;
#pragma unroll
    for (int a = 0; a < NCTW; ++a)
#pragma unroll
        for (int jt = 0; jt < D / 16; ++jt)
            *reinterpret_cast<f4*>(po + (16 * jt + i) * DH + 16 * (wv * NCTW + a) + 4 * G) = dwacc[a][jt];
}

// dw[e] = sum_b dw_part[b][e]
__global__ void k_feature_map_dw_reduce(const float* __restrict__ part, float* __restrict__ dw, int nblk,
                                        int64_t elems) {
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= elems) return;
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;   // independent chains: the loads overlap
    int b = 0;
    for (; b + 4 <= nblk; b += 4) {
        s0 += part[(int64_t)b * elems + e];
        s1 += part[(int64_t)(b + 1) * elems + e];
        s2 += part[(int64_t)(b + 2) * elems + e];
        s3 += part[(int64_t)(b + 3) * elems + e];
    }
    for (; b < nblk; ++b) s0 += part[(int64_t)b * elems + e];
    dw[e] = (s0 + s1) + (s2 + s3);
}

}  // namespace rfa
