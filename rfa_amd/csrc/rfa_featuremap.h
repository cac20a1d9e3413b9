// Fused random-feature map  phi(x) = scale * [sin(W x^), cos(W x^)],  x^ = x / (||x|| + 1e-3)
// and its backward, for gfx950.
//
// Replaces the chain of ATen kernels in random_project / _normalize
// (random_feature_attention/utils.py:100-120: norm, add, div, einsum, sin, cos,
// cat, mul) by one kernel per direction.  The projection W' of one head stays
// resident in LDS while a workgroup streams rows of x through the MFMA.
//
// Two forms.  Streaming (k_feature_map_fwd, k_feature_map_bwd_stream): every wave walks its own
// groups of 16 rows, rows move between registers and global memory in the lanes' own operand
// positions, no workgroup barrier in the row loop; the backward needs dW'[D][DH] of a head in one
// wave's accumulators (D * DH <= 4096).  Row blocks (k_feature_map_bwd, the other shapes): four
// waves share blocks of 64 rows through LDS and split dW' between them.
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
    static constexpr size_t kFwdLds = (size_t)(D * LDW) * 2;                                     // W' only
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

// Same, for a destination whose rows lie `rs` halves apart: dst points at this head's first column.
template <int F>
__device__ __forceinline__ void wave_rows_s2g_strided(const half_t* Ss, int ld, half_t* __restrict__ dst, int64_t rs,
                                                      int r0, int R, int lane) {
    constexpr int PPR = F / 8, RPI = 64 / PPR;
    static_assert(PPR <= 64 && 64 % PPR == 0, "row too long for one wave");
#pragma unroll
    for (int k = 0; k < 16 / RPI; ++k) {
        const int lr = k * RPI + lane / PPR, pc = lane % PPR;
        const uint4 val = *reinterpret_cast<const uint4*>(Ss + lr * ld + pc * 8);
        if (r0 + lr < R) *reinterpret_cast<uint4*>(dst + (int64_t)(r0 + lr) * rs + pc * 8) = val;
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

// ---- streaming kernels: waves that never wait for each other ---------------------------------
// A wave owns groups of 16 rows of one head and walks them with a stride; W' sits in LDS, read
// only.  Nothing a wave writes is read by another wave, so the row loop has no workgroup barrier.
//
// "Pair order": MFMA tile t of 16 features (or of 16 input columns) is made of the indices
//     32 (t / 2) + 8 G + 4 (t % 2) + e        at accumulator position m = 4 G + e,
// so that the accumulators of tiles 2p and 2p+1 together give lane (i, G) the 8 consecutive
// indices 32 p + 8 G .. + 7 of row i: 16 bytes that go to (and come from) global memory
// directly, without a pass through LDS to re-form rows.  pair_pos(f) (rfa_common.h) is the row of
// the operand matrix that holds index f.
constexpr int kFeatureWaves = 8;
constexpr int kFeatureThreads = 64 * kFeatureWaves;


// W' of one head -> LDS with its rows (features) in pair order
template <int D, int DH, int NT = kFeatureThreads>
__device__ __forceinline__ void load_w_pair_order(half_t* Ws, const half_t* __restrict__ wh, int tid) {
    constexpr int LDW = FeatureCfg<D, DH>::LDW;
    constexpr int PPR = DH / 8;
    for (int p = tid; p < D * PPR; p += NT) {
        const int r = p / PPR, c8 = p % PPR;
        *reinterpret_cast<uint4*>(Ws + pair_pos(r) * LDW + c8 * 8) = *reinterpret_cast<const uint4*>(wh + r * DH + c8 * 8);
    }
}

// grid = (nblk, H, 1 or 2); wave w of workgroup b takes the row groups 8 b + w, + 8 nblk, ...
// gridDim.z = 2 maps two tensors through the same W' in one launch (q and k of a module):
// workgroups with blockIdx.z = 1 take x1 / phi1.
template <int D, int DH>
__global__ __launch_bounds__(kFeatureThreads) void k_feature_map_fwd(
    const half_t* __restrict__ x0, const half_t* __restrict__ w, half_t* __restrict__ phi0,
    const half_t* __restrict__ x1, half_t* __restrict__ phi1, int R, int H, float scale) {
    const bool second = blockIdx.z != 0;
    const half_t* __restrict__ x = second ? x1 : x0;
    half_t* __restrict__ phi = second ? phi1 : phi0;
    constexpr int LDW = FeatureCfg<D, DH>::LDW;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    half_t* Ws = reinterpret_cast<half_t*>(smem_raw);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int i = lane & 15, G = lane >> 4;
    const int h = blockIdx.y;

    load_w_pair_order<D, DH>(Ws, w + (int64_t)h * D * DH, tid);

    const int ngrp = (R + 15) / 16, gstride = gridDim.x * kFeatureWaves;
    int grp = blockIdx.x * kFeatureWaves + wv;
    // Two sets of row registers: the loads of the next group are issued into the set the
    // current group does not use, so no set is ever copied (a third set, two groups in flight,
    // measured no faster).  Rows past R read the last row (no branch around the loads) and are
    // not stored.
    struct Rows { h8 x[DH / 32]; };
    auto issue_loads = [&](Rows& t, int g) {
        const half_t* px = x + ((int64_t)min(g * 16 + i, R - 1) * H + h) * DH + 8 * G;
#pragma unroll
        for (int cs = 0; cs < DH / 32; ++cs) t.x[cs] = *reinterpret_cast<const h8*>(px + cs * 32);
    };
    auto process = [&](const Rows& t, int g) {
        const int r = g * 16 + i;
        float ss = 0.f;
#pragma unroll
        for (int cs = 0; cs < DH / 32; ++cs) ss += dot_h8(__builtin_bit_cast(uint4, t.x[cs]), __builtin_bit_cast(uint4, t.x[cs]));
        ss = sum_over_groups(ss);
        const float inv_turns = rcp_nr(__builtin_amdgcn_sqrtf(ss) + 1e-3f) * 0.15915494309189535f;
        half_t* po = phi + ((int64_t)r * H + h) * (2 * D) + 8 * G;
#pragma unroll
        for (int p = 0; p < D / 32; ++p) {
            f4 acc[2] = {f4_zero(), f4_zero()};   // u^T tiles 2p, 2p+1 (m = feature, n = row)
#pragma unroll
            for (int q = 0; q < 2; ++q)
#pragma unroll
                for (int cs = 0; cs < DH / 32; ++cs)
                    acc[q] = mfma32(row8(Ws, LDW, 32 * p + 16 * q + i, cs * 32, G), t.x[cs], acc[q]);
            h8 sv, cv;
#pragma unroll
            for (int q = 0; q < 2; ++q)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float s_, c_;
                    sincos_turns(acc[q][e] * inv_turns, s_, c_);
                    sv[4 * q + e] = (half_t)(scale * s_);
                    cv[4 * q + e] = (half_t)(scale * c_);
                }
            if (r < R) {
                *reinterpret_cast<h8*>(po + 32 * p) = sv;
                *reinterpret_cast<h8*>(po + D + 32 * p) = cv;
            }
        }
    };
    Rows ra, rb;
    if (grp < ngrp) issue_loads(ra, grp);
    __syncthreads();   // W' in place
    while (grp < ngrp) {
        if (grp + gstride < ngrp) issue_loads(rb, grp + gstride);
        process(ra, grp);
        if ((grp += gstride) >= ngrp) break;
        if (grp + gstride < ngrp) issue_loads(ra, grp + gstride);
        process(rb, grp);
        grp += gstride;
    }
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
// The rows of dx lie dx_rs halves apart (H * DH for a tensor of its own).
template <int D, int DH>
__global__ __launch_bounds__(kThreads) void k_feature_map_bwd(
    const half_t* __restrict__ x0, const half_t* __restrict__ w, const half_t* __restrict__ gphi0,
    half_t* __restrict__ dx0, const half_t* __restrict__ x1, const half_t* __restrict__ gphi1,
    half_t* __restrict__ dx1, float* __restrict__ dw_part, int R, int H, float scale, int64_t dx_rs) {
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
        wave_rows_s2g_strided<DH>(Gs, LDG, dx + h * DH, dx_rs, r0, R, lane);

        // dW (m = c, n = j) += X^T Us over the 64 rows of the block
#pragma unroll
        for (int rs = 0; rs < (dw_part ? 2 : 0); ++rs) {
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

    if (!dw_part) return;      // dx only
    float* po = dw_part + ((int64_t)(blockIdx.z * gridDim.x + blockIdx.x) * H + h) * D * DH;
#pragma unroll
    for (int a = 0; a < NCTW; ++a)
#pragma unroll
        for (int jt = 0; jt < D / 16; ++jt)
            *reinterpret_cast<f4*>(po + (16 * jt + i) * DH + 16 * (wv * NCTW + a) + 4 * G) = dwacc[a][jt];
}

// LDS of the streaming backward: W' twice (rows in pair order for u = W' x; transposed, with the
// input columns in pair order, for y = du W'), per wave 16 rows of x and of du for the
// transposing reads of the dW product, and after the row loop the same bytes again as the
// area through which the eight waves exchange their dW (one copy of dW'[D][DH] per wave).
#ifndef RFA_FEATURE_BWD_WAVES
#define RFA_FEATURE_BWD_WAVES 8
#endif
constexpr int kFeatureBwdWaves = RFA_FEATURE_BWD_WAVES;
constexpr int kFeatureBwdThreads = 64 * kFeatureBwdWaves;

template <int D, int DH>
struct FeatureStreamCfg {
    static constexpr int LDW = DH + lds_pad(DH), LDT = D + lds_pad(D);
    // a row stride of 32 bytes mod 256 spreads the 8-byte pieces of a transposing read over all banks
    static constexpr int LDX = DH + 16, LDU = D + 16;
    static constexpr int kTiles = (DH / 16) * (D / 16);
    // the whole dW'[D][DH] of a head sits in the accumulators of every wave: 4 registers per tile
    static constexpr bool kFits = D * DH <= 4096;
    static constexpr size_t kLoop = (size_t)(D * LDW + DH * LDT + kFeatureBwdWaves * 16 * (LDX + LDU)) * 2;
    static constexpr size_t kReduce = (size_t)kFeatureBwdWaves * D * DH * 4;
    static constexpr size_t kLds = kLoop > kReduce ? kLoop : kReduce;
};

__device__ __forceinline__ f4 mfma16(h4 a, h4 b, f4 c) { return __builtin_amdgcn_mfma_f32_16x16x16f16(a, b, c, 0, 0, 0); }

// Backward of the feature map, streaming form (shapes with D * DH <= 4096).  grid = (nblk, H,
// 1 or 2) like the forward; wave w of workgroup b takes the row groups 8 b + w, + 8 nblk, ...
// Per group of 16 rows, with n = ||x||, inv = 1 / (n + 1e-3), u = W' x inv:
//     du  = scale (cos u * g_sin - sin u * g_cos) inv          accumulators of u, in registers
//     y   = du W'                                               du is the MFMA operand as it stands
//     dx  = y - x (x . y) / (n (n + 1e-3))   (0 where n = 0)    16 bytes per lane, stored directly
//     dW' += du^T x                                             over the wave's own 16 rows (k = 16 MFMA),
//                                                               operands by transposing LDS reads
// x and grad_phi arrive in the lane's own operand / accumulator positions (pair order), so no
// row is re-formed in LDS and no wave reads what another wrote: no workgroup barrier in the row
// loop.  At the end the eight waves add their dW' through LDS (one exchange, every wave sums and
// stores an eighth of the tiles) and the workgroup leaves one partial sum,
// dw_part[(z nblk + b)][h]; k_feature_map_dw_reduce sums the shares.
template <int D, int DH>
__global__ __launch_bounds__(kFeatureBwdThreads) void k_feature_map_bwd_stream(
    const half_t* __restrict__ x0, const half_t* __restrict__ w, const half_t* __restrict__ gphi0,
    half_t* __restrict__ dx0, const half_t* __restrict__ x1, const half_t* __restrict__ gphi1,
    half_t* __restrict__ dx1, float* __restrict__ dw_part, int R, int H, float scale, int64_t dx_rs,
    const half_t* __restrict__ copy_src, half_t* __restrict__ copy_dst) {
    if (blockIdx.z == 2) {
        // third job of a launch that fills a packed gradient: rows of copy_src [R, H, DH] -> rows of
        // copy_dst, dx_rs halves apart (this workgroup: head blockIdx.y, its waves' row groups)
        constexpr int PPR = DH / 8, RPI = 64 / PPR;
        const int lane = threadIdx.x & 63, h = blockIdx.y;
        const int ngrp = (R + 15) / 16;
        for (int g = blockIdx.x * kFeatureBwdWaves + (threadIdx.x >> 6); g < ngrp; g += gridDim.x * kFeatureBwdWaves) {
#pragma unroll
            for (int k = 0; k < 16 / RPI; ++k) {
                const int r = g * 16 + k * RPI + lane / PPR, pc = lane % PPR;
                if (r < R)
                    *reinterpret_cast<uint4*>(copy_dst + (int64_t)r * dx_rs + h * DH + pc * 8) =
                        *reinterpret_cast<const uint4*>(copy_src + ((int64_t)r * H + h) * DH + pc * 8);
            }
        }
        return;
    }
    const bool second = blockIdx.z != 0;
    const half_t* __restrict__ x = second ? x1 : x0;
    const half_t* __restrict__ gphi = second ? gphi1 : gphi0;
    half_t* __restrict__ dx = second ? dx1 : dx0;
    using Cfg = FeatureStreamCfg<D, DH>;
    static_assert(Cfg::kFits, "dW' of one head must fit the accumulators of a wave");
    constexpr int LDW = Cfg::LDW, LDT = Cfg::LDT, LDX = Cfg::LDX, LDU = Cfg::LDU;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    half_t* Ws = reinterpret_cast<half_t*>(smem_raw);
    half_t* WT = Ws + D * LDW;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    half_t* Xs = WT + DH * LDT + wv * 16 * (LDX + LDU);
    half_t* Us = Xs + 16 * LDX;
    const int i = lane & 15, G = lane >> 4;
    const int h = blockIdx.y;
    const half_t* wh = w + (int64_t)h * D * DH;

    load_w_pair_order<D, DH, kFeatureBwdThreads>(Ws, wh, tid);
    for (int p = tid; p < D * DH / 8; p += kFeatureBwdThreads) {
        const int j = p / (DH / 8), c8 = p % (DH / 8);
        const h8 v = *reinterpret_cast<const h8*>(wh + j * DH + c8 * 8);
#pragma unroll
        for (int e = 0; e < 8; ++e) WT[pair_pos(c8 * 8 + e) * LDT + j] = v[e];
    }

    f4 dwacc[DH / 16][D / 16];   // (m = c, n = j)
#pragma unroll
    for (int a = 0; a < DH / 16; ++a)
#pragma unroll
        for (int b = 0; b < D / 16; ++b) dwacc[a][b] = f4_zero();

    const int ngrp = (R + 15) / 16, gstride = gridDim.x * kFeatureBwdWaves;
    int grp = blockIdx.x * kFeatureBwdWaves + wv;
    // Two sets of row registers: the loads of the next group are issued into the set the
    // current group does not use, so no set is ever copied.  Rows past R read the last row (no
    // branch around the loads); their du is forced to 0, which keeps them out of dW', and their
    // dx is not stored.
    struct Rows { h8 x[DH / 32], gs[D / 32], gc[D / 32]; };
    auto issue_loads = [&](Rows& t, int g) {
        const int64_t row = (int64_t)min(g * 16 + i, R - 1) * H + h;
        const half_t* px = x + row * DH + 8 * G;
        const half_t* pg = gphi + row * (2 * D) + 8 * G;
#pragma unroll
        for (int cs = 0; cs < DH / 32; ++cs) t.x[cs] = *reinterpret_cast<const h8*>(px + cs * 32);
#pragma unroll
        for (int p = 0; p < D / 32; ++p) {
            t.gs[p] = *reinterpret_cast<const h8*>(pg + 32 * p);
            t.gc[p] = *reinterpret_cast<const h8*>(pg + D + 32 * p);
        }
    };
    const int trow = 4 * G + (i >> 2), tcol = 4 * (i & 3);    // this lane's address in a transposing read
    const bool want_dw = dw_part != nullptr;                  // no partial sums asked for: dx only
    auto process = [&](const Rows& t, int g) {
        const int r = g * 16 + i;
        float ss = 0.f;
#pragma unroll
        for (int cs = 0; cs < DH / 32; ++cs) {
            if (want_dw) *reinterpret_cast<h8*>(Xs + i * LDX + cs * 32 + 8 * G) = t.x[cs];
            ss += dot_h8(__builtin_bit_cast(uint4, t.x[cs]), __builtin_bit_cast(uint4, t.x[cs]));
        }
        ss = sum_over_groups(ss);
        const float nrm = __builtin_amdgcn_sqrtf(ss);
        const float inv = rcp_nr(nrm + 1e-3f);
        const float coef = nrm > 0.f ? inv * rcp_nr(nrm) : 0.f;
        const float inv_turns = inv * 0.15915494309189535f;
        const float sinv = r < R ? scale * inv : 0.f;

        h8 du[D / 32];
#pragma unroll
        for (int p = 0; p < D / 32; ++p) {
            f4 acc[2] = {f4_zero(), f4_zero()};   // u^T tiles 2p, 2p+1 (m = feature, n = row)
#pragma unroll
            for (int q = 0; q < 2; ++q)
#pragma unroll
                for (int cs = 0; cs < DH / 32; ++cs)
                    acc[q] = mfma32(row8(Ws, LDW, 32 * p + 16 * q + i, cs * 32, G), t.x[cs], acc[q]);
#pragma unroll
            for (int q = 0; q < 2; ++q)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float s_, c_;
                    sincos_turns(acc[q][e] * inv_turns, s_, c_);
                    du[p][4 * q + e] = (half_t)(sinv * (c_ * (float)t.gs[p][4 * q + e] - s_ * (float)t.gc[p][4 * q + e]));
                }
            if (want_dw) *reinterpret_cast<h8*>(Us + i * LDU + 32 * p + 8 * G) = du[p];
        }

        // y^T tiles (m = input column in pair order, n = row)
        f4 y[DH / 16];
        float xdot = 0.f;
#pragma unroll
        for (int ct = 0; ct < DH / 16; ++ct) {
            f4 acc = f4_zero();
#pragma unroll
            for (int p = 0; p < D / 32; ++p) acc = mfma32(row8(WT, LDT, 16 * ct + i, 32 * p, G), du[p], acc);
            y[ct] = acc;
#pragma unroll
            for (int e = 0; e < 4; ++e) xdot += acc[e] * (float)t.x[ct / 2][4 * (ct % 2) + e];
        }
        xdot = sum_over_groups(xdot) * coef;
        half_t* po = dx + (int64_t)r * dx_rs + h * DH + 8 * G;
#pragma unroll
        for (int u = 0; u < DH / 32; ++u) {
            h8 o;
#pragma unroll
            for (int q = 0; q < 2; ++q)
#pragma unroll
                for (int e = 0; e < 4; ++e) o[4 * q + e] = (half_t)(y[2 * u + q][e] - (float)t.x[u][4 * q + e] * xdot);
            if (r < R) *reinterpret_cast<h8*>(po + 32 * u) = o;
        }

        // dW' (m = c, n = j) += x^T du over the 16 rows of the group
        if (!want_dw) return;
        wave_lds_order();
        h4 xa[DH / 16];
#pragma unroll
        for (int a = 0; a < DH / 16; ++a) xa[a] = tr_read4(Xs + trow * LDX + 16 * a + tcol);
#pragma unroll
        for (int b = 0; b < D / 16; ++b) {
            const h4 ub = tr_read4(Us + trow * LDU + 16 * b + tcol);
#pragma unroll
            for (int a = 0; a < DH / 16; ++a) dwacc[a][b] = mfma16(xa[a], ub, dwacc[a][b]);
        }
        wave_lds_order();   // before the next group's rows overwrite Xs / Us
    };
    Rows ra, rb;
    if (grp < ngrp) issue_loads(ra, grp);
    __syncthreads();   // both copies of W' in place
    while (grp < ngrp) {
        if (grp + gstride < ngrp) issue_loads(rb, grp + gstride);
        process(ra, grp);
        if ((grp += gstride) >= ngrp) break;
        if (grp + gstride < ngrp) issue_loads(ra, grp + gstride);
        process(rb, grp);
        grp += gstride;
    }

    // The waves' sums, one round: every wave leaves its dW' in LDS, then wave w adds up tiles
    // w, w + 8, ... of all the waves, in wave order, and stores them.
    if (!want_dw) return;
    f4* red = reinterpret_cast<f4*>(smem_raw);
    __syncthreads();   // every wave is out of the row loop: its LDS becomes the exchange area
#pragma unroll
    for (int a = 0; a < DH / 16; ++a)
#pragma unroll
        for (int b = 0; b < D / 16; ++b) red[(wv * Cfg::kTiles + a * (D / 16) + b) * 64 + lane] = dwacc[a][b];
    __syncthreads();
    float* out = dw_part + ((int64_t)(blockIdx.z * gridDim.x + blockIdx.x) * H + h) * D * DH;
    for (int t = wv; t < Cfg::kTiles; t += kFeatureBwdWaves) {
        f4 sum = red[t * 64 + lane];
#pragma unroll
        for (int o = 1; o < kFeatureBwdWaves; ++o) sum += red[(o * Cfg::kTiles + t) * 64 + lane];
        const int a = t / (D / 16), b = t % (D / 16);
        *reinterpret_cast<f4*>(out + (16 * b + i) * DH + 16 * a + 4 * G) = sum;
    }
}

// Rows of src [R, W] (W halves, multiple of 8) -> rows of dst that lie rs halves apart; 16 bytes per
// thread.  The copy job of a packed gradient for the shapes whose backward has none of its own.
__global__ __launch_bounds__(kThreads) void k_copy_rows_strided(const half_t* __restrict__ src, half_t* __restrict__ dst,
                                                                int64_t R, int W, int64_t rs) {
    const int ppr = W / 8;
    const int64_t total = R * ppr;
    for (int64_t p = (int64_t)blockIdx.x * kThreads + threadIdx.x; p < total; p += (int64_t)gridDim.x * kThreads) {
        const int64_t r = p / ppr;
        const int pc = (int)(p % ppr);
        *reinterpret_cast<uint4*>(dst + r * rs + pc * 8) = *reinterpret_cast<const uint4*>(src + r * W + pc * 8);
    }
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
