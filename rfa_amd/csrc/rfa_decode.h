// Incremental decoding step of causal RFA for gfx950: one workgroup per
// (batch, head) streams that head's fp32 state S (K x d) and z (K) through the
// CU once -- read, rank-1 update, readout, write -- with 16-byte loads/stores.
//
// Replaces the per-token ATen chain of incremental_rfa
// (random_feature_attention/causal_attention.py:42-50: 4 einsum + clamp + div and
// a freshly allocated state per token):
//     S += phi_k (x) v ;  z += phi_k ;  out = (phi_q . S) / max(phi_q . z, 1)
// The FUSED variant also evaluates phi(q), phi(k) from the raw projected q, k
// (utils.py:100-120), so a decode step of CausalAttention is one kernel.
#pragma once
#include "rfa_common.h"

namespace rfa {

template <int KD, int DH>
struct DecodeCfg {
    static constexpr int CQ = DH / 4;             // float4 columns per state row
    static constexpr int RPP = kThreads / CQ;     // state rows covered per pass
    static constexpr int NR = KD / RPP;           // rows per thread
    static_assert(kThreads % CQ == 0 && KD % RPP == 0, "unsupported decode shape");
};

// phi_x[0..2D) = scale * [sin(W x^), cos(W x^)] for one head, written to LDS as fp32.
// All 256 threads take part; TPP threads share one feature.
template <int KD, int DH>
__device__ __forceinline__ void decode_feature_map(float* phi_q, float* phi_k,
                                                   const half_t* __restrict__ qrow,
                                                   const half_t* __restrict__ krow,
                                                   const half_t* __restrict__ wh, float scale, int tid) {
    constexpr int D = KD / 2;
    constexpr int TPP = kThreads / (2 * D);       // threads per (vector, feature) pair
    static_assert(TPP >= 1 && (TPP & (TPP - 1)) == 0 && TPP <= 8, "unsupported feature count");
    constexpr int SEG = DH / TPP;                 // elements of the dot product per thread
    static_assert(SEG % 8 == 0, "unsupported head dim");
    const int pair = tid / TPP, part = tid % TPP;
    const int vec = pair / D, j = pair % D;       // vec 0: q, 1: k
    const half_t* xr = (vec == 0 ? qrow : krow);
    // every thread needs ||x||^2 of its vector: recompute from the full row (DH halves, cached)
    float ss = 0.f, dot = 0.f;
#pragma unroll
    for (int c = 0; c < DH; c += 8) {
        h8 xv = *reinterpret_cast<const h8*>(xr + c);
#pragma unroll
        for (int e = 0; e < 8; ++e) ss += (float)xv[e] * (float)xv[e];
    }
#pragma unroll
    for (int c = 0; c < SEG; c += 8) {
        h8 xv = *reinterpret_cast<const h8*>(xr + part * SEG + c);
        h8 wv = *reinterpret_cast<const h8*>(wh + j * DH + part * SEG + c);
#pragma unroll
        for (int e = 0; e < 8; ++e) dot += (float)xv[e] * (float)wv[e];
    }
#pragma unroll
    for (int o = 1; o < TPP; o <<= 1) dot += __shfl_xor(dot, o, 64);
    if (part == 0) {
        const float u = dot * rcp_nr(sqrtf(ss) + 1e-3f);
        float s_, c_;
        fast_sincos(u, s_, c_);
        float* dst = (vec == 0 ? phi_q : phi_k);
        dst[j] = scale * s_;
        dst[D + j] = scale * c_;
    }
}

// grid = N = bsz * heads.  FUSED: q, k are raw [N, DH] rows and w is [H, D, DH];
// otherwise q, k are feature rows [N, KD] and w is unused.  The rows of batch entry b, head h
// start at b * qk_bstride + h * (row width) (v: b * v_bstride + h * DH): H * width for separate
// contiguous tensors, three times that where q, k, v are the three thirds of one projection's
// output rows.  s_in/s_out ([N, KD, DH] fp32) and z_in/z_out ([N, KD] fp32) may alias.
template <int KD, int DH, bool FUSED>
__global__ __launch_bounds__(kThreads) void k_decode_step(
    const half_t* __restrict__ q, const half_t* __restrict__ k, const half_t* __restrict__ v,
    const half_t* __restrict__ w, float scale, int H, int64_t qk_bstride, int64_t v_bstride, const float* s_in,
    const float* z_in, float* s_out, float* z_out, half_t* __restrict__ out) {
    using Cfg = DecodeCfg<KD, DH>;
    constexpr int CQ = Cfg::CQ, RPP = Cfg::RPP, NR = Cfg::NR;
    __shared__ float phi_q[KD];
    __shared__ float phi_k[KD];
    __shared__ float red[4][DH];
    __shared__ float redz[4];
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int n = blockIdx.x;
    const int cq = tid % CQ, kr = tid / CQ;
    const int b_ = n / H, h_ = n % H;
    constexpr int QKW = FUSED ? DH : KD;          // width of a q / k row
    const int64_t qk_off = (int64_t)b_ * qk_bstride + (int64_t)h_ * QKW;
    const int64_t v_off = (int64_t)b_ * v_bstride + (int64_t)h_ * DH;

    // issue the state loads first: they are the long pole
    const float* sp = s_in + (int64_t)n * KD * DH;
    f4 st[NR];
#pragma unroll
    for (int r = 0; r < NR; ++r) st[r] = *reinterpret_cast<const f4*>(sp + (int64_t)(kr + r * RPP) * DH + 4 * cq);
    float zv = 0.f;
    if (tid < KD) zv = z_in[(int64_t)n * KD + tid];
    h4 vh = *reinterpret_cast<const h4*>(v + v_off + 4 * cq);

    if (FUSED) {
        decode_feature_map<KD, DH>(phi_q, phi_k, q + qk_off, k + qk_off, w + (int64_t)h_ * (KD / 2) * DH, scale, tid);
    } else {
        if (tid < KD) {
            phi_q[tid] = (float)q[qk_off + tid];
            phi_k[tid] = (float)k[qk_off + tid];
        }
    }
    __syncthreads();

    f4 acc = f4_zero();
    float* so = s_out + (int64_t)n * KD * DH;
#pragma unroll
    for (int r = 0; r < NR; ++r) {
        const int kk = kr + r * RPP;
        const float pk = phi_k[kk], pq = phi_q[kk];
        f4 s = st[r];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            s[e] += pk * (float)vh[e];
            acc[e] += pq * s[e];
        }
        *reinterpret_cast<f4*>(so + (int64_t)kk * DH + 4 * cq) = s;
    }
    float qz = 0.f;
    if (tid < KD) {
        zv += phi_k[tid];
        z_out[(int64_t)n * KD + tid] = zv;
        qz = phi_q[tid] * zv;
    }
    // reduce acc over the row groups kr: lanes with equal cq inside the wave, then the 4 waves
#pragma unroll
    for (int o = CQ; o < 64; o <<= 1) {
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[e] += __shfl_xor(acc[e], o, 64);
    }
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) qz += __shfl_xor(qz, o, 64);
    if (lane < CQ) *reinterpret_cast<f4*>(&red[wv][4 * lane]) = acc;
    if (lane == 0) redz[wv] = qz;
    __syncthreads();
    if (tid < DH) {
        const float num = (red[0][tid] + red[1][tid]) + (red[2][tid] + red[3][tid]);
        const float den = fmaxf((redz[0] + redz[1]) + (redz[2] + redz[3]), 1.0f);
        out[(int64_t)n * DH + tid] = (half_t)(num / den);
    }
}

// Reads n16 16-byte pieces and throws them away: brings rows that a later kernel reads with a
// dependent, latency-bound access into the cache hierarchy at streaming speed.
__global__ __launch_bounds__(kThreads) void k_touch_rows(const uint4* __restrict__ a, const uint4* __restrict__ b,
                                                         const uint4* __restrict__ c, int64_t na, int64_t nb,
                                                         int64_t nc) {
    const int64_t stride = (int64_t)gridDim.x * kThreads;
    unsigned int acc = 0u;
    for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < na; i += stride) acc ^= a[i].x;
    for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < nb; i += stride) acc ^= b[i].x;
    for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < nc; i += stride) acc ^= c[i].x;
    asm volatile("" ::"v"(acc));
}

}  // namespace rfa
