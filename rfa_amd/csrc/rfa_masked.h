// Quadratic-form random-feature attention with explicit masks (gfx950): the path the
// reference takes when CausalAttention is built with cuda_causal_rfa = False
// (random_feature_attention/causal_attention.py:57-109, normaliser utils.py:123-130):
//
//     a_ts   = phi_q[t] . phi_k[s],  set to 0 where key s is padded or attn_mask[t][s] is set
//     r_t    = sum_s a_ts ;  n_t = max(|r_t|, 1e-3)            (not the clamp-at-1 of the scan path)
//     out_t  = sum_s a_ts v_s / n_t
// and its backward, with G^ = G / n and gz_t = [|r_t| >= 1e-3] * -sign(r_t) (g_t . out_t) / n_t:
//     P_ts   = G^_t . v_s + gz_t  on unmasked (t, s), else 0
//     dphi_q[t] = sum_s P_ts phi_k[s] ;  dphi_k[s] = sum_t P_ts phi_q[t] ;  dv_s = sum_t a_ts G^_t
//
// Layouts as in the scan kernels: phi_q, phi_k [T, N, KD], v, out, g [T, N, DH], fp16,
// N = bsz * heads.  attn_mask is a byte matrix [T][Tp] (1 = masked, Tp = T rounded up to 64,
// the padding columns set to 1) and, for the dK/dV kernel, its transpose [T(s)][Tp(t)] padded the
// same way; key_padding_mask is [B, T] bytes (1 = padded key).  Either may be NULL.
//
// Every 64-step block of queries (forward, dQ) or keys (dK/dV) is one workgroup of 4 waves,
// 16 steps each with the block's own rows in registers as the B operand of the tile products;
// the 64 x 64 tiles of the other side pass through LDS, and the masked tiles are reused from
// registers as the operand of the second product (no LDS round trip).
#pragma once
#include "rfa_common.h"

namespace rfa {

constexpr float kQuadEps = 1e-3f;   // reference utils.py:129

// Column fragment in "split" slot order from a row-major LDS array:
//     slots 0..3 = X[r0 + 4G + e][c0 + i],  slots 4..7 = X[r0 + 16 + 4G + e][c0 + i].
// It pairs with an operand built from two fp32 accumulator tiles (rows 4G + e of tile t and
// of tile t + 1) when the contraction runs over the rows of X.
__device__ __forceinline__ h8 col_split8(const half_t* X, int ld, int r0, int c0, int lane) {
    const int s = lane & 15, G = lane >> 4;
    const half_t* p = X + (r0 + 4 * G + (s >> 2)) * ld + c0 + 4 * (s & 3);
    h4 a = tr_read4(p);
    h4 b = tr_read4(p + 16 * ld);
    return __builtin_shufflevector(a, b, 0, 1, 2, 3, 4, 5, 6, 7);
}

// two fp32 accumulator tiles -> one fp16 operand in split slot order
__device__ __forceinline__ h8 tiles_to_h8(const f4& t0, const f4& t1) {
    h8 r;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        r[e] = (half_t)t0[e];
        r[4 + e] = (half_t)t1[e];
    }
    return r;
}

template <int KD, int DH>
struct MaskedCfg {
    static_assert(KD % 64 == 0 && DH % 64 == 0, "KD and DH must be multiples of 64");
    static constexpr int C = kChunk;
    static constexpr int LDQ = KD + lds_pad(KD);
    static constexpr int LDV = DH + lds_pad(DH);
    static constexpr size_t kLds = (size_t)(C * LDQ + C * LDV) * 2 + C * 4;
};

// four mask bytes (one per accumulator element) -> keep flags; NULL mask keeps everything
__device__ __forceinline__ uint32_t mask_word(const uint8_t* __restrict__ m, int64_t off) {
    return m ? *reinterpret_cast<const uint32_t*>(m + off) : 0u;
}

// ---------------------------------------------------------------------------
// forward, one block of 64 queries (nblk = ceil(T / 64) blocks per sequence); wave w owns queries [i0 + 16w, i0 + 16w + 16).
// rsum (may be NULL) receives r_t, fp32 [T][N], for the backward pass.
// ---------------------------------------------------------------------------
// Blocks of 64 mask columns that a workgroup can skip: skip[b] != 0 when every entry of the
// 64 x 64 tile (rows r0 .. r0 + 63, columns 64 b ..) of the byte mask m ([T][Tp]) is set.  Rows past
// T count as set.  For the causal mask this is every block above the diagonal, half of the work.
// All 256 threads take part (one 16-byte piece of a tile each, eight tiles in flight); ends with a
// workgroup barrier.  m == NULL: nothing is skipped.
constexpr int kMaxMaskBlocks = 1024;

__device__ __forceinline__ void masked_tile_skip(const uint8_t* __restrict__ m, int r0, int T, int Tp, int nblk,
                                                 unsigned char* skip, int tid) {
    if (!m) {
        for (int b = tid; b < nblk; b += 256) skip[b] = 0;
        __syncthreads();
        return;
    }
    const int r = r0 + (tid >> 2);
    const uint8_t* mrow = m + (int64_t)min(r, T - 1) * Tp + 16 * (tid & 3);
    for (int b0 = 0; b0 < nblk; b0 += 8) {
        uint4 x[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) x[u] = *reinterpret_cast<const uint4*>(mrow + 64 * min(b0 + u, nblk - 1));
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            // no zero byte in any of the four words <=> all 16 entries set
            auto full = [](uint32_t v) { return ((v - 0x01010101u) & ~v & 0x80808080u) == 0u; };
            const bool set = r >= T || (full(x[u].x) && full(x[u].y) && full(x[u].z) && full(x[u].w));
            const int all = __syncthreads_and(set ? 1 : 0);
            if (tid == 0 && b0 + u < nblk) skip[b0 + u] = all ? 1 : 0;
        }
    }
    __syncthreads();
}

// first block at or after b that is not skipped (nblk if none); uniform over the workgroup
__device__ __forceinline__ int next_live_block(const unsigned char* skip, int b, int nblk) {
    while (b < nblk && skip[b]) ++b;
    return b;
}

template <int KD, int DH>
__device__ __forceinline__ void masked_fwd_block(const int n, const int i0,
    
    const half_t* __restrict__ q, const half_t* __restrict__ k, const half_t* __restrict__ v,
    const uint8_t* __restrict__ pad_mask, const uint8_t* __restrict__ attn_mask, half_t* __restrict__ out,
    float* __restrict__ rsum, int T, int Tp, int N, int H) {
    using Cfg = MaskedCfg<KD, DH>;
    constexpr int C = Cfg::C, LDQ = Cfg::LDQ, LDV = Cfg::LDV;
    constexpr int NKS = KD / 32, NCT = DH / 16;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    half_t* Ks = reinterpret_cast<half_t*>(smem_raw);
    half_t* Vs = Ks + C * LDQ;

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int row = lane & 15, G = lane >> 4;
    const int nblk = (T + C - 1) / C;
    const int64_t k_stride = (int64_t)N * KD, v_stride = (int64_t)N * DH;
    const half_t* kb = k + (int64_t)n * KD;
    const half_t* vb = v + (int64_t)n * DH;
    const uint8_t* prow = pad_mask ? pad_mask + (int64_t)(n / H) * T : nullptr;

    const int ti = i0 + 16 * w + row;
    const int tic = min(ti, T - 1);
    h8 bq[NKS];
    {
        const half_t* qrow = q + ((int64_t)tic * N + n) * KD;
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) bq[ks] = *reinterpret_cast<const h8*>(qrow + 32 * ks + 8 * G);
    }
    __shared__ unsigned char skip[kMaxMaskBlocks];
    masked_tile_skip(attn_mask, i0, T, Tp, nblk, skip, tid);
    ChunkRegs<KD> rk;
    ChunkRegs<DH> rv;
    auto prefetch = [&](int jb) {
        const int t0 = jb * C;
        chunk_g2r<KD>(rk, kb + (int64_t)t0 * k_stride, k_stride, T - t0, tid);
        chunk_g2r<DH>(rv, vb + (int64_t)t0 * v_stride, v_stride, T - t0, tid);
        if (prow) chunk_mask_rows<KD>(rk, prow + t0, tid);
    };
    int jb = next_live_block(skip, 0, nblk);
    if (jb < nblk) prefetch(jb);

    f4 acc[NCT];
#pragma unroll
    for (int ct = 0; ct < NCT; ++ct) acc[ct] = f4_zero();
    float rpart = 0.f;

    while (jb < nblk) {
        chunk_r2s<KD>(rk, Ks, LDQ, tid);
        chunk_r2s<DH>(rv, Vs, LDV, tid);
        __syncthreads();
        const int jb_next = next_live_block(skip, jb + 1, nblk);
        if (jb_next < nblk) prefetch(jb_next);
        f4 at[4];   // A^T tiles (m = j, n = i)
#pragma unroll
        for (int jt = 0; jt < 4; ++jt) {
            at[jt] = f4_zero();
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks)
                at[jt] = mfma32(row8(Ks, LDQ, 16 * jt + row, 32 * ks, G), bq[ks], at[jt]);
            const uint32_t mw = mask_word(attn_mask, (int64_t)tic * Tp + jb * C + 16 * jt + 4 * G);
#pragma unroll
            for (int e = 0; e < 4; ++e) at[jt][e] = ((mw >> (8 * e)) & 0xffu) ? 0.f : at[jt][e];
            rpart += (at[jt][0] + at[jt][1]) + (at[jt][2] + at[jt][3]);
        }
#pragma unroll
        for (int jp = 0; jp < 2; ++jp) {
            const h8 ba = tiles_to_h8(at[2 * jp], at[2 * jp + 1]);
#pragma unroll
            for (int ct = 0; ct < NCT; ++ct)
                acc[ct] = mfma32(col_split8(Vs, LDV, 32 * jp, 16 * ct, lane), ba, acc[ct]);
        }
        __syncthreads();
        jb = jb_next;
    }

    const float r = sum_over_groups(rpart);
    const float inv = 1.0f / fmaxf(fabsf(r), kQuadEps);
    if (ti < T) {
        half_t* orow = out + ((int64_t)ti * N + n) * DH;
#pragma unroll
        for (int ct = 0; ct < NCT; ++ct) {
            f4 o = acc[ct];
            o[0] *= inv; o[1] *= inv; o[2] *= inv; o[3] *= inv;
            *reinterpret_cast<h4*>(orow + 16 * ct + 4 * G) = to_h4(o);
        }
        if (rsum && G == 0) rsum[(int64_t)ti * N + n] = r;
    }
}

// ---------------------------------------------------------------------------
// backward pre-pass, one thread group per row:  ghat = g / n,  gz as in the header.
// grid = ceil(T * N / (256 / (DH/8))), 256 threads; DH/8 adjacent lanes share one row.
// ---------------------------------------------------------------------------
template <int DH>
__global__ __launch_bounds__(256) void k_masked_bwd_prep(const half_t* __restrict__ g, const half_t* __restrict__ o,
                                                         const float* __restrict__ rsum, half_t* __restrict__ ghat,
                                                         float* __restrict__ gz, int64_t rows) {
    constexpr int PPR = DH / 8;
    const int64_t piece = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t r_ = piece / PPR;
    const int c8 = (int)(piece % PPR);
    const bool valid = r_ < rows;
    const int64_t rc = valid ? r_ : rows - 1;
    union { uint4 u; h8 h; } xg, xo;
    xg.u = *reinterpret_cast<const uint4*>(g + rc * DH + c8 * 8);
    xo.u = *reinterpret_cast<const uint4*>(o + rc * DH + c8 * 8);
    float dot = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) dot += (float)xg.h[e] * (float)xo.h[e];
#pragma unroll
    for (int m = 1; m < PPR; m <<= 1) dot += __shfl_xor(dot, m, 64);
    const float r = rsum[rc];
    const float inv = 1.0f / fmaxf(fabsf(r), kQuadEps);
    if (!valid) return;
    h8 y;
#pragma unroll
    for (int e = 0; e < 8; ++e) y[e] = (half_t)((float)xg.h[e] * inv);
    *reinterpret_cast<h8*>(ghat + r_ * DH + c8 * 8) = y;
    if (c8 == 0) gz[r_] = (fabsf(r) >= kQuadEps) ? (r > 0.f ? -dot * inv : dot * inv) : 0.f;
}

// ---------------------------------------------------------------------------
// dphi_q.  Same structure as the forward with (G^, V, K) in the roles of (Q, K, V).  Padded
// keys need no mask here: their phi_k rows are read as zero, so they add nothing to dphi_q.
// ---------------------------------------------------------------------------
template <int KD, int DH>
__device__ __forceinline__ void masked_dq_block(const int n, const int i0,
    
    const half_t* __restrict__ ghat, const float* __restrict__ gz, const half_t* __restrict__ k,
    const half_t* __restrict__ v, const uint8_t* __restrict__ pad_mask, const uint8_t* __restrict__ attn_mask,
    half_t* __restrict__ dq, int T, int Tp, int N, int H) {
    using Cfg = MaskedCfg<KD, DH>;
    constexpr int C = Cfg::C, LDQ = Cfg::LDQ, LDV = Cfg::LDV;
    constexpr int NCS = DH / 32, NKT = KD / 16;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    half_t* Ks = reinterpret_cast<half_t*>(smem_raw);
    half_t* Vs = Ks + C * LDQ;

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int row = lane & 15, G = lane >> 4;
    const int nblk = (T + C - 1) / C;
    const int64_t k_stride = (int64_t)N * KD, v_stride = (int64_t)N * DH;
    const half_t* kb = k + (int64_t)n * KD;
    const half_t* vb = v + (int64_t)n * DH;
    const uint8_t* prow = pad_mask ? pad_mask + (int64_t)(n / H) * T : nullptr;

    const int ti = i0 + 16 * w + row;
    const int tic = min(ti, T - 1);
    h8 bg[NCS];
    float gzi;
    {
        const int64_t tn = (int64_t)tic * N + n;
#pragma unroll
        for (int cs = 0; cs < NCS; ++cs) bg[cs] = *reinterpret_cast<const h8*>(ghat + tn * DH + 32 * cs + 8 * G);
        gzi = gz[tn];
    }
    __shared__ unsigned char skip[kMaxMaskBlocks];
    masked_tile_skip(attn_mask, i0, T, Tp, nblk, skip, tid);
    ChunkRegs<KD> rk;
    ChunkRegs<DH> rv;
    auto prefetch = [&](int jb) {
        const int t0 = jb * C;
        chunk_g2r<KD>(rk, kb + (int64_t)t0 * k_stride, k_stride, T - t0, tid);
        chunk_g2r<DH>(rv, vb + (int64_t)t0 * v_stride, v_stride, T - t0, tid);
        if (prow) chunk_mask_rows<KD>(rk, prow + t0, tid);
    };
    int jb = next_live_block(skip, 0, nblk);
    if (jb < nblk) prefetch(jb);

    f4 acc[NKT];   // dQ^T tiles (m = k, n = i)
#pragma unroll
    for (int kt = 0; kt < NKT; ++kt) acc[kt] = f4_zero();

    while (jb < nblk) {
        chunk_r2s<KD>(rk, Ks, LDQ, tid);
        chunk_r2s<DH>(rv, Vs, LDV, tid);
        __syncthreads();
        const int jb_next = next_live_block(skip, jb + 1, nblk);
        if (jb_next < nblk) prefetch(jb_next);
        f4 pt[4];   // P^T tiles (m = j, n = i)
#pragma unroll
        for (int jt = 0; jt < 4; ++jt) {
            pt[jt] = f4_zero();
#pragma unroll
            for (int cs = 0; cs < NCS; ++cs)
                pt[jt] = mfma32(row8(Vs, LDV, 16 * jt + row, 32 * cs, G), bg[cs], pt[jt]);
            const uint32_t mw = mask_word(attn_mask, (int64_t)tic * Tp + jb * C + 16 * jt + 4 * G);
#pragma unroll
            for (int e = 0; e < 4; ++e) pt[jt][e] = ((mw >> (8 * e)) & 0xffu) ? 0.f : pt[jt][e] + gzi;
        }
#pragma unroll
        for (int jp = 0; jp < 2; ++jp) {
            const h8 bp = tiles_to_h8(pt[2 * jp], pt[2 * jp + 1]);
#pragma unroll
            for (int kt = 0; kt < NKT; ++kt)
                acc[kt] = mfma32(col_split8(Ks, LDQ, 32 * jp, 16 * kt, lane), bp, acc[kt]);
        }
        __syncthreads();
        jb = jb_next;
    }
    if (ti < T) {
        half_t* drow = dq + ((int64_t)ti * N + n) * KD;
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt) *reinterpret_cast<h4*>(drow + 16 * kt + 4 * G) = to_h4(acc[kt]);
    }
}

// ---------------------------------------------------------------------------
// dphi_k and dv.  Wave w owns keys [j0 + 16w, j0 + 16w + 16) with their K, V rows in registers;
// tiles (m = t, n = s).  attn_mask_t is the transposed mask [T(s)][Tp(t)].  A padded key gets
// dphi_k = 0 (the gradient of masked_fill) and dv = 0 (its weights are zero).
// ---------------------------------------------------------------------------
template <int KD, int DH>
__device__ __forceinline__ void masked_dkdv_block(const int n, const int j0,
    
    const half_t* __restrict__ q, const half_t* __restrict__ k, const half_t* __restrict__ v,
    const half_t* __restrict__ ghat, const float* __restrict__ gz, const uint8_t* __restrict__ pad_mask,
    const uint8_t* __restrict__ attn_mask_t, half_t* __restrict__ dk, half_t* __restrict__ dv, int T, int Tp,
    int N, int H) {
    using Cfg = MaskedCfg<KD, DH>;
    constexpr int C = Cfg::C, LDQ = Cfg::LDQ, LDV = Cfg::LDV;
    constexpr int NKS = KD / 32, NCS = DH / 32, NKT = KD / 16, NCT = DH / 16;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    half_t* Qs = reinterpret_cast<half_t*>(smem_raw);
    half_t* Gs = Qs + C * LDQ;
    float* gzs = reinterpret_cast<float*>(Gs + C * LDV);

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int row = lane & 15, G = lane >> 4;
    const int nblk = (T + C - 1) / C;
    const int64_t k_stride = (int64_t)N * KD, v_stride = (int64_t)N * DH;
    const half_t* qb = q + (int64_t)n * KD;
    const half_t* gb = ghat + (int64_t)n * DH;

    const int tj = j0 + 16 * w + row;
    const int tjc = min(tj, T - 1);
    const bool padded = pad_mask && pad_mask[(int64_t)(n / H) * T + tjc];
    h8 bk[NKS], bv[NCS];
    {
        const int64_t tn = (int64_t)tjc * N + n;
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) bk[ks] = *reinterpret_cast<const h8*>(k + tn * KD + 32 * ks + 8 * G);
#pragma unroll
        for (int cs = 0; cs < NCS; ++cs) bv[cs] = *reinterpret_cast<const h8*>(v + tn * DH + 32 * cs + 8 * G);
    }
    ChunkRegs<KD> rq;
    ChunkRegs<DH> rg;
    float gz_next;
    auto prefetch = [&](int t0) {
        chunk_g2r<KD>(rq, qb + (int64_t)t0 * k_stride, k_stride, T - t0, tid);
        chunk_g2r<DH>(rg, gb + (int64_t)t0 * v_stride, v_stride, T - t0, tid);
        gz_next = gz[(int64_t)(t0 + min(tid & (C - 1), rg.rows - 1)) * N + n];
    };
    __shared__ unsigned char skip[kMaxMaskBlocks];
    masked_tile_skip(attn_mask_t, j0, T, Tp, nblk, skip, tid);
    int ib = next_live_block(skip, 0, nblk);
    if (ib < nblk) prefetch(ib * C);

    f4 acck[NKT], accv[NCT];   // dK^T (m = k, n = s), dV^T (m = c, n = s)
#pragma unroll
    for (int kt = 0; kt < NKT; ++kt) acck[kt] = f4_zero();
#pragma unroll
    for (int ct = 0; ct < NCT; ++ct) accv[ct] = f4_zero();

    while (ib < nblk) {
        chunk_r2s<KD>(rq, Qs, LDQ, tid);
        chunk_r2s<DH>(rg, Gs, LDV, tid);
        if (tid < C) gzs[tid] = tid < rg.rows ? gz_next : 0.f;
        __syncthreads();
        const int ib_next = next_live_block(skip, ib + 1, nblk);
        if (ib_next < nblk) prefetch(ib_next * C);
        f4 a_[4], p_[4];   // tiles (m = t, n = s)
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            a_[it] = f4_zero();
            p_[it] = f4_zero();
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks)
                a_[it] = mfma32(row8(Qs, LDQ, 16 * it + row, 32 * ks, G), bk[ks], a_[it]);
#pragma unroll
            for (int cs = 0; cs < NCS; ++cs)
                p_[it] = mfma32(row8(Gs, LDV, 16 * it + row, 32 * cs, G), bv[cs], p_[it]);
            const f4 gzv = *reinterpret_cast<const f4*>(gzs + 16 * it + 4 * G);
            const uint32_t mw = mask_word(attn_mask_t, (int64_t)tjc * Tp + ib * C + 16 * it + 4 * G);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const bool masked = padded || ((mw >> (8 * e)) & 0xffu);
                a_[it][e] = masked ? 0.f : a_[it][e];
                p_[it][e] = masked ? 0.f : p_[it][e] + gzv[e];
            }
        }
#pragma unroll
        for (int ip = 0; ip < 2; ++ip) {
            const h8 ba = tiles_to_h8(a_[2 * ip], a_[2 * ip + 1]);
            const h8 bp = tiles_to_h8(p_[2 * ip], p_[2 * ip + 1]);
#pragma unroll
            for (int ct = 0; ct < NCT; ++ct)
                accv[ct] = mfma32(col_split8(Gs, LDV, 32 * ip, 16 * ct, lane), ba, accv[ct]);
#pragma unroll
            for (int kt = 0; kt < NKT; ++kt)
                acck[kt] = mfma32(col_split8(Qs, LDQ, 32 * ip, 16 * kt, lane), bp, acck[kt]);
        }
        __syncthreads();
        ib = ib_next;
    }
    if (tj < T) {
        half_t* krow = dk + ((int64_t)tj * N + n) * KD;
        half_t* vrow = dv + ((int64_t)tj * N + n) * DH;
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt) *reinterpret_cast<h4*>(krow + 16 * kt + 4 * G) = to_h4(acck[kt]);
#pragma unroll
        for (int ct = 0; ct < NCT; ++ct) *reinterpret_cast<h4*>(vrow + 16 * ct + 4 * G) = to_h4(accv[ct]);
    }
}

// ---------------------------------------------------------------------------
// Kernels.  With an attention mask, grid = N * ceil(nblk / 2): a workgroup takes row blocks p and
// nblk - 1 - p of one sequence, one after the other.  With a causal mask block p has p + 1 live
// column blocks, so every workgroup does the same work (nblk + 1 tiles); without that pairing the
// last row blocks set the kernel time and skipping the masked tiles would not shorten it.
// Without a mask nothing is skipped and grid = N * nblk, one row block per workgroup.
// ---------------------------------------------------------------------------
#define RFA_MASKED_PAIR(CALL, PAIRED)                                          \
    const int nblk = (T + kChunk - 1) / kChunk;                                \
    const int per_seq = (PAIRED) ? (nblk + 1) / 2 : nblk;                      \
    const int n = blockIdx.x / per_seq, p = blockIdx.x % per_seq;              \
    CALL(p * kChunk);                                                          \
    if ((PAIRED) && nblk - 1 - p != p) {                                       \
        __syncthreads();                                                       \
        CALL((nblk - 1 - p) * kChunk);                                         \
    }

template <int KD, int DH>
__global__ __launch_bounds__(256) void k_masked_fwd(
    const half_t* __restrict__ q, const half_t* __restrict__ k, const half_t* __restrict__ v,
    const uint8_t* __restrict__ pad_mask, const uint8_t* __restrict__ attn_mask, half_t* __restrict__ out,
    float* __restrict__ rsum, int T, int Tp, int N, int H) {
#define RFA_CALL_BLOCK(R0) masked_fwd_block<KD, DH>(n, R0, q, k, v, pad_mask, attn_mask, out, rsum, T, Tp, N, H)
    RFA_MASKED_PAIR(RFA_CALL_BLOCK, attn_mask != nullptr)
#undef RFA_CALL_BLOCK
}

template <int KD, int DH>
__global__ __launch_bounds__(256) void k_masked_dq(
    const half_t* __restrict__ ghat, const float* __restrict__ gz, const half_t* __restrict__ k,
    const half_t* __restrict__ v, const uint8_t* __restrict__ pad_mask, const uint8_t* __restrict__ attn_mask,
    half_t* __restrict__ dq, int T, int Tp, int N, int H) {
#define RFA_CALL_BLOCK(R0) masked_dq_block<KD, DH>(n, R0, ghat, gz, k, v, pad_mask, attn_mask, dq, T, Tp, N, H)
    RFA_MASKED_PAIR(RFA_CALL_BLOCK, attn_mask != nullptr)
#undef RFA_CALL_BLOCK
}

template <int KD, int DH>
__global__ __launch_bounds__(256) void k_masked_dkdv(
    const half_t* __restrict__ q, const half_t* __restrict__ k, const half_t* __restrict__ v,
    const half_t* __restrict__ ghat, const float* __restrict__ gz, const uint8_t* __restrict__ pad_mask,
    const uint8_t* __restrict__ attn_mask_t, half_t* __restrict__ dk, half_t* __restrict__ dv, int T, int Tp,
    int N, int H) {
#define RFA_CALL_BLOCK(R0) masked_dkdv_block<KD, DH>(n, R0, q, k, v, ghat, gz, pad_mask, attn_mask_t, dk, dv, T, Tp, N, H)
    RFA_MASKED_PAIR(RFA_CALL_BLOCK, attn_mask_t != nullptr)
#undef RFA_CALL_BLOCK
}
#undef RFA_MASKED_PAIR

}  // namespace rfa
