// Causal random-feature attention as a chunked scan on MFMA tiles (gfx950).
//
// Replaces the reference's serial-in-time kernels
//   rfa_forward   (random_feature_attention/cuda/forward.cu:86-126)
//   rfa_backward  (random_feature_attention/cuda/backward.cu:453-527)
// and computes the formulas of RFA.forward_torch / RFA.backward_torch
// (random_feature_attention/rfa.py:46-103) with fp16 inputs, fp32 accumulation
// and an fp32 running state.
//
// Work decomposition.  One (batch*head) sequence n is cut into `nseg` segments
// of `seg_len` steps (a multiple of 64); one workgroup handles one (n, segment)
// and walks its 64-step chunks serially, carrying the state
//     S[k][c] = sum_t phi_k[t][k] v[t][c]   (K x d, fp32, in MFMA accumulators)
//     z[k]    = sum_t phi_k[t][k]           (K,     fp32)
// Segment totals are produced by a first pass (k_segment_state) and summed by
// the consumer, so all (n, segment) workgroups of a pass run concurrently.
//
// Per chunk (Q, K: 64 x KD features; V, G: 64 x DH values), forward:
//     A   = tril(Q K^T)                       den_raw = rowsum(A) + Q z
//     out = (A V + Q S) / max(den_raw, 1)     S += K^T V ;  z += K^T 1
// backward, forward-in-time sweep (k_causal_bwd_dq):
//     X = G V^T, Y = G S^T                    e = rowsum(A*X) + rowsum(Q*Y)  (= G . num)
//     den = max(den_raw,1);  gz = den_raw > 1 ? -e/den^2 : 0     (rfa.py:87-91)
//     P = tril(X/den + gz 1^T);  dQ = P K + Y/den + gz z^T       (rfa.py:93-94)
//     dR += Q^T (G/den);  dr += Q^T gz       (segment totals for the reverse sweep)
// backward, reverse-in-time sweep (k_causal_bwd_dkdv), R/r = sums over later steps:
//     dK = P^T Q + V R^T + 1 r^T ;  dV = A^T (G/den) + K R      (rfa.py:96-101)
//     R += Q^T (G/den);  r += Q^T gz
#pragma once
#include "rfa_common.h"

namespace rfa {

// NW = wavefronts per workgroup (4 or 8).  Wave w = 4*half + rb: in the tile phases it
// works on row (column) block rb of the 64 x 64 chunk matrices and, with 8 waves, on one
// half of that block's tiles; for the state it owns value columns [w*DS, (w+1)*DS) or
// feature rows [w*KS, (w+1)*KS).  8 waves halve the per-wave state for the large shapes.
template <int KD, int DH, int NW = 4>
struct CausalCfg {
    static_assert(NW == 4 || NW == 8, "4 or 8 waves");
    static_assert(KD % 64 == 0 && DH % 64 == 0, "KD and DH must be multiples of 64");
    // kernels owning value-column slices need DH % (16*NW) == 0, those owning feature-row
    // slices KD % (16*NW) == 0; each kernel asserts what it uses
    static constexpr int NT = 64 * NW;    // threads per workgroup
    static constexpr int NH = NW / 4;     // waves sharing one 16-row block in the tile phases
    static constexpr int JPW = 4 / NH;    // 16 x 16 tiles of that block per wave
    static constexpr int C = kChunk;
    static constexpr int LDQ = KD + lds_pad(KD);
    static constexpr int LDV = DH + lds_pad(DH);
    static constexpr int LDA = C + 8;
    static constexpr int DS = DH / NW;    // value columns owned by one wave
    static constexpr int KS = KD / NW;    // feature rows owned by one wave
    // chunks k_segment_state keeps in flight / in LDS at once (as many as fit in 128 KB, at most 4)
    static constexpr int kSegStateGroup =
        (size_t)(C * LDQ + C * LDV) * 2 * 4 <= 128 * 1024 ? 4 : ((size_t)(C * LDQ + C * LDV) * 2 * 2 <= 128 * 1024 ? 2 : 1);
    static constexpr size_t kSegStateLds = (size_t)(C * LDQ + C * LDV) * 2 * kSegStateGroup;
    static constexpr size_t kFwdLds = (size_t)(2 * C * LDQ + C * LDV + C * LDA) * 2 + (KD + NH * C) * 4;
    static constexpr size_t kBwdDqLds =
        (size_t)(2 * C * LDQ + 2 * C * LDV + C * LDA) * 2 + (size_t)(KD + (2 * NH + NW + 2) * C) * 4;
    static constexpr size_t kBwdDqSavedLds =
        (size_t)(2 * C * LDQ + 2 * C * LDV + C * LDA) * 2 + (size_t)(KD + C) * 4;
    static constexpr size_t kBwdDkLds =
        (size_t)(2 * C * LDQ + 2 * C * LDV + 2 * C * LDA) * 2 + (size_t)(KD + C) * 4;
};

// ---------------------------------------------------------------------------
// pass 0: per-segment totals  dS = K^T V (KD x DH),  dz = K^T 1
// grid = N * nseg_out: the causal passes compute nseg_out = nseg - 1 totals per
// sequence (the last segment's total is never consumed); cross attention computes
// the single total of the whole source (nseg = nseg_out = 1) straight into its
// state tensors.  pad_mask ([B, T] bytes, 1 = padded key; read only when MASKED) zeroes
// phi_k rows (reference: cross_attention.py:97-100).
// ---------------------------------------------------------------------------
//
// FRAG selects the layout of the totals in wsS: false = row-major [KD][DH] per
// (sequence, segment) (read by the backward sweep and by cross attention);
// true = accumulator-fragment order [wave][kt][ct][lane][4], which the forward
// scan, owning the same tiles, reads back with one 16-byte load per tile.
// z is accumulated on the MFMA too: z tile (m=k) = K^T 1 with an all-ones operand;
// wave w owns the feature tiles kt in [w*NKTW, (w+1)*NKTW).
// row_copy (FRAG only, may be NULL) receives a second, row-major copy of the totals: the
// forward pass of a training step hands it to the backward pass, which then skips this pass.
template <int KD, int DH, int NW, bool FRAG, bool MASKED = false>
__global__ __launch_bounds__(64 * NW) void k_segment_state(
    const half_t* __restrict__ k, const half_t* __restrict__ v, const uint8_t* __restrict__ pad_mask,
    int H, float* __restrict__ wsS, float* __restrict__ wsZ, float* __restrict__ row_copy, int T, int N,
    int nseg, int nseg_out, int seg_len) {
    using Cfg = CausalCfg<KD, DH, NW>;
    constexpr int NT = Cfg::NT;
    constexpr int C = Cfg::C, LDQ = Cfg::LDQ, LDV = Cfg::LDV, DS = Cfg::DS;
    constexpr int NKT = KD / 16, NCT = DS / 16, NKTW = NKT / NW;
    static_assert(DH % (16 * NW) == 0 && NKT % NW == 0, "shape does not split over the waves");
    extern __shared__ __align__(16) unsigned char smem_raw[];
    half_t* Ks = reinterpret_cast<half_t*>(smem_raw);   // kGroup buffers of [K chunk | V chunk]

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int row = lane & 15, G = lane >> 4;
    int n, seg;
    seq_seg_of_block(blockIdx.x, N, nseg_out, n, seg);
    // MASKED is a compile-time switch: a run-time test around the mask loads would be a branch
    // between the chunk loads, and the compiler drains all outstanding loads at its join
    const uint8_t* mrow = MASKED ? pad_mask + (int64_t)(n / H) * T : nullptr;
    const int t_begin = seg * seg_len;
    const int t_end = min(T, t_begin + seg_len);
    const int64_t k_stride = (int64_t)N * KD, v_stride = (int64_t)N * DH;
    const half_t* kb = k + (int64_t)n * KD;
    const half_t* vb = v + (int64_t)n * DH;

    f4 S[NKT][NCT];
#pragma unroll
    for (int a = 0; a < NKT; ++a)
#pragma unroll
        for (int b = 0; b < NCT; ++b) S[a][b] = f4_zero();
    f4 zacc[NKTW];
#pragma unroll
    for (int a = 0; a < NKTW; ++a) zacc[a] = f4_zero();
    const h8 ones = h8_ones();

    // Rolling prefetch kGroup chunks deep: chunk u lives in registers rk[u % kGroup] until it is
    // written to LDS buffer u % kGroup, and the load of chunk u + kGroup is issued right after
    // that write.  Between the products on buffer b for chunk u and its next write (chunk
    // u + kGroup) lie the barriers of the chunks in between, so one barrier per chunk suffices.
    // All loads are branch-free: a chunk past the end re-reads the last valid row and is never
    // used (a branch between loads makes the compiler drain the outstanding ones at its join).
    constexpr int kGroup = Cfg::kSegStateGroup;
    RFA_TICK_INIT();
    ChunkRegs<KD, NT> rk[kGroup];
    ChunkRegs<DH, NT> rv[kGroup];
    auto load_chunk = [&](int c, int t0_want) {
        const int t0 = min(t0_want, t_end - 1);
        chunk_g2r<KD, NT>(rk[c], kb + (int64_t)t0 * k_stride, k_stride, t_end - t0, tid);
        chunk_g2r<DH, NT>(rv[c], vb + (int64_t)t0 * v_stride, v_stride, t_end - t0, tid);
        if (MASKED) chunk_mask_rows<KD, NT>(rk[c], mrow + t0, tid);
    };
#pragma unroll
    for (int c = 0; c < kGroup; ++c) load_chunk(c, t_begin + c * C);
    RFA_TICK(20);
    for (int tg = t_begin; tg < t_end; tg += kGroup * C) {
#pragma unroll
        for (int c = 0; c < kGroup; ++c) {
            const int t0 = tg + c * C;
            if (t0 >= t_end) break;
            half_t* Kc = Ks + c * (C * LDQ + C * LDV);
            half_t* Vc = Kc + C * LDQ;
            chunk_r2s<KD, NT>(rk[c], Kc, LDQ, tid);
            chunk_r2s<DH, NT>(rv[c], Vc, LDV, tid);
            RFA_TICK(21);
            __syncthreads();
            RFA_TICK(22);
            load_chunk(c, t0 + kGroup * C);
            RFA_TICK(24);
            h8 bv[NCT][2];
#pragma unroll
            for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
                for (int js = 0; js < 2; ++js) bv[ct][js] = col8(Vc, LDV, js * 32, w * DS + 16 * ct, lane);
#pragma unroll
            for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
                for (int js = 0; js < 2; ++js) {
                    h8 ak = col8(Kc, LDQ, js * 32, 16 * kt, lane);
#pragma unroll
                    for (int ct = 0; ct < NCT; ++ct) S[kt][ct] = mfma32(ak, bv[ct][js], S[kt][ct]);
                }
#pragma unroll
            for (int a = 0; a < NKTW; ++a)
#pragma unroll
                for (int js = 0; js < 2; ++js)
                    zacc[a] = mfma32(col8(Kc, LDQ, js * 32, 16 * (w * NKTW + a), lane), ones, zacc[a]);
            RFA_TICK(23);
        }
    }
    float* so = wsS + ((int64_t)(n * nseg + seg) * KD) * DH;
    if (FRAG) {
        f4* sf = reinterpret_cast<f4*>(so) + (int64_t)w * NKT * NCT * 64;
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
            for (int ct = 0; ct < NCT; ++ct) sf[(kt * NCT + ct) * 64 + lane] = S[kt][ct];
    }
    if (!FRAG || row_copy) {
        if (FRAG) so = row_copy + ((int64_t)(n * nseg + seg) * KD) * DH;
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
            for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    so[(16 * kt + 4 * G + e) * DH + w * DS + 16 * ct + row] = S[kt][ct][e];
    }
    if (row == 0) {
#pragma unroll
        for (int a = 0; a < NKTW; ++a)
            *reinterpret_cast<f4*>(wsZ + (int64_t)(n * nseg + seg) * KD + 16 * (w * NKTW + a) + 4 * G) = zacc[a];
    }
    RFA_TICK(25);
}

// ---------------------------------------------------------------------------
// forward scan.  Wave w owns value columns [w*DS, (w+1)*DS) of S (all KD rows),
// held as accumulator tiles S[kt][ct] with element (k = 16kt+4G+e, c = w*DS+16ct+i).
// ---------------------------------------------------------------------------
//
// den_out (causal only, may be NULL) receives the raw denominators rowsum(A) + q.z, fp32
// [T][N], for a backward pass that reuses them.  final_s / final_z (causal only, may be NULL)
// receive the state after step T - 1, fp32 [N][KD][DH] / [N][KD].
//
// CAUSAL = false is the cross-attention readout (reference: cross_attention.py:266-269):
// the state is the fixed total S, z of the source (wsS/wsZ hold one state per
// sequence), there is no intra-chunk term and no update, and the denominator is
// max(|q.z|, 1); k and v are not read.
template <int KD, int DH, int NW, bool CAUSAL>
__global__ __launch_bounds__(64 * NW) void k_causal_fwd(
    const half_t* __restrict__ q, const half_t* __restrict__ k, const half_t* __restrict__ v,
    half_t* __restrict__ out, const float* __restrict__ wsS, const float* __restrict__ wsZ,
    float* __restrict__ den_out, float* __restrict__ final_s, float* __restrict__ final_z, int T, int N,
    int nseg, int seg_len, int prefixed, int* __restrict__ hdr_out, PlanWords plan) {
    using Cfg = CausalCfg<KD, DH, NW>;
    constexpr int NT = Cfg::NT;
    constexpr int C = Cfg::C, LDQ = Cfg::LDQ, LDV = Cfg::LDV, LDA = Cfg::LDA, DS = Cfg::DS;
    constexpr int NKT = KD / 16, NCT = DS / 16, NKTW = NKT / NW;
    static_assert(DH % (16 * NW) == 0 && NKT % NW == 0, "shape does not split over the waves");
    extern __shared__ __align__(16) unsigned char smem_raw[];
    plan_write(hdr_out, plan);
    half_t* Qs = reinterpret_cast<half_t*>(smem_raw);
    half_t* Ks = Qs + C * LDQ;
    half_t* Vs = Ks + C * LDQ;
    half_t* As = Vs + C * LDV;
    float* zs = reinterpret_cast<float*>(As + C * LDA);
    float* dparts = zs + KD;    // [NH][C] partial raw denominators

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int row = lane & 15, G = lane >> 4;
    const int rb = w & 3, half = w >> 2;   // tile-phase role: 16-row block and which of its tiles
    constexpr int JPW = Cfg::JPW, NH = Cfg::NH;
    int n, seg;
    seq_seg_of_block(blockIdx.x, N, nseg, n, seg);
    const int t_begin = seg * seg_len;
    const int t_end = min(T, t_begin + seg_len);
    const int64_t k_stride = (int64_t)N * KD, v_stride = (int64_t)N * DH;
    const half_t* qb = q + (int64_t)n * KD;
    const half_t* kb = k + (int64_t)n * KD;
    const half_t* vb = v + (int64_t)n * DH;
    half_t* ob = out + (int64_t)n * DH;

    RFA_TICK_INIT();
    ChunkRegs<KD, NT> rq, rk;
    ChunkRegs<DH, NT> rv;
    chunk_g2r<KD, NT>(rq, qb + (int64_t)t_begin * k_stride, k_stride, t_end - t_begin, tid);
    if (CAUSAL) {
        chunk_g2r<KD, NT>(rk, kb + (int64_t)t_begin * k_stride, k_stride, t_end - t_begin, tid);
        chunk_g2r<DH, NT>(rv, vb + (int64_t)t_begin * v_stride, v_stride, t_end - t_begin, tid);
    }

    // carried state = sum of the totals of all earlier segments (causal: stored in
    // fragment order by k_segment_state<FRAG=true>; cross: one row-major state)
    f4 S[NKT][NCT];
#pragma unroll
    for (int a = 0; a < NKT; ++a)
#pragma unroll
        for (int b = 0; b < NCT; ++b) S[a][b] = f4_zero();
    f4 zacc[NKTW];      // z for feature tiles kt = w*NKTW + a, element k = 16kt + 4G + e
#pragma unroll
    for (int a = 0; a < NKTW; ++a) zacc[a] = f4_zero();
    const h8 ones = h8_ones();
    // states to sum: every earlier segment's total, or the one exclusive prefix k_totals_scan left
    const int s_begin = (CAUSAL && prefixed) ? seg : 0;
    const int n_states = CAUSAL ? (prefixed ? seg + 1 : seg) : 1;
    const int state_stride = CAUSAL ? nseg : 1;     // states stored per sequence
    for (int s = s_begin; s < n_states; ++s) {
        const float* si = wsS + ((int64_t)(n * state_stride + s) * KD) * DH;
        if (CAUSAL) {
            const f4* sf = reinterpret_cast<const f4*>(si) + (int64_t)w * NKT * NCT * 64;
#pragma unroll
            for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
                for (int ct = 0; ct < NCT; ++ct) S[kt][ct] += sf[(kt * NCT + ct) * 64 + lane];
        } else {
#pragma unroll
            for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
                for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        S[kt][ct][e] += si[(16 * kt + 4 * G + e) * DH + w * DS + 16 * ct + row];
        }
#pragma unroll
        for (int a = 0; a < NKTW; ++a)
            zacc[a] += *reinterpret_cast<const f4*>(wsZ + (int64_t)(n * state_stride + s) * KD + 16 * (w * NKTW + a) + 4 * G);
    }

    RFA_TICK(0);
    for (int t0 = t_begin; t0 < t_end; t0 += C) {
        chunk_r2s<KD, NT>(rq, Qs, LDQ, tid);
        if (CAUSAL) {
            chunk_r2s<KD, NT>(rk, Ks, LDQ, tid);
            chunk_r2s<DH, NT>(rv, Vs, LDV, tid);
        }
        if (row == 0) {
#pragma unroll
            for (int a = 0; a < NKTW; ++a) *reinterpret_cast<f4*>(zs + 16 * (w * NKTW + a) + 4 * G) = zacc[a];
        }
        RFA_TICK(1);
        __syncthreads();
        RFA_TICK(2);
        if (t0 + C < t_end) {      // the next chunk in two parts: q here, k and v after the tile phase
            const int rows = t_end - t0 - C;
            chunk_g2r<KD, NT>(rq, qb + (int64_t)(t0 + C) * k_stride, k_stride, rows, tid);
        }

        RFA_TICK(3);
        // ---- phase A: rows i in [16rb, 16rb+16) of A as A^T tiles (m=j, n=i); this wave's
        // tiles are jt = half*JPW + a (all tiles of the row, branch-free: the last row block
        // needs them anyway)
        {
            f4 at[JPW];
#pragma unroll
            for (int a = 0; a < JPW; ++a) at[a] = f4_zero();
#pragma unroll
            for (int ks = 0; ks < (CAUSAL ? KD / 32 : 0); ++ks) {
                h8 bq = row8(Qs, LDQ, 16 * rb + row, ks * 32, G);
#pragma unroll
                for (int a = 0; a < JPW; ++a)
                    at[a] = mfma32(row8(Ks, LDQ, 16 * (half * JPW + a) + row, ks * 32, G), bq, at[a]);
            }
            float part = 0.f;
#pragma unroll
            for (int a = 0; a < JPW; ++a) {
                const int jt = half * JPW + a;
#pragma unroll
                for (int e = 0; e < 4; ++e) {   // keep j <= i
                    const bool keep = (jt < rb) || (jt == rb && 4 * G + e <= row);
                    at[a][e] = keep ? at[a][e] : 0.f;
                }
                part += at[a][0] + at[a][1] + at[a][2] + at[a][3];
            }
            // + q_i . z : this lane covers features [G*KD/4 + half*QZW, +QZW)
            constexpr int QZW = KD / 4 / NH;
            f4 qz4 = f4_zero();
#pragma unroll
            for (int kk = 0; kk < QZW; kk += 8) {
                const int k0 = G * (KD / 4) + half * QZW + kk;
                h8 qv = *reinterpret_cast<const h8*>(Qs + (16 * rb + row) * LDQ + k0);
                f4 z0 = *reinterpret_cast<const f4*>(zs + k0);
                f4 z1 = *reinterpret_cast<const f4*>(zs + k0 + 4);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    qz4[e] += (float)qv[e] * z0[e];
                    qz4[e] += (float)qv[4 + e] * z1[e];
                }
            }
            part += (qz4[0] + qz4[1]) + (qz4[2] + qz4[3]);
            part = sum_over_groups(part);
            if (G == 0) dparts[half * C + 16 * rb + row] = part;
            if (CAUSAL) {
#pragma unroll
                for (int a = 0; a < JPW; ++a)
                    *reinterpret_cast<h4*>(As + (16 * rb + row) * LDA + 16 * (half * JPW + a) + 4 * G) = to_h4(at[a]);
            }
        }
        if (CAUSAL && t0 + C < t_end) {
            const int rows = t_end - t0 - C;
            chunk_g2r<KD, NT>(rk, kb + (int64_t)(t0 + C) * k_stride, k_stride, rows, tid);
            chunk_g2r<DH, NT>(rv, vb + (int64_t)(t0 + C) * v_stride, v_stride, rows, tid);
        }
        RFA_TICK(4);
        __syncthreads();
        RFA_TICK(5);

        // ---- phase B: out^T tiles (m=c, n=i) for this wave's value columns, then state update
        {
            h8 av[NCT][2];   // V column fragments: element V[j = 32js+8G+e][c = w*DS+16ct+i]
            if (CAUSAL) {
#pragma unroll
                for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
                    for (int js = 0; js < 2; ++js) av[ct][js] = col8(Vs, LDV, js * 32, w * DS + 16 * ct, lane);
            }

            RFA_TICK(6);
            f4 acc[4][NCT];
#pragma unroll
            for (int it = 0; it < 4; ++it) {
#pragma unroll
                for (int ct = 0; ct < NCT; ++ct) acc[it][ct] = f4_zero();
#pragma unroll
                for (int js = 0; js < (CAUSAL ? 2 : 0); ++js) {
                    if (js == 0 || it >= 2) {
                        h8 ba = row8(As, LDA, 16 * it + row, js * 32, G);
#pragma unroll
                        for (int ct = 0; ct < NCT; ++ct) acc[it][ct] = mfma32(av[ct][js], ba, acc[it][ct]);
                    }
                }
            }
#pragma unroll
            for (int ks = 0; ks < KD / 32; ++ks) {
                // the four row operands first: their LDS latency runs behind the conversion of the state
                h8 bq[4];
#pragma unroll
                for (int it = 0; it < 4; ++it) bq[it] = row_split8(Qs, LDQ, 16 * it + row, ks * 32, G);
                __builtin_amdgcn_sched_barrier(0);
                h8 hi[NCT];
#pragma unroll
                for (int ct = 0; ct < NCT; ++ct) hi[ct] = acc_to_operand_rn(S[2 * ks][ct], S[2 * ks + 1][ct]);
#pragma unroll
                for (int it = 0; it < 4; ++it) {
#pragma unroll
                    for (int ct = 0; ct < NCT; ++ct) acc[it][ct] = mfma32(hi[ct], bq[it], acc[it][ct]);
                }
            }
            RFA_TICK(7);
#pragma unroll
            for (int it = 0; it < 4; ++it) {
                const int i = 16 * it + row;
                float dr = dparts[i];
#pragma unroll
                for (int h = 1; h < NH; ++h) dr += dparts[h * C + i];
                const float inv = rcp_nr(fmaxf(CAUSAL ? dr : fabsf(dr), 1.0f));
                if (t0 + i < t_end) {
                    if (CAUSAL && den_out && w == 0 && G == 0) den_out[(int64_t)(t0 + i) * N + n] = dr;
#pragma unroll
                    for (int ct = 0; ct < NCT; ++ct) {
                        f4 o = acc[it][ct];
                        o[0] *= inv; o[1] *= inv; o[2] *= inv; o[3] *= inv;
                        *reinterpret_cast<h4*>(ob + (int64_t)(t0 + i) * v_stride + w * DS + 16 * ct + 4 * G) = to_h4(o);
                    }
                }
            }
            RFA_TICK(8);
            if (CAUSAL) {
                // S (m=k, n=c) += K^T V
#pragma unroll
                for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
                    for (int js = 0; js < 2; ++js) {
                        h8 ak = col8(Ks, LDQ, js * 32, 16 * kt, lane);
#pragma unroll
                        for (int ct = 0; ct < NCT; ++ct) S[kt][ct] = mfma32(ak, av[ct][js], S[kt][ct]);
                    }
#pragma unroll
                for (int a = 0; a < NKTW; ++a)
#pragma unroll
                    for (int js = 0; js < 2; ++js)
                        zacc[a] = mfma32(col8(Ks, LDQ, js * 32, 16 * (w * NKTW + a), lane), ones, zacc[a]);
            }
        }
        RFA_TICK(9);
        __syncthreads();
        RFA_TICK(10);
    }
    // the state after the last step of the sequence, for a decode loop that continues from it
    if (CAUSAL && final_s && seg == nseg - 1) {
        float* so = final_s + (int64_t)n * KD * DH;
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
            for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
                for (int e = 0; e < 4; ++e) so[(16 * kt + 4 * G + e) * DH + w * DS + 16 * ct + row] = S[kt][ct][e];
        if (row == 0) {
#pragma unroll
            for (int a = 0; a < NKTW; ++a)
                *reinterpret_cast<f4*>(final_z + (int64_t)n * KD + 16 * (w * NKTW + a) + 4 * G) = zacc[a];
        }
    }
}

// ---------------------------------------------------------------------------
// forward scan, two-stage pipeline (causal only).  8 waves: waves 0-3 ("tile group")
// bring chunk u into LDS and form what depends on q, k alone -- the masked A^T tiles,
// z and the denominators -- while waves 4-7 ("state group") finish chunk u-1: output
// tiles, division, store and the update of S.  Each SIMD holds one wave of either
// group, so the two stages overlap instead of adding up; the chunk arrays are double
// buffered and the groups meet at two workgroup barriers per chunk.  State-group wave
// w owns value columns [w*DS, (w+1)*DS) of S exactly like k_causal_fwd with 4 waves
// (same fragment-order segment totals).
// ---------------------------------------------------------------------------
template <int KD, int DH>
struct FwdPipeCfg {
    using Base = CausalCfg<KD, DH, 4>;
    static constexpr int C = Base::C, LDQ = Base::LDQ, LDV = Base::LDV, LDA = Base::LDA;
    static constexpr int kBufHalves = 2 * C * LDQ + C * LDV + C * LDA;
    static constexpr size_t kBufBytes = (size_t)kBufHalves * 2 + C * 4;     // + dens[C]
    static constexpr size_t kLds = 2 * kBufBytes + KD * 4;                   // + zs[KD]
    static_assert(kBufBytes % 16 == 0, "buffer alignment");
};

__device__ __forceinline__ void wg_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
}

//
// RECOMPUTE: no segment totals.  A workgroup first rebuilds the state at its segment's first step
// by streaming the k, v rows of everything before it through the same state update (one barrier
// and about a fifth of a scan chunk's time per 64 steps: the rows come out of the L2 of the XCD
// that holds all segments of the sequence), then scans.  Segments are cut so that prefix plus
// scan take every workgroup about equally long (SegBounds: later segments are shorter).  One
// launch, no workspace; pays while a sequence has few segments.
struct SegBounds {
    int first[17];      // segment s covers chunks [first[s], first[s + 1])
};

template <int KD, int DH, bool RECOMPUTE = false>
__global__ __launch_bounds__(512) void k_causal_fwd_pipe(
    const half_t* __restrict__ q, const half_t* __restrict__ k, const half_t* __restrict__ v,
    half_t* __restrict__ out, const float* __restrict__ wsS, const float* __restrict__ wsZ,
    float* __restrict__ den_out, float* __restrict__ final_s, float* __restrict__ final_z, int T, int N,
    int nseg, int seg_len, int prefixed, int* __restrict__ hdr_out, PlanWords plan, SegBounds bounds, int wide_rows) {
    // wide_rows: 64 rows of a tensor span 4 GiB or more, beyond the 32-bit lane offsets of the
    // full-chunk loads; every chunk then takes the clamped 64-bit row addresses (never with RECOMPUTE)
    plan_write(hdr_out, plan);
    using Cfg = FwdPipeCfg<KD, DH>;
    constexpr int NT = 256;      // threads per group
    constexpr int C = Cfg::C, LDQ = Cfg::LDQ, LDV = Cfg::LDV, LDA = Cfg::LDA, DS = DH / 4;
    constexpr int NKT = KD / 16, NCT = DS / 16, NKTW = NKT / 4;
    static_assert(DH % 64 == 0 && NKT % 4 == 0, "shape does not split over the waves");
    extern __shared__ __align__(16) unsigned char smem_raw[];
    float* zs = reinterpret_cast<float*>(smem_raw + 2 * Cfg::kBufBytes);

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const bool tile_group = wave < 4;
    const int w = wave & 3;                    // wave inside its group
    const int tid = threadIdx.x & (NT - 1);    // thread inside its group
    const int row = lane & 15, G = lane >> 4;
    int n, seg;
    seq_seg_of_block(blockIdx.x, N, nseg, n, seg);
    const int t_begin = RECOMPUTE ? bounds.first[seg] * C : seg * seg_len;
    const int t_end = min(T, RECOMPUTE ? bounds.first[seg + 1] * C : t_begin + seg_len);
    const int n_chunks = t_end > t_begin ? (t_end - t_begin + C - 1) / C : 0;
    const int n_prefix = (RECOMPUTE && n_chunks > 0) ? bounds.first[seg] : 0;     // full chunks before the segment
    const int64_t k_stride = (int64_t)N * KD, v_stride = (int64_t)N * DH;

    RFA_TICK_INIT();
    // Both branches run n_prefix iterations with one barrier each and one more barrier (RECOMPUTE),
    // then n_chunks + 1 iterations with exactly two barriers each.
    if (tile_group) {
        const half_t* qb = q + (int64_t)n * KD;
        const half_t* kb = k + (int64_t)n * KD;
        const half_t* vb = v + (int64_t)n * DH;
        ChunkRegs<KD, NT> rq, rk;
        ChunkRegs<DH, NT> rv;
        // full chunks: wave-uniform base plus one lane offset per tensor; only the last chunk of the
        // sequence can be short and takes the clamped row addresses
        RowPtrs<KD, NT> pq_, pk_;
        RowPtrs<DH, NT> pv_;
        pq_.init(qb, k_stride, tid);
        pk_.init(kb, k_stride, tid);
        pv_.init(vb, v_stride, tid);
        if (n_chunks > 0) {
            chunk_g2r<KD, NT>(rq, qb + (int64_t)t_begin * k_stride, k_stride, t_end - t_begin, tid);
            chunk_g2r<KD, NT>(rk, kb + (int64_t)t_begin * k_stride, k_stride, t_end - t_begin, tid);
            chunk_g2r<DH, NT>(rv, vb + (int64_t)t_begin * v_stride, v_stride, t_end - t_begin, tid);
        }
        f4 zacc[NKTW];      // z for feature tiles kt = w*NKTW + a, element k = 16kt + 4G + e
#pragma unroll
        for (int a = 0; a < NKTW; ++a) zacc[a] = f4_zero();
        const h8 ones = h8_ones();
        if constexpr (RECOMPUTE) {
            // the k, v rows of the chunks before the segment, three chunks in flight
            ChunkRegs<KD, NT> xk[3];
            ChunkRegs<DH, NT> xv[3];
            auto request = [&](auto set, int c) __attribute__((always_inline)) {
                constexpr int S_ = decltype(set)::value;
                const int64_t t0 = (int64_t)min(c, max(n_prefix - 1, 0)) * C;     // past the prefix: any valid chunk, never used
                pk_.load_full(xk[S_], t0 * k_stride);
                pv_.load_full(xv[S_], t0 * v_stride);
            };
            auto step = [&](auto set, int jc) __attribute__((always_inline)) {
                constexpr int S_ = decltype(set)::value;
                unsigned char* base = smem_raw + (jc & 1) * Cfg::kBufBytes;
                half_t* Ks = reinterpret_cast<half_t*>(base) + C * LDQ;
                half_t* Vs = Ks + C * LDQ;
                chunk_r2s<KD, NT>(xk[S_], Ks, LDQ, tid);
                chunk_r2s<DH, NT>(xv[S_], Vs, LDV, tid);
                wg_barrier();
                request(set, jc + 3);
#pragma unroll
                for (int a = 0; a < NKTW; ++a)
#pragma unroll
                    for (int js = 0; js < 2; ++js)
                        zacc[a] = mfma32(col8(Ks, LDQ, js * 32, 16 * (w * NKTW + a), lane), ones, zacc[a]);
            };
            using I0 = std::integral_constant<int, 0>;
            using I1 = std::integral_constant<int, 1>;
            using I2 = std::integral_constant<int, 2>;
            if (n_prefix > 0) {
                request(I0{}, 0);
                request(I1{}, 1);
                request(I2{}, 2);
            }
            for (int jc = 0; jc < n_prefix; jc += 3) {
                step(I0{}, jc);
                if (jc + 1 < n_prefix) step(I1{}, jc + 1);
                if (jc + 2 < n_prefix) step(I2{}, jc + 2);
            }
            wg_barrier();       // the state group has read the last prefix chunk
        } else {
            struct ZSlot { f4 z[NKTW]; };
            sum_slots<4, ZSlot>(prefixed ? seg : 0, prefixed ? seg + 1 : seg,
                [&](int s, ZSlot& t) {
#pragma unroll
                    for (int a = 0; a < NKTW; ++a)
                        t.z[a] = *reinterpret_cast<const f4*>(wsZ + (int64_t)(n * nseg + s) * KD + 16 * (w * NKTW + a) + 4 * G);
                },
                [&](const ZSlot& t, float keep) {
#pragma unroll
                    for (int a = 0; a < NKTW; ++a) zacc[a] += keep * t.z[a];
                });
        }
        RFA_TICK_AT(0, 0);
        for (int it = 0; it <= n_chunks; ++it) {
            unsigned char* base = smem_raw + (it & 1) * Cfg::kBufBytes;
            half_t* Qs = reinterpret_cast<half_t*>(base);
            half_t* Ks = Qs + C * LDQ;
            half_t* Vs = Ks + C * LDQ;
            half_t* As = Vs + C * LDV;
            float* dens = reinterpret_cast<float*>(As + C * LDA);
            const bool live = it < n_chunks;
            if (live) {
                chunk_r2s<KD, NT>(rq, Qs, LDQ, tid);
                chunk_r2s<KD, NT>(rk, Ks, LDQ, tid);
                chunk_r2s<DH, NT>(rv, Vs, LDV, tid);
                if (row == 0) {
#pragma unroll
                    for (int a = 0; a < NKTW; ++a) *reinterpret_cast<f4*>(zs + 16 * (w * NKTW + a) + 4 * G) = zacc[a];
                }
            }
            RFA_TICK_AT(1, 0);
            wg_barrier();
            RFA_TICK_AT(2, 0);
            if (live) {
                const int t0 = t_begin + it * C;
                const int rows_next = t_end - t0 - C;
                const bool fast_rows = rows_next >= C && !wide_rows;
                if (fast_rows) pq_.load_full(rq, (int64_t)(t0 + C) * k_stride);
                else if (rows_next > 0) chunk_g2r<KD, NT>(rq, qb + (int64_t)(t0 + C) * k_stride, k_stride, rows_next, tid);
                RFA_TICK_AT(3, 0);
                // rows i in [16w, 16w+16) of A as A^T tiles (m=j, n=i), all four j tiles
                f4 at[4];
#pragma unroll
                for (int a = 0; a < 4; ++a) at[a] = f4_zero();
#pragma unroll
                for (int ks = 0; ks < KD / 32; ++ks) {
                    h8 bq = row8(Qs, LDQ, 16 * w + row, ks * 32, G);
#pragma unroll
                    for (int a = 0; a < 4; ++a) at[a] = mfma32(row8(Ks, LDQ, 16 * a + row, ks * 32, G), bq, at[a]);
                }
                if (fast_rows) {              // second part of the next chunk's rows
                    pk_.load_full(rk, (int64_t)(t0 + C) * k_stride);
                    pv_.load_full(rv, (int64_t)(t0 + C) * v_stride);
                } else if (rows_next > 0) {
                    chunk_g2r<KD, NT>(rk, kb + (int64_t)(t0 + C) * k_stride, k_stride, rows_next, tid);
                    chunk_g2r<DH, NT>(rv, vb + (int64_t)(t0 + C) * v_stride, v_stride, rows_next, tid);
                }
                float part = 0.f;
#pragma unroll
                for (int a = 0; a < 4; ++a) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {   // keep j <= i
                        const bool keep = (a < w) || (a == w && 4 * G + e <= row);
                        at[a][e] = keep ? at[a][e] : 0.f;
                    }
                    part += at[a][0] + at[a][1] + at[a][2] + at[a][3];
                }
                // + q_i . z : this lane covers features [G*KD/4, (G+1)*KD/4)
                f4 qz4 = f4_zero();
#pragma unroll
                for (int kk = 0; kk < KD / 4; kk += 8) {
                    const int k0 = G * (KD / 4) + kk;
                    h8 qv = *reinterpret_cast<const h8*>(Qs + (16 * w + row) * LDQ + k0);
                    f4 z0 = *reinterpret_cast<const f4*>(zs + k0);
                    f4 z1 = *reinterpret_cast<const f4*>(zs + k0 + 4);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        qz4[e] += (float)qv[e] * z0[e];
                        qz4[e] += (float)qv[4 + e] * z1[e];
                    }
                }
                part += (qz4[0] + qz4[1]) + (qz4[2] + qz4[3]);
                part = sum_over_groups(part);
                if (G == 0) {
                    dens[16 * w + row] = part;
                    if (den_out && t0 + 16 * w + row < t_end) den_out[(int64_t)(t0 + 16 * w + row) * N + n] = part;
                }
#pragma unroll
                for (int a = 0; a < 4; ++a)
                    *reinterpret_cast<h4*>(As + (16 * w + row) * LDA + 16 * a + 4 * G) = to_h4(at[a]);
                // z += K^T 1 for the next chunk
#pragma unroll
                for (int a = 0; a < NKTW; ++a)
#pragma unroll
                    for (int js = 0; js < 2; ++js)
                        zacc[a] = mfma32(col8(Ks, LDQ, js * 32, 16 * (w * NKTW + a), lane), ones, zacc[a]);
            }
            RFA_TICK_AT(4, 0);
            wg_barrier();
            RFA_TICK_AT(5, 0);
        }
        if (final_z && seg == nseg - 1 && row == 0) {
#pragma unroll
            for (int a = 0; a < NKTW; ++a)
                *reinterpret_cast<f4*>(final_z + (int64_t)n * KD + 16 * (w * NKTW + a) + 4 * G) = zacc[a];
        }
    } else {
        half_t* ob = out + (int64_t)n * DH;
        f4 S[NKT][NCT];
#pragma unroll
        for (int a = 0; a < NKT; ++a)
#pragma unroll
            for (int b = 0; b < NCT; ++b) S[a][b] = f4_zero();
        if constexpr (RECOMPUTE) {
            for (int jc = 0; jc < n_prefix; ++jc) {
                wg_barrier();
                const half_t* Ks = reinterpret_cast<const half_t*>(smem_raw + (jc & 1) * Cfg::kBufBytes) + C * LDQ;
                const half_t* Vs = Ks + C * LDQ;
                h8 av[NCT][2];
#pragma unroll
                for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
                    for (int js = 0; js < 2; ++js) av[ct][js] = col8(Vs, LDV, js * 32, w * DS + 16 * ct, lane);
#pragma unroll
                for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
                    for (int js = 0; js < 2; ++js) {
                        h8 ak = col8(Ks, LDQ, js * 32, 16 * kt, lane);
#pragma unroll
                        for (int ct = 0; ct < NCT; ++ct) S[kt][ct] = mfma32(ak, av[ct][js], S[kt][ct]);
                    }
            }
            wg_barrier();
        } else {
            struct SSlot { f4 s[NKT][NCT]; };
            constexpr int GRP = (NKT * NCT <= 8) ? 3 : 1;     // 32 registers per slot at K = 128, d = 64
            sum_slots<GRP, SSlot>(prefixed ? seg : 0, prefixed ? seg + 1 : seg,
                [&](int s, SSlot& t) {
                    const f4* sf = reinterpret_cast<const f4*>(wsS + ((int64_t)(n * nseg + s) * KD) * DH) + (int64_t)w * NKT * NCT * 64;
#pragma unroll
                    for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
                        for (int ct = 0; ct < NCT; ++ct) t.s[kt][ct] = sf[(kt * NCT + ct) * 64 + lane];
                },
                [&](const SSlot& t, float keep) {
#pragma unroll
                    for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
                        for (int ct = 0; ct < NCT; ++ct) S[kt][ct] += keep * t.s[kt][ct];
                });
        }
        RFA_TICK_AT(8, 256);
        for (int it = 0; it <= n_chunks; ++it) {
            unsigned char* base = smem_raw + ((it + 1) & 1) * Cfg::kBufBytes;   // chunk it - 1
            const half_t* Qs = reinterpret_cast<const half_t*>(base);
            const half_t* Ks = Qs + C * LDQ;
            const half_t* Vs = Ks + C * LDQ;
            const half_t* As = Vs + C * LDV;
            const float* dens = reinterpret_cast<const float*>(As + C * LDA);
            const bool live = it >= 1;
            const int t0 = t_begin + (it - 1) * C;
            h8 av[NCT][2];   // V column fragments: element V[j = 32js+8G+e][c = w*DS+16ct+i]
            f4 acc[4][NCT];  // out^T tiles (m=c, n=i)
            if (live) {
#pragma unroll
                for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
                    for (int js = 0; js < 2; ++js) av[ct][js] = col8(Vs, LDV, js * 32, w * DS + 16 * ct, lane);
#pragma unroll
                for (int i4 = 0; i4 < 4; ++i4) {
#pragma unroll
                    for (int ct = 0; ct < NCT; ++ct) acc[i4][ct] = f4_zero();
#pragma unroll
                    for (int js = 0; js < 2; ++js) {
                        if (js == 0 || i4 >= 2) {
                            h8 ba = row8(As, LDA, 16 * i4 + row, js * 32, G);
#pragma unroll
                            for (int ct = 0; ct < NCT; ++ct) acc[i4][ct] = mfma32(av[ct][js], ba, acc[i4][ct]);
                        }
                    }
                }
            }
            RFA_TICK_AT(9, 256);
            wg_barrier();
            RFA_TICK_AT(10, 256);
            if (live) {
#pragma unroll
                for (int ks = 0; ks < KD / 32; ++ks) {
                    // the four row operands first: their LDS latency runs behind the conversion of the state
                    h8 bq[4];
#pragma unroll
                    for (int i4 = 0; i4 < 4; ++i4) bq[i4] = row_split8(Qs, LDQ, 16 * i4 + row, ks * 32, G);
                    __builtin_amdgcn_sched_barrier(0);
                    h8 sh[NCT];
#pragma unroll
                    for (int ct = 0; ct < NCT; ++ct) sh[ct] = acc_to_operand_rn(S[2 * ks][ct], S[2 * ks + 1][ct]);
#pragma unroll
                    for (int i4 = 0; i4 < 4; ++i4)
#pragma unroll
                        for (int ct = 0; ct < NCT; ++ct) acc[i4][ct] = mfma32(sh[ct], bq[i4], acc[i4][ct]);
                }
                RFA_TICK_AT(11, 256);
#pragma unroll
                for (int i4 = 0; i4 < 4; ++i4) {
                    const int i = 16 * i4 + row;
                    const float inv = rcp_nr(fmaxf(dens[i], 1.0f));
                    if (t0 + i < t_end) {
#pragma unroll
                        for (int ct = 0; ct < NCT; ++ct) {
                            f4 o = acc[i4][ct];
                            o[0] *= inv; o[1] *= inv; o[2] *= inv; o[3] *= inv;
                            *reinterpret_cast<h4*>(ob + (int64_t)(t0 + i) * v_stride + w * DS + 16 * ct + 4 * G) = to_h4(o);
                        }
                    }
                }
                RFA_TICK_AT(12, 256);
                // S (m=k, n=c) += K^T V
#pragma unroll
                for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
                    for (int js = 0; js < 2; ++js) {
                        h8 ak = col8(Ks, LDQ, js * 32, 16 * kt, lane);
#pragma unroll
                        for (int ct = 0; ct < NCT; ++ct) S[kt][ct] = mfma32(ak, av[ct][js], S[kt][ct]);
                    }
            }
            RFA_TICK_AT(13, 256);
            wg_barrier();
            RFA_TICK_AT(14, 256);
        }
        if (final_s && seg == nseg - 1) {
            float* so = final_s + (int64_t)n * KD * DH;
#pragma unroll
            for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
                for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
                    for (int e = 0; e < 4; ++e) so[(16 * kt + 4 * G + e) * DH + w * DS + 16 * ct + row] = S[kt][ct][e];
        }
    }
}

// ---------------------------------------------------------------------------
// backward, forward-in-time sweep: dQ, per-step (den, gz) stash, segment totals
// dR = Q^T (G/den), dr = Q^T gz.  Wave w owns feature rows [w*KS, (w+1)*KS):
// ST[ct][kt] / RT[ct][kt] hold element (c = 16ct+4G+e, k = w*KS+16kt+i).
// ---------------------------------------------------------------------------
//
// CAUSAL = false is the backward of the cross-attention readout: the state is the
// fixed source total (one per sequence in wsS/wsZ), den = max(|q.z|, 1),
// gz = -e/den^2 * sign(q.z) * [|q.z| > 1], dQ = Y/den + gz z^T, and the totals
// dR, dr written to wsR/wsr (one per sequence, nseg must be 1) are the gradients
// of the state (dS, dz).  k and v are not read; den_ws/gz_ws are not written.
template <int KD, int DH, int NW, bool CAUSAL>
__global__ __launch_bounds__(64 * NW) void k_causal_bwd_dq(
    const half_t* __restrict__ q, const half_t* __restrict__ k, const half_t* __restrict__ v,
    const half_t* __restrict__ g, half_t* __restrict__ dq, const float* __restrict__ wsS,
    const float* __restrict__ wsZ, float* __restrict__ wsR, float* __restrict__ wsr,
    float* __restrict__ den_ws, float* __restrict__ gz_ws, int T, int N, int nseg, int seg_len, int prefixed) {
    using Cfg = CausalCfg<KD, DH, NW>;
    constexpr int NT = Cfg::NT;
    constexpr int C = Cfg::C, LDQ = Cfg::LDQ, LDV = Cfg::LDV, LDA = Cfg::LDA, KS = Cfg::KS;
    constexpr int NKT = KS / 16, NCT = DH / 16;
    static_assert(KD % (16 * NW) == 0, "feature rows do not split over the waves");
    extern __shared__ __align__(16) unsigned char smem_raw[];
    half_t* Qs = reinterpret_cast<half_t*>(smem_raw);
    half_t* Ks = Qs + C * LDQ;
    half_t* Vs = Ks + C * LDQ;
    half_t* Gs = Vs + C * LDV;
    half_t* Ps = Gs + C * LDV;
    float* zs = reinterpret_cast<float*>(Ps + C * LDA);
    float* drs = zs + KD;        // [NH][C] partial den_raw per row
    float* e1s = drs + Cfg::NH * C;   // [NH][C] partial rowsum(A*X)
    float* e2p = e1s + Cfg::NH * C;   // [NW][C] per-wave partial rowsum(Q*Y)
    float* dens = e2p + NW * C;
    float* gzs = dens + C;

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int row = lane & 15, G = lane >> 4;
    const int rb = w & 3, half = w >> 2;   // tile-phase role: 16-row block and which of its tiles
    constexpr int JPW = Cfg::JPW, NH = Cfg::NH;
    int n, seg;
    seq_seg_of_block(blockIdx.x, N, nseg, n, seg);
    const int t_begin = seg * seg_len;
    const int t_end = min(T, t_begin + seg_len);
    const int64_t k_stride = (int64_t)N * KD, v_stride = (int64_t)N * DH;
    const half_t* qb = q + (int64_t)n * KD;
    const half_t* kb = k + (int64_t)n * KD;
    const half_t* vb = v + (int64_t)n * DH;
    const half_t* gb = g + (int64_t)n * DH;
    half_t* dqb = dq + (int64_t)n * KD;

    f4 ST[NCT][NKT], RT[NCT][NKT];
#pragma unroll
    for (int a = 0; a < NCT; ++a)
#pragma unroll
        for (int b = 0; b < NKT; ++b) { ST[a][b] = f4_zero(); RT[a][b] = f4_zero(); }
    // z and dr for this wave's feature slice, as MFMA tiles (m=k): element k = w*KS + 16kt + 4G + e
    f4 zacc[NKT], racc[NKT];
#pragma unroll
    for (int b = 0; b < NKT; ++b) { zacc[b] = f4_zero(); racc[b] = f4_zero(); }
    const h8 ones = h8_ones();
    const int s_begin = (CAUSAL && prefixed) ? seg : 0;
    const int n_states = CAUSAL ? (prefixed ? seg + 1 : seg) : 1;
    const int state_stride = CAUSAL ? nseg : 1;
    for (int s = s_begin; s < n_states; ++s) {
        const float* si = wsS + ((int64_t)(n * state_stride + s) * KD) * DH;
#pragma unroll
        for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
            for (int kt = 0; kt < NKT; ++kt) {
                f4 x = *reinterpret_cast<const f4*>(si + (w * KS + 16 * kt + row) * DH + 16 * ct + 4 * G);
                ST[ct][kt] += x;
            }
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt)
            zacc[kt] += *reinterpret_cast<const f4*>(wsZ + (int64_t)(n * state_stride + s) * KD + w * KS + 16 * kt + 4 * G);
    }

    ChunkRegs<KD, NT> rq, rk;
    ChunkRegs<DH, NT> rv, rg;
    {
        const int rows = t_end - t_begin;
        chunk_g2r<KD, NT>(rq, qb + (int64_t)t_begin * k_stride, k_stride, rows, tid);
        chunk_g2r<DH, NT>(rg, gb + (int64_t)t_begin * v_stride, v_stride, rows, tid);
        if (CAUSAL) {
            chunk_g2r<KD, NT>(rk, kb + (int64_t)t_begin * k_stride, k_stride, rows, tid);
            chunk_g2r<DH, NT>(rv, vb + (int64_t)t_begin * v_stride, v_stride, rows, tid);
        }
    }

    for (int t0 = t_begin; t0 < t_end; t0 += C) {
        chunk_r2s<KD, NT>(rq, Qs, LDQ, tid);
        chunk_r2s<DH, NT>(rg, Gs, LDV, tid);
        if (CAUSAL) {
            chunk_r2s<KD, NT>(rk, Ks, LDQ, tid);
            chunk_r2s<DH, NT>(rv, Vs, LDV, tid);
        }
        if (row == 0) {
#pragma unroll
            for (int kt = 0; kt < NKT; ++kt) *reinterpret_cast<f4*>(zs + w * KS + 16 * kt + 4 * G) = zacc[kt];
        }
        __syncthreads();
        if (t0 + C < t_end) {
            const int rows = t_end - t0 - C;
            chunk_g2r<KD, NT>(rq, qb + (int64_t)(t0 + C) * k_stride, k_stride, rows, tid);
            chunk_g2r<DH, NT>(rg, gb + (int64_t)(t0 + C) * v_stride, v_stride, rows, tid);
            if (CAUSAL) {
                chunk_g2r<KD, NT>(rk, kb + (int64_t)(t0 + C) * k_stride, k_stride, rows, tid);
                chunk_g2r<DH, NT>(rv, vb + (int64_t)(t0 + C) * v_stride, v_stride, rows, tid);
            }
        }

        // ---- phase A
        f4 xt[JPW];         // X^T tiles (m=j, n=i): rows i of block rb, tiles jt = half*JPW + a; kept for phase C
        f4 yt[NKT][4];      // Y^T tiles (m=k, n=i), k in this wave's slice, all i
        {
            f4 at[JPW];
#pragma unroll
            for (int a = 0; a < JPW; ++a) { at[a] = f4_zero(); xt[a] = f4_zero(); }
#pragma unroll
            for (int ks = 0; ks < (CAUSAL ? KD / 32 : 0); ++ks) {
                h8 bq = row8(Qs, LDQ, 16 * rb + row, ks * 32, G);
#pragma unroll
                for (int a = 0; a < JPW; ++a)   // all tiles of the row block, branch-free
                    at[a] = mfma32(row8(Ks, LDQ, 16 * (half * JPW + a) + row, ks * 32, G), bq, at[a]);
            }
#pragma unroll
            for (int cs = 0; cs < (CAUSAL ? DH / 32 : 0); ++cs) {
                h8 bg = row8(Gs, LDV, 16 * rb + row, cs * 32, G);
#pragma unroll
                for (int a = 0; a < JPW; ++a)
                    xt[a] = mfma32(row8(Vs, LDV, 16 * (half * JPW + a) + row, cs * 32, G), bg, xt[a]);
            }
            float part_d = 0.f, part_e = 0.f;
#pragma unroll
            for (int a = 0; a < JPW; ++a) {
                const int jt = half * JPW + a;
#pragma unroll
                for (int e = 0; e < 4; ++e) {   // keep j <= i
                    const bool keep = (jt < rb) || (jt == rb && 4 * G + e <= row);
                    at[a][e] = keep ? at[a][e] : 0.f;
                    part_d += at[a][e];
                    part_e += at[a][e] * xt[a][e];
                }
            }
            constexpr int QZW = KD / 4 / NH;   // this lane covers features [G*KD/4 + half*QZW, +QZW)
            f4 qz4 = f4_zero();
#pragma unroll
            for (int kk = 0; kk < QZW; kk += 8) {
                const int k0 = G * (KD / 4) + half * QZW + kk;
                h8 qv = *reinterpret_cast<const h8*>(Qs + (16 * rb + row) * LDQ + k0);
                f4 z0 = *reinterpret_cast<const f4*>(zs + k0);
                f4 z1 = *reinterpret_cast<const f4*>(zs + k0 + 4);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    qz4[e] += (float)qv[e] * z0[e];
                    qz4[e] += (float)qv[4 + e] * z1[e];
                }
            }
            part_d += (qz4[0] + qz4[1]) + (qz4[2] + qz4[3]);
            part_d = sum_over_groups(part_d);
            part_e = sum_over_groups(part_e);
            if (G == 0) {
                drs[half * C + 16 * rb + row] = part_d;
                e1s[half * C + 16 * rb + row] = part_e;
            }

#pragma unroll
            for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
                for (int it = 0; it < 4; ++it) yt[kt][it] = f4_zero();
#pragma unroll
            for (int cs = 0; cs < DH / 32; ++cs) {
                h8 bg[4];
#pragma unroll
                for (int it = 0; it < 4; ++it) bg[it] = row_split8(Gs, LDV, 16 * it + row, cs * 32, G);
                __builtin_amdgcn_sched_barrier(0);
                h8 hi[NKT];
#pragma unroll
                for (int kt = 0; kt < NKT; ++kt) hi[kt] = acc_to_operand_rn(ST[2 * cs][kt], ST[2 * cs + 1][kt]);
#pragma unroll
                for (int it = 0; it < 4; ++it) {
#pragma unroll
                    for (int kt = 0; kt < NKT; ++kt) yt[kt][it] = mfma32(hi[kt], bg[it], yt[kt][it]);
                }
            }
            float e2[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
                for (int it = 0; it < 4; ++it) {
                    h4 qv = *reinterpret_cast<const h4*>(Qs + (16 * it + row) * LDQ + w * KS + 16 * kt + 4 * G);
#pragma unroll
                    for (int e = 0; e < 4; ++e) e2[it] += yt[kt][it][e] * (float)qv[e];
                }
#pragma unroll
            for (int it = 0; it < 4; ++it) {
                float x = sum_over_groups(e2[it]);
                if (G == 0) e2p[w * C + 16 * it + row] = x;
            }
        }
        __syncthreads();

        // ---- phase B: denominators and d(qz) for the 64 rows of the chunk
        if (tid < C) {
            float dr = drs[tid], e = e1s[tid];
#pragma unroll
            for (int h = 1; h < NH; ++h) { dr += drs[h * C + tid]; e += e1s[h * C + tid]; }
            float e2sum = 0.f;
#pragma unroll
            for (int ww = 0; ww < NW; ++ww) e2sum += e2p[ww * C + tid];
            e += e2sum;
            const float den = fmaxf(CAUSAL ? dr : fabsf(dr), 1.0f);
            float gz;
            if (CAUSAL) {
                gz = (dr > 1.0f) ? -e / (den * den) : 0.f;
            } else {
                gz = (fabsf(dr) > 1.0f) ? (dr > 0.f ? -e : e) / (den * den) : 0.f;
            }
            dens[tid] = den;
            gzs[tid] = gz;
            if (CAUSAL && t0 + tid < t_end) {
                den_ws[(int64_t)(t0 + tid) * N + n] = den;
                gz_ws[(int64_t)(t0 + tid) * N + n] = gz;
            }
        }
        __syncthreads();

        // ---- phase C: P rows of this wave; G <- G/den in place
        {
            const int i = 16 * rb + row;
            const float inv = rcp_nr(dens[i]);
            const float gzi = gzs[i];
#pragma unroll
            for (int a = 0; a < (CAUSAL ? JPW : 0); ++a) {
                const int jt = half * JPW + a;
                h4 pv;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int j = 16 * jt + 4 * G + e;
                    pv[e] = (j <= i) ? (half_t)(xt[a][e] * inv + gzi) : (half_t)0.f;
                }
                *reinterpret_cast<h4*>(Ps + i * LDA + 16 * jt + 4 * G) = pv;
            }
            constexpr int PPR = DH / 8;
#pragma unroll
            for (int it = 0; it < ChunkRegs<DH, NT>::kPieces; ++it) {
                const int p = tid + NT * it;
                const int r_ = p / PPR, c8 = p % PPR;
                const float sc = rcp_nr(dens[r_]);
                h8 x = *reinterpret_cast<const h8*>(Gs + r_ * LDV + c8 * 8);
#pragma unroll
                for (int e = 0; e < 8; ++e) x[e] = (half_t)((float)x[e] * sc);
                *reinterpret_cast<h8*>(Gs + r_ * LDV + c8 * 8) = x;
            }
        }
        __syncthreads();

        // ---- phase D: dQ^T tiles (m=k, n=i), then the carried sums
        {
            h8 kf[NKT][2];   // K column fragments: K[j = 32js+8G+e][k = w*KS+16kt+i]
            if (CAUSAL) {
#pragma unroll
                for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
                    for (int js = 0; js < 2; ++js) kf[kt][js] = col8(Ks, LDQ, js * 32, w * KS + 16 * kt, lane);
            }
#pragma unroll
            for (int it = 0; it < 4; ++it) {
                const int i = 16 * it + row;
                const float inv = rcp_nr(dens[i]);
                const float gzi = gzs[i];
                h8 bp0, bp1;
                if (CAUSAL) {
                    bp0 = row8(Ps, LDA, i, 0, G);
                    bp1 = row8(Ps, LDA, i, 32, G);
                }
#pragma unroll
                for (int kt = 0; kt < NKT; ++kt) {
                    f4 zv = *reinterpret_cast<const f4*>(zs + w * KS + 16 * kt + 4 * G);
                    f4 acc;
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[e] = yt[kt][it][e] * inv + gzi * zv[e];
                    if (CAUSAL) {
                        acc = mfma32(kf[kt][0], bp0, acc);
                        if (it >= 2) acc = mfma32(kf[kt][1], bp1, acc);
                    }
                    if (t0 + i < t_end)
                        *reinterpret_cast<h4*>(dqb + (int64_t)(t0 + i) * k_stride + w * KS + 16 * kt + 4 * G) = to_h4(acc);
                }
            }
#pragma unroll
            for (int js = 0; js < 2; ++js) {
                h8 qf[NKT];   // Q column fragments
#pragma unroll
                for (int kt = 0; kt < NKT; ++kt) qf[kt] = col8(Qs, LDQ, js * 32, w * KS + 16 * kt, lane);
                // dr (m=k) += Q^T gz, z (m=k) += K^T 1: the vector operand is the same for all n
                h8 ghi, glo;
                f8_to_operand(*reinterpret_cast<const f4*>(gzs + js * 32 + 8 * G),
                              *reinterpret_cast<const f4*>(gzs + js * 32 + 8 * G + 4), ghi, glo);
#pragma unroll
                for (int kt = 0; kt < NKT; ++kt) {
                    racc[kt] = mfma32(qf[kt], ghi, racc[kt]);
                    if (CAUSAL) zacc[kt] = mfma32(kf[kt][js], ones, zacc[kt]);
                }
#pragma unroll
                for (int kt = 0; kt < NKT; ++kt) racc[kt] = mfma32(qf[kt], glo, racc[kt]);
#pragma unroll
                for (int ct = 0; ct < NCT; ++ct) {
                    h8 gf = col8(Gs, LDV, js * 32, 16 * ct, lane);
#pragma unroll
                    for (int kt = 0; kt < NKT; ++kt) RT[ct][kt] = mfma32(gf, qf[kt], RT[ct][kt]);
                    if (CAUSAL) {
                        h8 vf = col8(Vs, LDV, js * 32, 16 * ct, lane);
#pragma unroll
                        for (int kt = 0; kt < NKT; ++kt) ST[ct][kt] = mfma32(vf, kf[kt][js], ST[ct][kt]);
                    }
                }
            }
        }
        __syncthreads();
    }

    if (!CAUSAL || seg > 0) {   // causal: totals of segment 0 are never consumed
        float* ro = wsR + ((int64_t)(n * nseg + seg) * KD) * DH;
#pragma unroll
        for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
            for (int kt = 0; kt < NKT; ++kt)
                *reinterpret_cast<f4*>(ro + (w * KS + 16 * kt + row) * DH + 16 * ct + 4 * G) = RT[ct][kt];
        if (row == 0) {
#pragma unroll
            for (int kt = 0; kt < NKT; ++kt)
                *reinterpret_cast<f4*>(wsr + (int64_t)(n * nseg + seg) * KD + w * KS + 16 * kt + 4 * G) = racc[kt];
        }
    }
}

// ---------------------------------------------------------------------------
// backward, forward-in-time sweep for a backward pass that has the forward's output and
// raw denominators (rfa_causal_forward_save).  With num = out * den the reference's
// g . num (rfa.py:91) is (g . out) * den, so
//     gz_i = den_raw_i > 1 ? -(g_i . out_i) / den_i : 0
// is known when a chunk is loaded, and the sweep needs neither A = Q K^T nor the row sums
// of A*X and Q*Y:  per chunk, with G^ = G / den written to LDS at load time,
//     X^T = V G^T (tiles for 16 rows per wave),  P = tril(X + gz 1^T)
//     dQ^T = K^T P^T + S G^T + z gz^T ;  dR += G^T Q, dr += Q^T gz, S += V^T K, z += K^T 1
// Same state ownership, totals and (gz) stash as k_causal_bwd_dq<.., CAUSAL = true>.
// ---------------------------------------------------------------------------
template <int KD, int DH, int NW, int NWF, int KDG = KD>
__global__ __launch_bounds__(64 * NW) void k_causal_bwd_dq_saved(
    const half_t* __restrict__ q, const half_t* __restrict__ k, const half_t* __restrict__ v,
    const half_t* __restrict__ g, const half_t* __restrict__ o, const float* __restrict__ den_raw,
    half_t* __restrict__ dq, const float* __restrict__ wsS, const float* __restrict__ wsZ,
    float* __restrict__ wsR, float* __restrict__ wsr, float* __restrict__ gz_ws, int T, int N, int nseg,
    int seg_len, int prefixed, int s_nseg, int s_ratio, const int* __restrict__ hdr_in, PlanWords plan) {
    using Cfg = CausalCfg<KD, DH, NW>;
    constexpr int NT = Cfg::NT;
    constexpr int C = Cfg::C, LDQ = Cfg::LDQ, LDV = Cfg::LDV, LDA = Cfg::LDA, KS = Cfg::KS;
    constexpr int NKT = KS / 16, NCT = DH / 16;
    constexpr int PPR = DH / 8, VP = ChunkRegs<DH, NT>::kPieces;
    static_assert(KD % (16 * NW) == 0, "feature rows do not split over the waves");
    extern __shared__ __align__(16) unsigned char smem_raw[];
    half_t* Qs = reinterpret_cast<half_t*>(smem_raw);
    half_t* Ks = Qs + C * LDQ;
    half_t* Vs = Ks + C * LDQ;
    half_t* Gs = Vs + C * LDV;        // G / den
    half_t* Ps = Gs + C * LDV;
    float* zs = reinterpret_cast<float*>(Ps + C * LDA);
    float* gzs = zs + KD;

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int row = lane & 15, G = lane >> 4;
    const int rb = w & 3, half = w >> 2;
    constexpr int JPW = Cfg::JPW;
    // KDG > KD: the feature rows are split over KDG / KD workgroups per (sequence, segment);
    // this one owns features [koff, koff + KD) of the KDG-wide rows
    static_assert(KDG % KD == 0, "feature split");
    const int nsq = N * nseg;
    const int koff = (int)(blockIdx.x / nsq) * KD;
    const int bid = blockIdx.x % nsq;
    int n, seg;
    seq_seg_of_block(bid, N, nseg, n, seg);
    const int t_begin = seg * seg_len;
    const int t_end = min(T, t_begin + seg_len);
    const int64_t k_stride = (int64_t)N * KDG, v_stride = (int64_t)N * DH;
    const half_t* qb = q + (int64_t)n * KDG + koff;
    const half_t* kb = k + (int64_t)n * KDG + koff;
    const half_t* vb = v + (int64_t)n * DH;
    const half_t* gb = g + (int64_t)n * DH;
    const half_t* ob = o + (int64_t)n * DH;
    half_t* dqb = dq + (int64_t)n * KDG + koff;
    if (!plan_matches(hdr_in, plan)) {      // the saved buffer was written for another plan
        poison_rows<KD>(dqb, k_stride, t_begin, t_end);
        return;
    }

    f4 ST[NCT][NKT], RT[NCT][NKT];
#pragma unroll
    for (int a = 0; a < NCT; ++a)
#pragma unroll
        for (int b = 0; b < NKT; ++b) { ST[a][b] = f4_zero(); RT[a][b] = f4_zero(); }
    f4 zacc[NKT], racc[NKT];
#pragma unroll
    for (int b = 0; b < NKT; ++b) { zacc[b] = f4_zero(); racc[b] = f4_zero(); }
    const h8 ones = h8_ones();
    // The segment totals are read in the accumulator-fragment order the forward pass left them
    // in (k_segment_state<FRAG = true> for NWF waves: [wave][kt][ct][lane][4], element
    // (k = 16kt + 4G + e, c = wave*DSF + 16ct + i)); this wave needs (c = 16ct + 4G + e,
    // k = w*KS + 16kt + row), i.e. four scalar loads per tile, once per workgroup.
    // The forward may have cut the sequence into s_ratio times as many segments as this sweep
    // (s_nseg per sequence; only with scanned totals, where slot seg * s_ratio is the state at
    // this segment's first step).
    constexpr int DSF = DH / NWF, NCTF = DSF / 16, NKTF = KDG / 16;
    for (int s = prefixed ? seg : 0; s < (prefixed ? seg + 1 : seg); ++s) {
        const float* si = wsS + ((int64_t)(n * s_nseg + s * s_ratio) * KDG) * DH;
#pragma unroll
        for (int ct = 0; ct < NCT; ++ct) {
            const int wf = (16 * ct) / DSF, ctf = ((16 * ct) % DSF) / 16;
#pragma unroll
            for (int kt = 0; kt < NKT; ++kt) {
                const int ktf = (koff + w * KS + 16 * kt) / 16;
                const float* tile = si + (int64_t)((wf * NKTF + ktf) * NCTF + ctf) * 256 + ((row >> 2) * 16 + 4 * G) * 4 + (row & 3);
#pragma unroll
                for (int e = 0; e < 4; ++e) ST[ct][kt][e] += tile[4 * e];
            }
        }
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt)
            zacc[kt] += *reinterpret_cast<const f4*>(wsZ + (int64_t)(n * s_nseg + s * s_ratio) * KDG + koff + w * KS + 16 * kt + 4 * G);
    }

    RFA_TICK_INIT();
    ChunkRegs<KD, NT> rq, rk;
    ChunkRegs<DH, NT> rv, rg, ro;
    float dn[VP];
    auto prefetch_a = [&](int t0) {
        const int rows = t_end - t0;
        chunk_g2r<KD, NT>(rq, qb + (int64_t)t0 * k_stride, k_stride, rows, tid);
        chunk_g2r<DH, NT>(rg, gb + (int64_t)t0 * v_stride, v_stride, rows, tid);
        chunk_g2r<DH, NT>(ro, ob + (int64_t)t0 * v_stride, v_stride, rows, tid);
    };
    auto prefetch_b = [&](int t0) {
        const int rows = t_end - t0;
        chunk_g2r<KD, NT>(rk, kb + (int64_t)t0 * k_stride, k_stride, rows, tid);
        chunk_g2r<DH, NT>(rv, vb + (int64_t)t0 * v_stride, v_stride, rows, tid);
#pragma unroll
        for (int it = 0; it < VP; ++it) {
            const int r_ = min((tid + NT * it) / PPR, rv.rows - 1);
            dn[it] = den_raw[(int64_t)(t0 + r_) * N + n];
        }
    };
    prefetch_a(t_begin);
    prefetch_b(t_begin);
    RFA_TICK(0);

    for (int t0 = t_begin; t0 < t_end; t0 += C) {
        chunk_r2s<KD, NT>(rq, Qs, LDQ, tid);
        chunk_r2s<KD, NT>(rk, Ks, LDQ, tid);
        chunk_r2s<DH, NT>(rv, Vs, LDV, tid);
        // G^ = G / den into LDS; gz from g . out (the PPR lanes holding one row are adjacent)
#pragma unroll
        for (int it = 0; it < VP; ++it) {
            const int pc = tid + NT * it;
            const int r_ = pc / PPR, c8 = pc % PPR;
            const float dot = sum_adjacent<PPR>(dot_h8(rg.v[it], ro.v[it]));
            const bool valid = r_ < rg.rows;
            const float inv = valid ? rcp_nr(fmaxf(dn[it], 1.0f)) : 0.f;
            const float gzv = (valid && dn[it] > 1.0f) ? -dot * inv : 0.f;
            *reinterpret_cast<uint4*>(Gs + r_ * LDV + c8 * 8) = scale_h8(rg.v[it], inv);
            if (c8 == 0) {
                gzs[r_] = gzv;
                if (valid && koff == 0) gz_ws[(int64_t)(t0 + r_) * N + n] = gzv;
            }
        }
        if (row == 0) {
#pragma unroll
            for (int kt = 0; kt < NKT; ++kt) *reinterpret_cast<f4*>(zs + w * KS + 16 * kt + 4 * G) = zacc[kt];
        }
        RFA_TICK(1);
        __syncthreads();
        RFA_TICK(2);
        // The next chunk is requested in two parts, q, g, out here and k, v, den after the second
        // barrier (0.8 us per config-2 sweep: the requests of the 256 workgroups, which run in step,
        // are spread over the chunk).  The feature-half form keeps them together (1 % faster at
        // T = 16384, K = 256, d = 128); in the dK/dV sweep the split changed nothing.
        constexpr bool kSplitPrefetch = (KDG == KD);
        if (t0 + C < t_end) {
            prefetch_a(t0 + C);
            if (!kSplitPrefetch) prefetch_b(t0 + C);
        }
        RFA_TICK(3);

        // ---- phase A: P rows of this wave's row block (tiles jt = half*JPW + a); Y^T for the wave's feature slice
        f4 yt[NKT][4];      // (S G^T) tiles (m=k, n=i), k in this wave's slice, all i
        {
            const int i = 16 * rb + row;
            const float gzi = gzs[i];
            f4 xt[JPW];     // X^T tiles (m=j, n=i)
#pragma unroll
            for (int a = 0; a < JPW; ++a) xt[a] = f4_zero();
#pragma unroll
            for (int cs = 0; cs < DH / 32; ++cs) {
                h8 bg = row8(Gs, LDV, i, cs * 32, G);
#pragma unroll
                for (int a = 0; a < JPW; ++a)
                    xt[a] = mfma32(row8(Vs, LDV, 16 * (half * JPW + a) + row, cs * 32, G), bg, xt[a]);
            }
#pragma unroll
            for (int a = 0; a < JPW; ++a) {
                const int jt = half * JPW + a;
                h4 pv;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int j = 16 * jt + 4 * G + e;
                    pv[e] = (j <= i) ? (half_t)(xt[a][e] + gzi) : (half_t)0.f;
                }
                *reinterpret_cast<h4*>(Ps + i * LDA + 16 * jt + 4 * G) = pv;
            }
            RFA_TICK(4);
#pragma unroll
            for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
                for (int it = 0; it < 4; ++it) yt[kt][it] = f4_zero();
#pragma unroll
            for (int cs = 0; cs < DH / 32; ++cs) {
                // the four row operands first: their LDS latency runs behind the conversion of the state
                h8 bg[4];
#pragma unroll
                for (int it = 0; it < 4; ++it) bg[it] = row_split8(Gs, LDV, 16 * it + row, cs * 32, G);
                __builtin_amdgcn_sched_barrier(0);
                h8 hi[NKT];
#pragma unroll
                for (int kt = 0; kt < NKT; ++kt) hi[kt] = acc_to_operand_rn(ST[2 * cs][kt], ST[2 * cs + 1][kt]);
#pragma unroll
                for (int it = 0; it < 4; ++it) {
#pragma unroll
                    for (int kt = 0; kt < NKT; ++kt) yt[kt][it] = mfma32(hi[kt], bg[it], yt[kt][it]);
                }
            }
        }
        RFA_TICK(5);
        __syncthreads();
        RFA_TICK(6);
        if (kSplitPrefetch && t0 + C < t_end) prefetch_b(t0 + C);

        // ---- phase D: dQ^T tiles (m=k, n=i), then the carried sums
        {
            h8 kf[NKT][2];   // K column fragments: K[j = 32js+8G+e][k = w*KS+16kt+i]
#pragma unroll
            for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
                for (int js = 0; js < 2; ++js) kf[kt][js] = col8(Ks, LDQ, js * 32, w * KS + 16 * kt, lane);
#pragma unroll
            for (int it = 0; it < 4; ++it) {
                const int i = 16 * it + row;
                const float gzi = gzs[i];
                const h8 bp0 = row8(Ps, LDA, i, 0, G);
                const h8 bp1 = row8(Ps, LDA, i, 32, G);
#pragma unroll
                for (int kt = 0; kt < NKT; ++kt) {
                    f4 zv = *reinterpret_cast<const f4*>(zs + w * KS + 16 * kt + 4 * G);
                    f4 acc;
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[e] = yt[kt][it][e] + gzi * zv[e];
                    acc = mfma32(kf[kt][0], bp0, acc);
                    if (it >= 2) acc = mfma32(kf[kt][1], bp1, acc);
                    if (t0 + i < t_end)
                        *reinterpret_cast<h4*>(dqb + (int64_t)(t0 + i) * k_stride + w * KS + 16 * kt + 4 * G) = to_h4(acc);
                }
            }
            RFA_TICK(7);
#pragma unroll
            for (int js = 0; js < 2; ++js) {
                h8 qf[NKT];   // Q column fragments
#pragma unroll
                for (int kt = 0; kt < NKT; ++kt) qf[kt] = col8(Qs, LDQ, js * 32, w * KS + 16 * kt, lane);
                h8 ghi, glo;
                f8_to_operand(*reinterpret_cast<const f4*>(gzs + js * 32 + 8 * G),
                              *reinterpret_cast<const f4*>(gzs + js * 32 + 8 * G + 4), ghi, glo);
#pragma unroll
                for (int kt = 0; kt < NKT; ++kt) {
                    racc[kt] = mfma32(qf[kt], ghi, racc[kt]);
                    zacc[kt] = mfma32(kf[kt][js], ones, zacc[kt]);
                }
#pragma unroll
                for (int kt = 0; kt < NKT; ++kt) racc[kt] = mfma32(qf[kt], glo, racc[kt]);
#pragma unroll
                for (int ct = 0; ct < NCT; ++ct) {
                    h8 gf = col8(Gs, LDV, js * 32, 16 * ct, lane);
                    h8 vf = col8(Vs, LDV, js * 32, 16 * ct, lane);
#pragma unroll
                    for (int kt = 0; kt < NKT; ++kt) RT[ct][kt] = mfma32(gf, qf[kt], RT[ct][kt]);
#pragma unroll
                    for (int kt = 0; kt < NKT; ++kt) ST[ct][kt] = mfma32(vf, kf[kt][js], ST[ct][kt]);
                }
            }
        }
        RFA_TICK(8);
        __syncthreads();
        RFA_TICK(9);
    }

    if (seg > 0) {   // totals of segment 0 are never consumed
        float* ro_ = wsR + ((int64_t)(n * nseg + seg) * KDG) * DH;
#pragma unroll
        for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
            for (int kt = 0; kt < NKT; ++kt)
                *reinterpret_cast<f4*>(ro_ + (koff + w * KS + 16 * kt + row) * DH + 16 * ct + 4 * G) = RT[ct][kt];
        if (row == 0) {
#pragma unroll
            for (int kt = 0; kt < NKT; ++kt)
                *reinterpret_cast<f4*>(wsr + (int64_t)(n * nseg + seg) * KDG + koff + w * KS + 16 * kt + 4 * G) = racc[kt];
        }
    }
    RFA_TICK(10);
}

// ---------------------------------------------------------------------------
// backward, reverse-in-time sweep: dK, dV.  R is carried twice, once per
// contraction: RT[ct][kt] (c = 16ct+4G+e, k = w*KS+16kt+i) contracts over c for
// dK; RR[kt][ct] (k = 16kt+4G+e, c = w*DS+16ct+i) contracts over k for dV.
// ---------------------------------------------------------------------------
//
// CAUSAL = false is the backward of the cross-attention state: R, r are the fixed
// gradients dS, dz (one per sequence in wsR/wsr), dK = V dS^T + 1 dz^T,
// dV = K dS; q, g, den_ws, gz_ws are not read.  pad_mask ([B, T] bytes, may be
// NULL; H heads per batch entry) marks padded keys: their phi_k rows are read as
// zero and their dK rows are written as zero (the gradient of masked_fill).
//
// SPLIT (8 waves only): the state phase is divided by role instead of by slice.  Waves
// 0-3 carry RT and r and produce dK, waves 4-7 carry RR and produce dV, each for a
// quarter of the feature rows / value columns; the tile phase is shared by all 8 waves
// as usual.  Two waves per SIMD then work on independent halves of the state phase.
template <int KD, int DH, int NW, bool CAUSAL, bool SPLIT = false>
__global__ __launch_bounds__(64 * NW) void k_causal_bwd_dkdv(
    const half_t* __restrict__ q, const half_t* __restrict__ k, const half_t* __restrict__ v,
    const half_t* __restrict__ g, half_t* __restrict__ dk, half_t* __restrict__ dv,
    const float* __restrict__ wsR, const float* __restrict__ wsr, const float* __restrict__ den_ws,
    const float* __restrict__ gz_ws, const uint8_t* __restrict__ pad_mask, int H, int T, int N,
    int nseg, int seg_len, int prefixed, const int* __restrict__ hdr_in, PlanWords plan) {
    using Cfg = CausalCfg<KD, DH, NW>;
    constexpr int NT = Cfg::NT;
    static_assert(!SPLIT || NW == 8, "the role split needs 8 waves");
    constexpr int NOWN = SPLIT ? 4 : NW;             // waves sharing one role
    constexpr int C = Cfg::C, LDQ = Cfg::LDQ, LDV = Cfg::LDV, LDA = Cfg::LDA, KS = KD / NOWN, DS = DH / NOWN;
    constexpr int NKT = KS / 16, NCT = DH / 16;      // RT tiles
    constexpr int NKT2 = KD / 16, NCT2 = DS / 16;    // RR tiles
    static_assert(KD % (16 * NOWN) == 0 && DH % (16 * NOWN) == 0, "shape does not split over the waves");
    extern __shared__ __align__(16) unsigned char smem_raw[];
    half_t* Qs = reinterpret_cast<half_t*>(smem_raw);
    half_t* Ks = Qs + C * LDQ;
    half_t* Vs = Ks + C * LDQ;
    half_t* Gs = Vs + C * LDV;       // G / den
    half_t* ATs = Gs + C * LDV;      // AT[j][i] = A[i][j]
    half_t* PTs = ATs + C * LDA;     // PT[j][i] = P[i][j]
    float* rs = reinterpret_cast<float*>(PTs + C * LDA);
    float* gzs = rs + KD;

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int row = lane & 15, G = lane >> 4;
    const int rb = w & 3, half = w >> 2;   // tile-phase role: 16-row block and which of its tiles
    const int ws = SPLIT ? (w & 3) : w;    // state-phase slice
    const bool do_dk = !SPLIT || w < 4, do_dv = !SPLIT || w >= 4;
    constexpr int JPW = Cfg::JPW;
    int n, seg;
    seq_seg_of_block(blockIdx.x, N, nseg, n, seg);
    const int t_begin = seg * seg_len;
    const int t_end = min(T, t_begin + seg_len);
    const int64_t k_stride = (int64_t)N * KD, v_stride = (int64_t)N * DH;
    const half_t* qb = q + (int64_t)n * KD;
    const half_t* kb = k + (int64_t)n * KD;
    const half_t* vb = v + (int64_t)n * DH;
    const half_t* gb = g + (int64_t)n * DH;
    half_t* dkb = dk + (int64_t)n * KD;
    half_t* dvb = dv + (int64_t)n * DH;
    if (!plan_matches(hdr_in, plan)) {
        poison_rows<KD>(dkb, k_stride, t_begin, t_end);
        poison_rows<DH>(dvb, v_stride, t_begin, t_end);
        return;
    }

    f4 RT[NCT][NKT], RR[NKT2][NCT2];
#pragma unroll
    for (int a = 0; a < NCT; ++a)
#pragma unroll
        for (int b = 0; b < NKT; ++b) RT[a][b] = f4_zero();
#pragma unroll
    for (int a = 0; a < NKT2; ++a)
#pragma unroll
        for (int b = 0; b < NCT2; ++b) RR[a][b] = f4_zero();
    f4 racc[NKT];     // r for this wave's feature slice (m=k tiles): k = w*KS + 16kt + 4G + e
#pragma unroll
    for (int b = 0; b < NKT; ++b) racc[b] = f4_zero();
    const uint8_t* mrow = (!CAUSAL && pad_mask) ? pad_mask + (int64_t)(n / H) * T : nullptr;
    // later segments' totals, or the one exclusive suffix k_totals_scan left
    const int s_first = CAUSAL ? (prefixed ? seg : seg + 1) : 0, s_last = CAUSAL ? (prefixed ? seg + 1 : nseg) : 1;
    const int state_stride = CAUSAL ? nseg : 1;
    {
        // The carried state at the segment's last step, R = sum of the slots [s_first, s_last): all
        // threads add the slots up with coalesced 16-byte loads and pass the sum through LDS (which
        // the first chunk does not need yet); each wave then takes its fragments from there.  Reading
        // the fragments straight from HBM costs the dV waves 32 scalar loads per lane and slot.
        constexpr int LDR = DH + 4;                          // floats; spreads the rows over the banks
        constexpr bool kStaged = (size_t)KD * LDR * 4 <= Cfg::kBwdDkLds;   // the sum fits the chunk buffers
        if constexpr (kStaged) {
        constexpr int PER = KD * DH / 4 / NT;
        static_assert((KD * DH / 4) % NT == 0, "state does not divide over the threads");
        float* Rs = reinterpret_cast<float*>(smem_raw);
        f4 sum[PER];
#pragma unroll
        for (int it = 0; it < PER; ++it) sum[it] = f4_zero();
        {
            struct RSlot { f4 s[PER]; f4 r[NKT]; };
            constexpr int GRP = (PER + NKT <= 8) ? 3 : 1;
            sum_slots<GRP, RSlot>(s_first, s_last,
                [&](int s, RSlot& t) {
                    const float* ri = wsR + ((int64_t)(n * state_stride + s) * KD) * DH;
#pragma unroll
                    for (int it = 0; it < PER; ++it) t.s[it] = *reinterpret_cast<const f4*>(ri + (int64_t)(tid + NT * it) * 4);
#pragma unroll
                    for (int kt = 0; kt < NKT; ++kt)
                        t.r[kt] = *reinterpret_cast<const f4*>(wsr + (int64_t)(n * state_stride + s) * KD + ws * KS + 16 * kt + 4 * G);
                },
                [&](const RSlot& t, float keep) {
#pragma unroll
                    for (int it = 0; it < PER; ++it) sum[it] += keep * t.s[it];
                    if (do_dk) {
#pragma unroll
                        for (int kt = 0; kt < NKT; ++kt) racc[kt] += keep * t.r[kt];
                    }
                });
        }
#pragma unroll
        for (int it = 0; it < PER; ++it) {
            const int e0 = (tid + NT * it) * 4;
            *reinterpret_cast<f4*>(Rs + (e0 / DH) * LDR + e0 % DH) = sum[it];
        }
        __syncthreads();
        if (do_dk) {
#pragma unroll
            for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
                for (int kt = 0; kt < NKT; ++kt)
                    RT[ct][kt] = *reinterpret_cast<const f4*>(Rs + (ws * KS + 16 * kt + row) * LDR + 16 * ct + 4 * G);
        }
        if (do_dv) {
#pragma unroll
            for (int kt = 0; kt < NKT2; ++kt)
#pragma unroll
                for (int ct = 0; ct < NCT2; ++ct)
#pragma unroll
                    for (int e = 0; e < 4; ++e) RR[kt][ct][e] = Rs[(16 * kt + 4 * G + e) * LDR + ws * DS + 16 * ct + row];
        }
        __syncthreads();                                     // before the first chunk overwrites the staged state
        } else {
            for (int s = s_first; s < s_last; ++s) {
                const float* ri = wsR + ((int64_t)(n * state_stride + s) * KD) * DH;
                if (do_dk) {
#pragma unroll
                    for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
                        for (int kt = 0; kt < NKT; ++kt)
                            RT[ct][kt] += *reinterpret_cast<const f4*>(ri + (ws * KS + 16 * kt + row) * DH + 16 * ct + 4 * G);
#pragma unroll
                    for (int kt = 0; kt < NKT; ++kt)
                        racc[kt] += *reinterpret_cast<const f4*>(wsr + (int64_t)(n * state_stride + s) * KD + ws * KS + 16 * kt + 4 * G);
                }
                if (do_dv) {
#pragma unroll
                    for (int kt = 0; kt < NKT2; ++kt)
#pragma unroll
                        for (int ct = 0; ct < NCT2; ++ct)
#pragma unroll
                            for (int e = 0; e < 4; ++e)
                                RR[kt][ct][e] += ri[(16 * kt + 4 * G + e) * DH + ws * DS + 16 * ct + row];
                }
            }
        }
    }

    ChunkRegs<KD, NT> rq, rk;
    ChunkRegs<DH, NT> rv, rg;
    float inv_den[ChunkRegs<DH, NT>::kPieces];
    float gz_next = 0.f;
    constexpr int PPRV = DH / 8;
    auto prefetch = [&](int t0) {
        const int rows = t_end - t0;
        chunk_g2r<KD, NT>(rk, kb + (int64_t)t0 * k_stride, k_stride, rows, tid);
        chunk_g2r<DH, NT>(rv, vb + (int64_t)t0 * v_stride, v_stride, rows, tid);
        if (CAUSAL) {
            chunk_g2r<KD, NT>(rq, qb + (int64_t)t0 * k_stride, k_stride, rows, tid);
            chunk_g2r<DH, NT>(rg, gb + (int64_t)t0 * v_stride, v_stride, rows, tid);
#pragma unroll
            for (int it = 0; it < ChunkRegs<DH, NT>::kPieces; ++it) {
                // raw den only: dividing here would wait for the loads issued just above
                // (rows past the end read the last valid one; chunk_r2s_scaled zeroes them)
                const int r_ = min((tid + NT * it) / PPRV, rg.rows - 1);
                inv_den[it] = den_ws[(int64_t)(t0 + r_) * N + n];
            }
            gz_next = gz_ws[(int64_t)(t0 + min(tid, rg.rows - 1)) * N + n];
        } else if (mrow) {
            chunk_mask_rows<KD, NT>(rk, mrow + t0, tid);
        }
    };

    const int n_chunks = (t_end - t_begin + C - 1) / C;
    prefetch(t_begin + (n_chunks - 1) * C);
    for (int ci = n_chunks - 1; ci >= 0; --ci) {
        const int t0 = t_begin + ci * C;
        chunk_r2s<KD, NT>(rk, Ks, LDQ, tid);
        chunk_r2s<DH, NT>(rv, Vs, LDV, tid);
        if (CAUSAL) {
            chunk_r2s<KD, NT>(rq, Qs, LDQ, tid);
#pragma unroll
            for (int it = 0; it < ChunkRegs<DH, NT>::kPieces; ++it)
                inv_den[it] = rcp_nr(fmaxf(inv_den[it], 1.0f));   // den_ws may hold raw or clamped denominators
            chunk_r2s_scaled<DH, NT>(rg, inv_den, Gs, LDV, tid);
            if (tid < C) gzs[tid] = tid < rg.rows ? gz_next : 0.f;
        }
        if (row == 0 && do_dk) {
#pragma unroll
            for (int kt = 0; kt < NKT; ++kt) *reinterpret_cast<f4*>(rs + ws * KS + 16 * kt + 4 * G) = racc[kt];
        }
        __syncthreads();
        if (ci > 0) prefetch(t0 - C);

        // ---- phase A: columns j in [16rb, 16rb+16) of A and P (tiles m=i, n=j)
        if (CAUSAL) {
            f4 a_[JPW], p_[JPW];   // tiles it = half*JPW + a of column block rb
#pragma unroll
            for (int a = 0; a < JPW; ++a) { a_[a] = f4_zero(); p_[a] = f4_zero(); }
#pragma unroll
            for (int ks = 0; ks < KD / 32; ++ks) {
                h8 bk = row8(Ks, LDQ, 16 * rb + row, ks * 32, G);
#pragma unroll
                for (int a = 0; a < JPW; ++a)   // all tiles of the column block, branch-free
                    a_[a] = mfma32(row8(Qs, LDQ, 16 * (half * JPW + a) + row, ks * 32, G), bk, a_[a]);
            }
#pragma unroll
            for (int cs = 0; cs < DH / 32; ++cs) {
                h8 bv = row8(Vs, LDV, 16 * rb + row, cs * 32, G);
#pragma unroll
                for (int a = 0; a < JPW; ++a)
                    p_[a] = mfma32(row8(Gs, LDV, 16 * (half * JPW + a) + row, cs * 32, G), bv, p_[a]);
            }
            const int j = 16 * rb + row;
#pragma unroll
            for (int a = 0; a < JPW; ++a) {
                const int it = half * JPW + a;
                h4 av, pv;
                f4 gzv = *reinterpret_cast<const f4*>(gzs + 16 * it + 4 * G);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int i = 16 * it + 4 * G + e;
                    av[e] = (i >= j) ? (half_t)a_[a][e] : (half_t)0.f;
                    pv[e] = (i >= j) ? (half_t)(p_[a][e] + gzv[e]) : (half_t)0.f;
                }
                *reinterpret_cast<h4*>(ATs + j * LDA + 16 * it + 4 * G) = av;
                *reinterpret_cast<h4*>(PTs + j * LDA + 16 * it + 4 * G) = pv;
            }
        }
        if (CAUSAL) __syncthreads();

        // ---- phase B
        {
            h8 qf[NKT][2];    // Q column fragments for this wave's feature slice
            h8 gf2[NCT2][2];  // (G/den) column fragments for this wave's value slice
            if (CAUSAL) {
                if (do_dk) {
#pragma unroll
                    for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
                        for (int is = 0; is < 2; ++is) qf[kt][is] = col8(Qs, LDQ, is * 32, ws * KS + 16 * kt, lane);
                }
                if (do_dv) {
#pragma unroll
                    for (int ct = 0; ct < NCT2; ++ct)
#pragma unroll
                        for (int is = 0; is < 2; ++is) gf2[ct][is] = col8(Gs, LDV, is * 32, ws * DS + 16 * ct, lane);
                }
            }

            if (do_dk) {
            // dK^T tiles (m=k, n=j)
            f4 dkacc[NKT][4];
#pragma unroll
            for (int kt = 0; kt < NKT; ++kt) {
                f4 rv4 = *reinterpret_cast<const f4*>(rs + ws * KS + 16 * kt + 4 * G);
#pragma unroll
                for (int jt = 0; jt < 4; ++jt) {
                    f4 acc = rv4;
                    if (CAUSAL) {
                        if (jt < 2) acc = mfma32(qf[kt][0], row8(PTs, LDA, 16 * jt + row, 0, G), acc);
                        acc = mfma32(qf[kt][1], row8(PTs, LDA, 16 * jt + row, 32, G), acc);
                    }
                    dkacc[kt][jt] = acc;
                }
            }
#pragma unroll
            for (int cs = 0; cs < DH / 32; ++cs) {
                // the four row operands first: their LDS latency runs behind the conversion of the state
                h8 bvv[4];
#pragma unroll
                for (int jt = 0; jt < 4; ++jt) bvv[jt] = row_split8(Vs, LDV, 16 * jt + row, cs * 32, G);
                __builtin_amdgcn_sched_barrier(0);     // keep the reads ahead of the conversion
                h8 hi[NKT];
#pragma unroll
                for (int kt = 0; kt < NKT; ++kt) hi[kt] = acc_to_operand_rn(RT[2 * cs][kt], RT[2 * cs + 1][kt]);
#pragma unroll
                for (int jt = 0; jt < 4; ++jt) {
#pragma unroll
                    for (int kt = 0; kt < NKT; ++kt) dkacc[kt][jt] = mfma32(hi[kt], bvv[jt], dkacc[kt][jt]);
                }
            }
#pragma unroll
            for (int jt = 0; jt < 4; ++jt) {
                const int jj = 16 * jt + row;
                if (t0 + jj < t_end) {
                    const bool padded = mrow && mrow[t0 + jj];
#pragma unroll
                    for (int kt = 0; kt < NKT; ++kt)
                        *reinterpret_cast<h4*>(dkb + (int64_t)(t0 + jj) * k_stride + ws * KS + 16 * kt + 4 * G) =
                            padded ? h4_zero() : to_h4(dkacc[kt][jt]);
                }
            }
            }

            if (do_dv) {
            // dV^T tiles (m=c, n=j)
            f4 dvacc[NCT2][4];
#pragma unroll
            for (int ct = 0; ct < NCT2; ++ct)
#pragma unroll
                for (int jt = 0; jt < 4; ++jt) {
                    f4 acc = f4_zero();
                    if (CAUSAL) {
                        if (jt < 2) acc = mfma32(gf2[ct][0], row8(ATs, LDA, 16 * jt + row, 0, G), acc);
                        acc = mfma32(gf2[ct][1], row8(ATs, LDA, 16 * jt + row, 32, G), acc);
                    }
                    dvacc[ct][jt] = acc;
                }
#pragma unroll
            for (int ks = 0; ks < KD / 32; ++ks) {
                h8 bkk[4];
#pragma unroll
                for (int jt = 0; jt < 4; ++jt) bkk[jt] = row_split8(Ks, LDQ, 16 * jt + row, ks * 32, G);
                __builtin_amdgcn_sched_barrier(0);     // keep the reads ahead of the conversion
                h8 hi[NCT2];
#pragma unroll
                for (int ct = 0; ct < NCT2; ++ct) hi[ct] = acc_to_operand_rn(RR[2 * ks][ct], RR[2 * ks + 1][ct]);
#pragma unroll
                for (int jt = 0; jt < 4; ++jt) {
#pragma unroll
                    for (int ct = 0; ct < NCT2; ++ct) dvacc[ct][jt] = mfma32(hi[ct], bkk[jt], dvacc[ct][jt]);
                }
            }
#pragma unroll
            for (int jt = 0; jt < 4; ++jt) {
                const int jj = 16 * jt + row;
                if (t0 + jj < t_end) {
#pragma unroll
                    for (int ct = 0; ct < NCT2; ++ct)
                        *reinterpret_cast<h4*>(dvb + (int64_t)(t0 + jj) * v_stride + ws * DS + 16 * ct + 4 * G) = to_h4(dvacc[ct][jt]);
                }
            }
            }

            // carried sums
#pragma unroll
            for (int is = 0; is < (CAUSAL ? 2 : 0); ++is) {
                if (do_dk) {
                    h8 ghi, glo;   // r (m=k) += Q^T gz
                    f8_to_operand(*reinterpret_cast<const f4*>(gzs + is * 32 + 8 * G),
                                  *reinterpret_cast<const f4*>(gzs + is * 32 + 8 * G + 4), ghi, glo);
#pragma unroll
                    for (int kt = 0; kt < NKT; ++kt) racc[kt] = mfma32(qf[kt][is], ghi, racc[kt]);
#pragma unroll
                    for (int kt = 0; kt < NKT; ++kt) racc[kt] = mfma32(qf[kt][is], glo, racc[kt]);
#pragma unroll
                    for (int ct = 0; ct < NCT; ++ct) {
                        h8 gf = col8(Gs, LDV, is * 32, 16 * ct, lane);
#pragma unroll
                        for (int kt = 0; kt < NKT; ++kt) RT[ct][kt] = mfma32(gf, qf[kt][is], RT[ct][kt]);
                    }
                }
                if (do_dv) {
#pragma unroll
                    for (int kt = 0; kt < NKT2; ++kt) {
                        h8 qa = col8(Qs, LDQ, is * 32, 16 * kt, lane);
#pragma unroll
                        for (int ct = 0; ct < NCT2; ++ct) RR[kt][ct] = mfma32(qa, gf2[ct][is], RR[kt][ct]);
                    }
                }
            }
        }
        __syncthreads();
    }
}


// ---------------------------------------------------------------------------
// backward, reverse-in-time sweep with dK and dV in separate workgroups (causal only).
// The two gradients share the masked tiles' inputs but nothing else:
//     dK = P^T Q + V R^T + 1 r^T   reads q, v, g   carries R^T (d x K) and r
//     dV = A^T (G/den) + K R       reads q, k, g   carries R   (K x d)
// so a workgroup of either role holds one copy of R instead of two and loads three of the
// four operands; the two roles of a (sequence, segment) run side by side on one CU where
// LDS and registers allow, each hiding the other's LDS and memory latency.
// grid = 2 * N * nseg: blocks [0, N*nseg) compute dK, blocks [N*nseg, 2*N*nseg) compute dV.
// ---------------------------------------------------------------------------
template <int KD, int DH, int NW>
struct DkDvRoleCfg {
    using Base = CausalCfg<KD, DH, NW>;
    static constexpr int C = Base::C, LDQ = Base::LDQ, LDV = Base::LDV, LDA = Base::LDA;
    static constexpr size_t kDkLds = (size_t)(C * LDQ + 2 * C * LDV + C * LDA) * 2 + (size_t)(KD + C) * 4;
    static constexpr size_t kDvLds = (size_t)(2 * C * LDQ + C * LDV + C * LDA) * 2;
    static constexpr size_t kLds = kDkLds > kDvLds ? kDkLds : kDvLds;
};

template <int KD, int DH, int NW>
__device__ __forceinline__ void dkdv_role_dk(
    unsigned char* smem_raw, int bid, const half_t* __restrict__ q, const half_t* __restrict__ v,
    const half_t* __restrict__ g, half_t* __restrict__ dk, const float* __restrict__ wsR,
    const float* __restrict__ wsr, const float* __restrict__ den_ws, const float* __restrict__ gz_ws, int T,
    int N, int nseg, int seg_len, int prefixed) {
    using Cfg = CausalCfg<KD, DH, NW>;
    constexpr int NT = Cfg::NT;
    constexpr int C = Cfg::C, LDQ = Cfg::LDQ, LDV = Cfg::LDV, LDA = Cfg::LDA, KS = KD / NW;
    constexpr int NKT = KS / 16, NCT = DH / 16, JPW = Cfg::JPW;
    constexpr int PPRV = DH / 8, VP = ChunkRegs<DH, NT>::kPieces;
    static_assert(KD % (16 * NW) == 0, "feature rows do not split over the waves");
    half_t* Qs = reinterpret_cast<half_t*>(smem_raw);
    half_t* Vs = Qs + C * LDQ;
    half_t* Gs = Vs + C * LDV;       // G / den
    half_t* PTs = Gs + C * LDV;      // PT[j][i] = P[i][j]
    float* rs = reinterpret_cast<float*>(PTs + C * LDA);
    float* gzs = rs + KD;

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int row = lane & 15, G = lane >> 4;
    const int rb = w & 3, half = w >> 2;
    int n, seg;
    seq_seg_of_block(bid, N, nseg, n, seg);
    const int t_begin = seg * seg_len;
    const int t_end = min(T, t_begin + seg_len);
    const int64_t k_stride = (int64_t)N * KD, v_stride = (int64_t)N * DH;
    const half_t* qb = q + (int64_t)n * KD;
    const half_t* vb = v + (int64_t)n * DH;
    const half_t* gb = g + (int64_t)n * DH;
    half_t* dkb = dk + (int64_t)n * KD;

    f4 RT[NCT][NKT];   // element (c = 16ct+4G+e, k = w*KS+16kt+i)
#pragma unroll
    for (int a = 0; a < NCT; ++a)
#pragma unroll
        for (int b = 0; b < NKT; ++b) RT[a][b] = f4_zero();
    f4 racc[NKT];
#pragma unroll
    for (int b = 0; b < NKT; ++b) racc[b] = f4_zero();
    for (int s = prefixed ? seg : seg + 1; s < (prefixed ? seg + 1 : nseg); ++s) {
        const float* ri = wsR + ((int64_t)(n * nseg + s) * KD) * DH;
#pragma unroll
        for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
            for (int kt = 0; kt < NKT; ++kt)
                RT[ct][kt] += *reinterpret_cast<const f4*>(ri + (w * KS + 16 * kt + row) * DH + 16 * ct + 4 * G);
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt)
            racc[kt] += *reinterpret_cast<const f4*>(wsr + (int64_t)(n * nseg + s) * KD + w * KS + 16 * kt + 4 * G);
    }

    ChunkRegs<KD, NT> rq;
    ChunkRegs<DH, NT> rv, rg;
    float inv_den[VP];
    float gz_next = 0.f;
    auto prefetch = [&](int t0) {
        const int rows = t_end - t0;
        chunk_g2r<KD, NT>(rq, qb + (int64_t)t0 * k_stride, k_stride, rows, tid);
        chunk_g2r<DH, NT>(rv, vb + (int64_t)t0 * v_stride, v_stride, rows, tid);
        chunk_g2r<DH, NT>(rg, gb + (int64_t)t0 * v_stride, v_stride, rows, tid);
#pragma unroll
        for (int it = 0; it < VP; ++it) {
            const int r_ = min((tid + NT * it) / PPRV, rg.rows - 1);
            inv_den[it] = den_ws[(int64_t)(t0 + r_) * N + n];
        }
        gz_next = gz_ws[(int64_t)(t0 + min(tid & (C - 1), rg.rows - 1)) * N + n];
    };
    const int n_chunks = (t_end - t_begin + C - 1) / C;
    prefetch(t_begin + (n_chunks - 1) * C);
    for (int ci = n_chunks - 1; ci >= 0; --ci) {
        const int t0 = t_begin + ci * C;
        chunk_r2s<KD, NT>(rq, Qs, LDQ, tid);
        chunk_r2s<DH, NT>(rv, Vs, LDV, tid);
#pragma unroll
        for (int it = 0; it < VP; ++it) inv_den[it] = rcp_nr(fmaxf(inv_den[it], 1.0f));
        chunk_r2s_scaled<DH, NT>(rg, inv_den, Gs, LDV, tid);
        if (tid < C) gzs[tid] = tid < rg.rows ? gz_next : 0.f;
        if (row == 0) {
#pragma unroll
            for (int kt = 0; kt < NKT; ++kt) *reinterpret_cast<f4*>(rs + w * KS + 16 * kt + 4 * G) = racc[kt];
        }
        __syncthreads();
        if (ci > 0) prefetch(t0 - C);

        // ---- P tiles (m=i, n=j) for column block rb, rows 16*(half*JPW + a)
        {
            f4 p_[JPW];
#pragma unroll
            for (int a = 0; a < JPW; ++a) p_[a] = f4_zero();
#pragma unroll
            for (int cs = 0; cs < DH / 32; ++cs) {
                h8 bv = row8(Vs, LDV, 16 * rb + row, cs * 32, G);
#pragma unroll
                for (int a = 0; a < JPW; ++a)
                    p_[a] = mfma32(row8(Gs, LDV, 16 * (half * JPW + a) + row, cs * 32, G), bv, p_[a]);
            }
            const int j = 16 * rb + row;
#pragma unroll
            for (int a = 0; a < JPW; ++a) {
                const int it = half * JPW + a;
                h4 pv;
                f4 gzv = *reinterpret_cast<const f4*>(gzs + 16 * it + 4 * G);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int i = 16 * it + 4 * G + e;
                    pv[e] = (i >= j) ? (half_t)(p_[a][e] + gzv[e]) : (half_t)0.f;
                }
                *reinterpret_cast<h4*>(PTs + j * LDA + 16 * it + 4 * G) = pv;
            }
        }
        __syncthreads();

        // ---- dK^T tiles (m=k, n=j) and the carried sums
        {
            h8 qf[NKT][2];
#pragma unroll
            for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
                for (int is = 0; is < 2; ++is) qf[kt][is] = col8(Qs, LDQ, is * 32, w * KS + 16 * kt, lane);
            f4 dkacc[NKT][4];
#pragma unroll
            for (int kt = 0; kt < NKT; ++kt) {
                f4 rv4 = *reinterpret_cast<const f4*>(rs + w * KS + 16 * kt + 4 * G);
#pragma unroll
                for (int jt = 0; jt < 4; ++jt) {
                    f4 acc = rv4;
                    if (jt < 2) acc = mfma32(qf[kt][0], row8(PTs, LDA, 16 * jt + row, 0, G), acc);
                    acc = mfma32(qf[kt][1], row8(PTs, LDA, 16 * jt + row, 32, G), acc);
                    dkacc[kt][jt] = acc;
                }
            }
#pragma unroll
            for (int cs = 0; cs < DH / 32; ++cs) {
                h8 bvv[4];
#pragma unroll
                for (int jt = 0; jt < 4; ++jt) bvv[jt] = row_split8(Vs, LDV, 16 * jt + row, cs * 32, G);
                __builtin_amdgcn_sched_barrier(0);     // keep the reads ahead of the conversion
                h8 hi[NKT];
#pragma unroll
                for (int kt = 0; kt < NKT; ++kt) hi[kt] = acc_to_operand_rn(RT[2 * cs][kt], RT[2 * cs + 1][kt]);
#pragma unroll
                for (int jt = 0; jt < 4; ++jt) {
#pragma unroll
                    for (int kt = 0; kt < NKT; ++kt) dkacc[kt][jt] = mfma32(hi[kt], bvv[jt], dkacc[kt][jt]);
                }
            }
#pragma unroll
            for (int jt = 0; jt < 4; ++jt) {
                const int jj = 16 * jt + row;
                if (t0 + jj < t_end) {
#pragma unroll
                    for (int kt = 0; kt < NKT; ++kt)
                        *reinterpret_cast<h4*>(dkb + (int64_t)(t0 + jj) * k_stride + w * KS + 16 * kt + 4 * G) = to_h4(dkacc[kt][jt]);
                }
            }
#pragma unroll
            for (int is = 0; is < 2; ++is) {
                h8 ghi, glo;   // r (m=k) += Q^T gz
                f8_to_operand(*reinterpret_cast<const f4*>(gzs + is * 32 + 8 * G),
                              *reinterpret_cast<const f4*>(gzs + is * 32 + 8 * G + 4), ghi, glo);
#pragma unroll
                for (int kt = 0; kt < NKT; ++kt) racc[kt] = mfma32(qf[kt][is], ghi, racc[kt]);
#pragma unroll
                for (int kt = 0; kt < NKT; ++kt) racc[kt] = mfma32(qf[kt][is], glo, racc[kt]);
#pragma unroll
                for (int ct = 0; ct < NCT; ++ct) {
                    h8 gf = col8(Gs, LDV, is * 32, 16 * ct, lane);
#pragma unroll
                    for (int kt = 0; kt < NKT; ++kt) RT[ct][kt] = mfma32(gf, qf[kt][is], RT[ct][kt]);
                }
            }
        }
        __syncthreads();
    }
}

template <int KD, int DH, int NW>
__device__ __forceinline__ void dkdv_role_dv(
    unsigned char* smem_raw, int bid, const half_t* __restrict__ q, const half_t* __restrict__ k,
    const half_t* __restrict__ g, half_t* __restrict__ dv, const float* __restrict__ wsR,
    const float* __restrict__ den_ws, int T, int N, int nseg, int seg_len, int prefixed) {
    using Cfg = CausalCfg<KD, DH, NW>;
    constexpr int NT = Cfg::NT;
    constexpr int C = Cfg::C, LDQ = Cfg::LDQ, LDV = Cfg::LDV, LDA = Cfg::LDA, DS = DH / NW;
    constexpr int NKT2 = KD / 16, NCT2 = DS / 16, JPW = Cfg::JPW;
    constexpr int PPRV = DH / 8, VP = ChunkRegs<DH, NT>::kPieces;
    static_assert(DH % (16 * NW) == 0, "value columns do not split over the waves");
    half_t* Qs = reinterpret_cast<half_t*>(smem_raw);
    half_t* Ks = Qs + C * LDQ;
    half_t* Gs = Ks + C * LDQ;       // G / den
    half_t* ATs = Gs + C * LDV;      // AT[j][i] = A[i][j]

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int row = lane & 15, G = lane >> 4;
    const int rb = w & 3, half = w >> 2;
    int n, seg;
    seq_seg_of_block(bid, N, nseg, n, seg);
    const int t_begin = seg * seg_len;
    const int t_end = min(T, t_begin + seg_len);
    const int64_t k_stride = (int64_t)N * KD, v_stride = (int64_t)N * DH;
    const half_t* qb = q + (int64_t)n * KD;
    const half_t* kb = k + (int64_t)n * KD;
    const half_t* gb = g + (int64_t)n * DH;
    half_t* dvb = dv + (int64_t)n * DH;

    f4 RR[NKT2][NCT2];   // element (k = 16kt+4G+e, c = w*DS+16ct+i)
#pragma unroll
    for (int a = 0; a < NKT2; ++a)
#pragma unroll
        for (int b = 0; b < NCT2; ++b) RR[a][b] = f4_zero();
    for (int s = prefixed ? seg : seg + 1; s < (prefixed ? seg + 1 : nseg); ++s) {
        const float* ri = wsR + ((int64_t)(n * nseg + s) * KD) * DH;
#pragma unroll
        for (int kt = 0; kt < NKT2; ++kt)
#pragma unroll
            for (int ct = 0; ct < NCT2; ++ct)
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    RR[kt][ct][e] += ri[(16 * kt + 4 * G + e) * DH + w * DS + 16 * ct + row];
    }

    ChunkRegs<KD, NT> rq, rk;
    ChunkRegs<DH, NT> rg;
    float inv_den[VP];
    // the next chunk is requested in two parts, k after the first barrier, q, g, den after the second
    auto prefetch_a = [&](int t0) {
        chunk_g2r<KD, NT>(rk, kb + (int64_t)t0 * k_stride, k_stride, t_end - t0, tid);
    };
    auto prefetch_b = [&](int t0) {
        const int rows = t_end - t0;
        chunk_g2r<KD, NT>(rq, qb + (int64_t)t0 * k_stride, k_stride, rows, tid);
        chunk_g2r<DH, NT>(rg, gb + (int64_t)t0 * v_stride, v_stride, rows, tid);
#pragma unroll
        for (int it = 0; it < VP; ++it) {
            const int r_ = min((tid + NT * it) / PPRV, rg.rows - 1);
            inv_den[it] = den_ws[(int64_t)(t0 + r_) * N + n];
        }
    };
    const int n_chunks = (t_end - t_begin + C - 1) / C;
    prefetch_a(t_begin + (n_chunks - 1) * C);
    prefetch_b(t_begin + (n_chunks - 1) * C);
    for (int ci = n_chunks - 1; ci >= 0; --ci) {
        const int t0 = t_begin + ci * C;
        chunk_r2s<KD, NT>(rk, Ks, LDQ, tid);
        chunk_r2s<KD, NT>(rq, Qs, LDQ, tid);
#pragma unroll
        for (int it = 0; it < VP; ++it) inv_den[it] = rcp_nr(fmaxf(inv_den[it], 1.0f));
        chunk_r2s_scaled<DH, NT>(rg, inv_den, Gs, LDV, tid);
        __syncthreads();
        if (ci > 0) prefetch_a(t0 - C);

        // ---- A tiles (m=i, n=j) for column block rb, rows 16*(half*JPW + a)
        {
            f4 a_[JPW];
#pragma unroll
            for (int a = 0; a < JPW; ++a) a_[a] = f4_zero();
#pragma unroll
            for (int ks = 0; ks < KD / 32; ++ks) {
                h8 bk = row8(Ks, LDQ, 16 * rb + row, ks * 32, G);
#pragma unroll
                for (int a = 0; a < JPW; ++a)
                    a_[a] = mfma32(row8(Qs, LDQ, 16 * (half * JPW + a) + row, ks * 32, G), bk, a_[a]);
            }
            const int j = 16 * rb + row;
#pragma unroll
            for (int a = 0; a < JPW; ++a) {
                const int it = half * JPW + a;
                h4 av;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int i = 16 * it + 4 * G + e;
                    av[e] = (i >= j) ? (half_t)a_[a][e] : (half_t)0.f;
                }
                *reinterpret_cast<h4*>(ATs + j * LDA + 16 * it + 4 * G) = av;
            }
        }
        __syncthreads();
        if (ci > 0) prefetch_b(t0 - C);

        // ---- dV^T tiles (m=c, n=j) and the carried sum
        {
            h8 gf2[NCT2][2];
#pragma unroll
            for (int ct = 0; ct < NCT2; ++ct)
#pragma unroll
                for (int is = 0; is < 2; ++is) gf2[ct][is] = col8(Gs, LDV, is * 32, w * DS + 16 * ct, lane);
            f4 dvacc[NCT2][4];
#pragma unroll
            for (int ct = 0; ct < NCT2; ++ct)
#pragma unroll
                for (int jt = 0; jt < 4; ++jt) {
                    f4 acc = f4_zero();
                    if (jt < 2) acc = mfma32(gf2[ct][0], row8(ATs, LDA, 16 * jt + row, 0, G), acc);
                    acc = mfma32(gf2[ct][1], row8(ATs, LDA, 16 * jt + row, 32, G), acc);
                    dvacc[ct][jt] = acc;
                }
#pragma unroll
            for (int ks = 0; ks < KD / 32; ++ks) {
                h8 bkk[4];
#pragma unroll
                for (int jt = 0; jt < 4; ++jt) bkk[jt] = row_split8(Ks, LDQ, 16 * jt + row, ks * 32, G);
                __builtin_amdgcn_sched_barrier(0);     // keep the reads ahead of the conversion
                h8 hi[NCT2];
#pragma unroll
                for (int ct = 0; ct < NCT2; ++ct) hi[ct] = acc_to_operand_rn(RR[2 * ks][ct], RR[2 * ks + 1][ct]);
#pragma unroll
                for (int jt = 0; jt < 4; ++jt) {
#pragma unroll
                    for (int ct = 0; ct < NCT2; ++ct) dvacc[ct][jt] = mfma32(hi[ct], bkk[jt], dvacc[ct][jt]);
                }
            }
#pragma unroll
            for (int jt = 0; jt < 4; ++jt) {
                const int jj = 16 * jt + row;
                if (t0 + jj < t_end) {
#pragma unroll
                    for (int ct = 0; ct < NCT2; ++ct)
                        *reinterpret_cast<h4*>(dvb + (int64_t)(t0 + jj) * v_stride + w * DS + 16 * ct + 4 * G) = to_h4(dvacc[ct][jt]);
                }
            }
#pragma unroll
            for (int is = 0; is < 2; ++is)
#pragma unroll
                for (int kt = 0; kt < NKT2; ++kt) {
                    h8 qa = col8(Qs, LDQ, is * 32, 16 * kt, lane);
#pragma unroll
                    for (int ct = 0; ct < NCT2; ++ct) RR[kt][ct] = mfma32(qa, gf2[ct][is], RR[kt][ct]);
                }
        }
        __syncthreads();
    }
}

template <int KD, int DH, int NW>
__global__ __launch_bounds__(64 * NW) void k_causal_bwd_dkdv_roles(
    const half_t* __restrict__ q, const half_t* __restrict__ k, const half_t* __restrict__ v,
    const half_t* __restrict__ g, half_t* __restrict__ dk, half_t* __restrict__ dv,
    const float* __restrict__ wsR, const float* __restrict__ wsr, const float* __restrict__ den_ws,
    const float* __restrict__ gz_ws, int T, int N, int nseg, int seg_len, int prefixed,
    const int* __restrict__ hdr_in, PlanWords plan) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    const int nsq = N * nseg;
    if (!plan_matches(hdr_in, plan)) {
        const bool is_dk = (int)blockIdx.x < nsq;
        int n, seg;
        seq_seg_of_block(is_dk ? blockIdx.x : blockIdx.x - nsq, N, nseg, n, seg);
        const int t_begin = seg * seg_len, t_end = min(T, t_begin + seg_len);
        if (is_dk) poison_rows<KD>(dk + (int64_t)n * KD, (int64_t)N * KD, t_begin, t_end);
        else poison_rows<DH>(dv + (int64_t)n * DH, (int64_t)N * DH, t_begin, t_end);
        return;
    }
    if ((int)blockIdx.x < nsq)
        dkdv_role_dk<KD, DH, NW>(smem_raw, blockIdx.x, q, v, g, dk, wsR, wsr, den_ws, gz_ws, T, N, nseg, seg_len, prefixed);
    else
        dkdv_role_dv<KD, DH, NW>(smem_raw, blockIdx.x - nsq, q, k, g, dv, wsR, den_ws, T, N, nseg, seg_len, prefixed);
}

// ---------------------------------------------------------------------------
// Exclusive scan of the segment totals over the segment axis, in place.  A consumer of segment
// s otherwise adds up the totals of every earlier (forward sweeps) or later (reverse sweep)
// segment itself, (nseg - 1) / 2 state reads on average per workgroup; with many segments of a
// large state one pass over the totals is cheaper.
//   a [N][nseg][Ma], b [N][nseg][Mb] fp32 (Ma, Mb multiples of 4; b may be NULL)
//   REVERSE = false: slot s <- sum of slots s' < s; slot nseg - 1 is never read (no total is
//                    stored for the last segment)
//   REVERSE = true : slot s <- sum of slots s' > s; slot 0 is never read
// grid = (ceil((Ma + Mb) / 4 / 256), N); one thread owns four consecutive elements of every slot.
// ---------------------------------------------------------------------------
constexpr int kMaxSegments = 16;

template <bool REVERSE>
__global__ __launch_bounds__(kThreads) void k_totals_scan(float* __restrict__ a, int64_t Ma, float* __restrict__ b,
                                                          int64_t Mb, int nseg) {
    int64_t e = ((int64_t)blockIdx.x * kThreads + threadIdx.x) * 4;
    float* base;
    int64_t M;
    if (e < Ma) {
        base = a; M = Ma;
    } else {
        e -= Ma;
        if (!b || e >= Mb) return;
        base = b; M = Mb;
    }
    float* col = base + (int64_t)blockIdx.y * nseg * M + e;
    f4 t[kMaxSegments];
#pragma unroll
    for (int s = 0; s < kMaxSegments; ++s) {
        const bool live = REVERSE ? (s >= 1 && s < nseg) : (s < nseg - 1);
        t[s] = f4_zero();
        if (live) t[s] = *reinterpret_cast<const f4*>(col + (int64_t)s * M);
    }
    f4 run = f4_zero();
    if (REVERSE) {
#pragma unroll
        for (int s = kMaxSegments - 1; s >= 0; --s) {
            if (s < nseg) {
                *reinterpret_cast<f4*>(col + (int64_t)s * M) = run;
                run[0] += t[s][0]; run[1] += t[s][1]; run[2] += t[s][2]; run[3] += t[s][3];
            }
        }
    } else {
#pragma unroll
        for (int s = 0; s < kMaxSegments; ++s) {
            if (s < nseg) {
                *reinterpret_cast<f4*>(col + (int64_t)s * M) = run;
                run[0] += t[s][0]; run[1] += t[s][1]; run[2] += t[s][2]; run[3] += t[s][3];
            }
        }
    }
}

}  // namespace rfa
