// Causal random-feature attention backward without time segments (gfx950): parallelism from
// slices of the state instead of from cutting the sequence.
//
// The chunked scan of rfa_causal.h cuts a sequence into time segments so that bsz * heads
// sequences fill the GPU; every segment then needs the state at its first step, which costs a
// pass over q, g for the segment totals, and two sweeps over the sequence (dQ needs the sum over
// earlier steps, dK and dV the sum over later ones).  Here a workgroup walks a whole sequence
// and owns a slice of the state:
//
//   feature slice  [koff, koff + 64) of phi:   dQ[:, slice], dK[:, slice]
//       carries S[slice, :] and R[slice, :]   (reads g, out, v whole; q, k slice)
//   value slice    [coff, coff + 64) of v:      dV[:, slice]
//       carries R[:, slice]                    (reads q, k whole; g slice)
//
// with  S = sum_{s <= t} phi_k[s] (x) v[s],  R = sum_{s > t} phi_q[s] (x) g^[s],  g^ = g / den
// (rfa.py:66-103).  Both run backwards in time.  R grows as the sweep proceeds; S of the chunk
// before the current one is the forward's final state minus what the sweep has passed, so the
// backward needs no totals pass, no second sweep, and reads every chunk of q, k, v, g, out once
// from HBM (the slices of one sequence sit on one XCD and walk in step, so the rows they share
// come out of that L2).  The dQ/dK slices and the dV slices of a sequence are separate
// workgroups of one launch.
//
// Formulas per 64-step chunk (Q, K: 64 x KD;  V, G^: 64 x DH;  gz_i = [den_raw_i > 1] * -(g_i . out_i) / den_i):
//     P  = tril(G^ V^T + gz 1^T)              A = tril(Q K^T)
//     dQ = P K + G^ S_prev^T + gz z_prev^T     (S_prev, z_prev: state before the chunk)
//     dK = P^T Q + V R_next^T + 1 r_next^T     (R_next, r_next: sums over later chunks)
//     dV = A^T G^ + K R_next
//
// A workgroup is a pipeline of 8 waves, two per SIMD.  Waves 0-3 (loader group) bring chunk c from
// HBM into LDS and form its masked tile matrix (P or A^T); waves 4-7 work on chunk c + 1 (the one
// staged an iteration earlier), each on 32 features or 32 value columns: waves 4, 5 dQ and waves
// 6, 7 dK in the feature-slice role, the two halves of the dV rows in the value-slice role.  The
// groups meet at two workgroup barriers per chunk; the chunk arrays and the tile matrix are
// double buffered.  Only the loader group issues loads and only the others issue stores, so
// neither kind waits for the other.  What bounds the kernel is instruction issue and dependent
// latency with two waves per SIMD, not bytes: the loader's per-element work (row scaling, row
// dot products, masks) is therefore written with the fewest vector instructions that give the
// same rounding (mixed-precision multiply-add, two-element dot products, lane permutes inside
// the vector unit), and addresses are a wave-uniform base plus one 32-bit offset per lane.
#pragma once
#include <type_traits>

#include "rfa_common.h"

namespace rfa {

constexpr int kSliceWidth = 64;     // features (dQ/dK role) or value columns (dV role) per workgroup
constexpr int kSlicedThreads = 512; // 8 waves: loader group (4) + four product waves
constexpr int kGroupThreads = 256;  // threads per group

// Workgroup index -> (sequence, role).  The wps workgroups of a sequence get indices that are
// equal mod kXcds, i.e. the same XCD, and consecutive positions there.
__device__ __forceinline__ void seq_role_of_block(int b, int wps, int& n, int& role) {
    const int xcd = b % kXcds, l = b / kXcds;
    role = l % wps;
    n = kXcds * (l / wps) + xcd;
}

// threads per workgroup for feature slices of SW: the loader group and SW / 32 product waves each for dQ and dK
constexpr int sliced_threads(int SW) { return 256 + 64 * 2 * (SW / 32); }

template <int KD, int DH, int SW = kSliceWidth>
struct SlicedBwdCfg {
    static_assert(SW % 64 == 0 && KD % SW == 0, "feature slice width");
    static constexpr int C = kChunk, KSL = SW, CSL = kSliceWidth;
    static constexpr int NA = KD / KSL;             // dQ/dK workgroups per sequence
    static constexpr int NB = DH / CSL;             // dV workgroups per sequence
    static constexpr int NPW = KSL / 32;            // product waves per output (dQ, dK) of the feature-slice role
    static constexpr int kThreads = sliced_threads(SW);   // >= the 512 of the dV role
    static constexpr int LDS_ = KSL + lds_pad(KSL); // row stride of a feature-slice array
    static constexpr int LDG_ = CSL + lds_pad(CSL); // row stride of a value-slice array
    static constexpr int LDQ = KD + lds_pad(KD);
    static constexpr int LDV = DH + lds_pad(DH);
    static constexpr int LDA = C + 8;
    // dQ/dK role, per stage: Q slice | K slice | V | G^ | P | gz
    static constexpr size_t kStageA = (size_t)(2 * C * LDS_ + 2 * C * LDV + C * LDA) * 2 + C * 4;
    // dV role, per stage: Q | K | G^ slice | A^T
    static constexpr size_t kStageB = (size_t)(2 * C * LDQ + C * LDG_ + C * LDA) * 2;
    static constexpr size_t kLds = 2 * (kStageA > kStageB ? kStageA : kStageB);
    static_assert(kStageA % 16 == 0 && kStageB % 16 == 0, "stage alignment");
};

__device__ __forceinline__ void wg_sync() { __syncthreads(); }

// ---------------------------------------------------------------------------
// dQ, dK for features [koff, koff + 64) of one sequence.
//   loader group: stages Q, K slices, V, G^ = G / den and gz, then P = tril(G^ V^T + gz 1^T)
//   dQ group: wave wf owns features kw = koff + 16 wf .. + 15; NS[ct] = -S^T tile
//             (c = 16ct + 4G + e, k = kw + i), nz = -z tile (k = kw + 4G + e).  S and z are
//             carried negated so that the MFMA can step them backwards by adding K^T V.
//   dK group: same features; RT[ct] = R^T tile, r as a tile.
// ---------------------------------------------------------------------------
template <int KD, int DH, int SW>
__device__ __forceinline__ void sliced_bwd_dqdk(
    unsigned char* smem, int n, int koff, const half_t* __restrict__ q, const half_t* __restrict__ k,
    const half_t* __restrict__ v, const half_t* __restrict__ g, const half_t* __restrict__ o,
    const float* __restrict__ den_raw, half_t* __restrict__ dq, half_t* __restrict__ dk,
    const float* __restrict__ final_s, const float* __restrict__ final_z, int T, int N) {
    using Cfg = SlicedBwdCfg<KD, DH, SW>;
    constexpr int NT = kGroupThreads, C = Cfg::C, KSL = Cfg::KSL, NPW = Cfg::NPW;
    constexpr int LDK = Cfg::LDS_, LDV = Cfg::LDV, LDA = Cfg::LDA;
    [[maybe_unused]] constexpr int kDqTick = 256, kDkTick = 256 + 64 * NPW;     // first thread of the dQ / dK waves (phase timing)
    constexpr int NCT = DH / 16;
    constexpr int PPR = DH / 8, VP = ChunkRegs<DH, NT>::kPieces;
    constexpr size_t kStage = Cfg::kLds / 2;

    const int lane = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int grp = w < 4 ? 0 : 1 + (w - 4) / NPW;      // loader | NPW dQ waves | NPW dK waves
    const int wf = w & 3;                       // loader: row block of the P tiles
    const int tid = (w & 3) * 64 + lane;        // thread inside the loader group
    const int row = lane & 15, G = lane >> 4;
    const int kl0 = 32 * ((w - 4) % NPW);       // product waves: first of this wave's 32 features, local to the slice arrays
    const unsigned out_lane_off = (unsigned)row * (unsigned)(N * KD * 2) + 8u * G;   // bytes: row `row` of a 16-step tile, 4 halves from 4G
    const int64_t k_stride = (int64_t)N * KD, v_stride = (int64_t)N * DH;
    const int n_chunks = (T + C - 1) / C;
    RFA_TICK_INIT();

    struct Stage { half_t *Qs, *Ks, *Vs, *Gs, *Ps; float* gzs; };
    auto stage_of = [&](int i) __attribute__((always_inline)) {
        Stage st;
        st.Qs = reinterpret_cast<half_t*>(smem + (i & 1) * kStage);
        st.Ks = st.Qs + C * LDK;
        st.Vs = st.Ks + C * LDK;
        st.Gs = st.Vs + C * LDV;                 // G / den
        st.Ps = st.Gs + C * LDV;
        st.gzs = reinterpret_cast<float*>(st.Ps + C * LDA);
        return st;
    };

    // Iteration i = 0 .. n_chunks: the loader group stages chunk n_chunks - 1 - i (none in the last
    // iteration), the product groups work on chunk n_chunks - i (none in the first).  Every wave
    // passes exactly two barriers per iteration.
    if (grp == 0) {
        const half_t* qb = q + (int64_t)n * KD + koff;
        const half_t* kb = k + (int64_t)n * KD + koff;
        const half_t* vb = v + (int64_t)n * DH;
        const half_t* gb = g + (int64_t)n * DH;
        const half_t* ob = o + (int64_t)n * DH;
        RowPtrs<KSL, NT> pq, pk;
        RowPtrs<DH, NT> pv, pg, po;
        pq.init(qb, k_stride, tid);
        pk.init(kb, k_stride, tid);
        pv.init(vb, v_stride, tid);
        pg.init(gb, v_stride, tid);
        po.init(ob, v_stride, tid);
        // Two register sets of chunk rows: while chunk c is staged, the rows of chunks c - 1 and
        // c - 2 are on their way, so a load has two chunk periods to arrive.
        struct RowSet {
            ChunkRegs<KSL, NT> rq, rk;
            ChunkRegs<DH, NT> rv, rg, ro;
            float dn[VP];
        };
        RowSet s0, s1;
        // which halves of this lane's P elements lie on or below the diagonal: element (i = 16wf + row,
        // j = 16jt + 4G + e) is kept when j <= i
        uint2 tril_mask[4];
#pragma unroll
        for (int jt = 0; jt < 4; ++jt) {
            auto keep = [&](int e) { return (16 * jt + 4 * G + e <= 16 * wf + row) ? 0xffffu : 0u; };
            tril_mask[jt].x = keep(0) | (keep(1) << 16);
            tril_mask[jt].y = keep(2) | (keep(3) << 16);
        }
        // the last chunk of the sequence may be short: clamped row addresses
        auto prefetch_ragged = [&](RowSet& r, int c) __attribute__((always_inline)) {
            const int t0 = c * C, rows = T - t0;
            chunk_g2r<KSL, NT>(r.rq, qb + (int64_t)t0 * k_stride, k_stride, rows, tid);
            chunk_g2r<KSL, NT>(r.rk, kb + (int64_t)t0 * k_stride, k_stride, rows, tid);
            chunk_g2r<DH, NT>(r.rv, vb + (int64_t)t0 * v_stride, v_stride, rows, tid);
            chunk_g2r<DH, NT>(r.rg, gb + (int64_t)t0 * v_stride, v_stride, rows, tid);
            chunk_g2r<DH, NT>(r.ro, ob + (int64_t)t0 * v_stride, v_stride, rows, tid);
#pragma unroll
            for (int it = 0; it < VP; ++it) {
                const int r_ = min((tid + NT * it) / PPR, r.rg.rows - 1);
                r.dn[it] = den_raw[(int64_t)(t0 + r_) * N + n];
            }
        };
        // a full chunk; c may be a chunk that is never used (the caller clamps it to an existing
        // one: no branch around the loads)
        auto prefetch = [&](RowSet& r, int c) __attribute__((always_inline)) {
            const int64_t t0 = (int64_t)c * C;
            pq.load_full(r.rq, t0 * k_stride);
            pk.load_full(r.rk, t0 * k_stride);
            pv.load_full(r.rv, t0 * v_stride);
            pg.load_full(r.rg, t0 * v_stride);
            po.load_full(r.ro, t0 * v_stride);
#pragma unroll
            for (int it = 0; it < VP; ++it) r.dn[it] = den_raw[(t0 + (tid + NT * it) / PPR) * N + n];
        };
        // rows in `r` -> LDS: Q, K slices, V, G^ = G / den, gz from g . out (the PPR lanes holding
        // one row are adjacent); barrier; chunk c_next requested into `r`; P tiles; barrier
        auto stage_chunk = [&](int i, RowSet& r, int c_next, bool do_prefetch) __attribute__((always_inline)) {
            const Stage st = stage_of(i);
            chunk_r2s<KSL, NT>(r.rq, st.Qs, LDK, tid);
            chunk_r2s<KSL, NT>(r.rk, st.Ks, LDK, tid);
            chunk_r2s<DH, NT>(r.rv, st.Vs, LDV, tid);
#pragma unroll
            for (int it = 0; it < VP; ++it) {
                const int pc = tid + NT * it;
                const int r_ = pc / PPR, c8 = pc % PPR;
                const float dot = sum_adjacent<PPR>(dot_h8(r.rg.v[it], r.ro.v[it]));
                const bool valid = r_ < r.rg.rows;
                const float inv = valid ? rcp_nr(fmaxf(r.dn[it], 1.0f)) : 0.f;
                const float gzv = (valid && r.dn[it] > 1.0f) ? -dot * inv : 0.f;
                *reinterpret_cast<uint4*>(st.Gs + r_ * LDV + c8 * 8) = scale_h8(r.rg.v[it], inv);
                if (c8 == 0) st.gzs[r_] = gzv;
            }
            RFA_TICK_AT(1, 0);
            wg_sync();
            RFA_TICK_AT(2, 0);
            if (do_prefetch) prefetch(r, c_next);
            RFA_TICK_AT(3, 0);
            // P = tril(G^ V^T + gz 1^T) as X^T tiles (m = j, n = i): row block wf, all four column
            // tiles, no branch around the products (the element mask j <= i zeroes what lies above
            // the diagonal; a product under a wave-uniform branch whose result is read right after
            // the join has been seen to be read too early)
            {
                const int ii = 16 * wf + row;
                const float gzi = st.gzs[ii];
                // gz enters as the accumulator the products start from (column i of X^T is this lane)
                f4 gz4;
                gz4[0] = gzi; gz4[1] = gzi; gz4[2] = gzi; gz4[3] = gzi;
                f4 xt[4];
#pragma unroll
                for (int jt = 0; jt < 4; ++jt) xt[jt] = gz4;
#pragma unroll
                for (int cs = 0; cs < DH / 32; ++cs) {
                    const h8 bg = row8(st.Gs, LDV, ii, cs * 32, G);
#pragma unroll
                    for (int jt = 0; jt < 4; ++jt) xt[jt] = mfma32(row8(st.Vs, LDV, 16 * jt + row, cs * 32, G), bg, xt[jt]);
                }
#pragma unroll
                for (int jt = 0; jt < 4; ++jt) {
                    // rounded pairs, then the halves above the diagonal cleared by a mask that is set up once
                    uint2 pv_;
                    pv_.x = pack_h2(xt[jt][0], xt[jt][1]) & tril_mask[jt].x;
                    pv_.y = pack_h2(xt[jt][2], xt[jt][3]) & tril_mask[jt].y;
                    *reinterpret_cast<uint2*>(st.Ps + ii * LDA + 16 * jt + 4 * G) = pv_;
                }
            }
            RFA_TICK_AT(4, 0);
            wg_sync();
            RFA_TICK_AT(5, 0);
        };

        // With a single chunk nothing but that (possibly short) chunk may be read.  Otherwise
        // every chunk but the last is full, and chunks past the start are requested again as
        // chunk 0 (never used) rather than under a branch.
        const bool multi = n_chunks > 1;
        prefetch_ragged(s0, n_chunks - 1);
        if (multi) prefetch(s1, n_chunks - 2);
        // i = 0 stages the last chunk from s0
        stage_chunk(0, s0, max(n_chunks - 3, 0), multi);
        for (int i = 1; i < n_chunks; i += 2) {
            stage_chunk(i, s1, max(n_chunks - 3 - i, 0), true);
            if (i + 1 >= n_chunks) break;
            stage_chunk(i + 1, s0, max(n_chunks - 4 - i, 0), true);
        }
        wg_sync();      // the last iteration: the product groups finish chunk 0
        wg_sync();
    } else if (grp == 1) {
        half_t* dqb = dq + (int64_t)n * KD + koff;
        f4 NS[2][NCT], nz[2];
#pragma unroll
        for (int kt = 0; kt < 2; ++kt) {
            const float* sp = final_s + ((int64_t)n * KD + koff + kl0 + 16 * kt + row) * DH + 4 * G;
#pragma unroll
            for (int ct = 0; ct < NCT; ++ct) {
                const f4 x = *reinterpret_cast<const f4*>(sp + 16 * ct);
                NS[kt][ct][0] = -x[0]; NS[kt][ct][1] = -x[1]; NS[kt][ct][2] = -x[2]; NS[kt][ct][3] = -x[3];
            }
            const f4 x = *reinterpret_cast<const f4*>(final_z + (int64_t)n * KD + koff + kl0 + 16 * kt + 4 * G);
            nz[kt][0] = -x[0]; nz[kt][1] = -x[1]; nz[kt][2] = -x[2]; nz[kt][3] = -x[3];
        }
        const h8 ones = h8_ones();
        // RAGGED: the chunk may have fewer than 64 steps (only the last chunk of the sequence, the
        // first one worked on); full chunks store unconditionally
        auto chunk_body = [&](auto ragged_tag, int i) __attribute__((always_inline)) {
            constexpr bool RAGGED = decltype(ragged_tag)::value;
            const int t0 = (n_chunks - i) * C;
            const Stage st = stage_of(i - 1);
            // the state one chunk back: -S_prev = -S + K^T V, -z_prev = -z + K^T 1.  Every operand
            // read from LDS serves both feature tiles of the wave.
            h8 kf[2][2];     // K column fragments: K[j = 32js + 8G + e][k = kl0 + 16kt + i]
#pragma unroll
            for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                for (int js = 0; js < 2; ++js) kf[kt][js] = col8(st.Ks, LDK, js * 32, kl0 + 16 * kt, lane);
#pragma unroll
            for (int js = 0; js < 2; ++js) {
                h8 vc[NCT];
#pragma unroll
                for (int ct = 0; ct < NCT; ++ct) vc[ct] = col8(st.Vs, LDV, js * 32, 16 * ct, lane);
#pragma unroll
                for (int kt = 0; kt < 2; ++kt) {
#pragma unroll
                    for (int ct = 0; ct < NCT; ++ct) NS[kt][ct] = mfma32(vc[ct], kf[kt][js], NS[kt][ct]);
                    nz[kt] = mfma32(kf[kt][js], ones, nz[kt]);
                }
            }
            // dQ^T tiles (m = k, n = i)
            f4 yt[2][4];       // -(S_prev G^T)
#pragma unroll
            for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                for (int it = 0; it < 4; ++it) yt[kt][it] = f4_zero();
#pragma unroll
            for (int cs = 0; cs < DH / 32; ++cs) {
                h8 bg[4];
#pragma unroll
                for (int it = 0; it < 4; ++it) bg[it] = row_split8(st.Gs, LDV, 16 * it + row, cs * 32, G);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int kt = 0; kt < 2; ++kt) {
                    const h8 sh = acc_to_operand_rn(NS[kt][2 * cs], NS[kt][2 * cs + 1]);
#pragma unroll
                    for (int it = 0; it < 4; ++it) yt[kt][it] = mfma32(sh, bg[it], yt[kt][it]);
                }
            }
            RFA_TICK_AT(11, kDqTick);
            wg_sync();
            RFA_TICK_AT(12, kDqTick);
#pragma unroll
            for (int it = 0; it < 4; ++it) {
                const int ii = 16 * it + row;
                const float gzi = st.gzs[ii];
                const h8 p0 = row8(st.Ps, LDA, ii, 0, G);
                h8 p1 = p0;
                if (it >= 2) p1 = row8(st.Ps, LDA, ii, 32, G);
#pragma unroll
                for (int kt = 0; kt < 2; ++kt) {
                    f4 acc;
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[e] = -(yt[kt][it][e] + gzi * nz[kt][e]);
                    acc = mfma32(kf[kt][0], p0, acc);
                    if (it >= 2) acc = mfma32(kf[kt][1], p1, acc);
                    if (!RAGGED || t0 + ii < T)
                        store_lane(dqb + (int64_t)(t0 + 16 * it) * k_stride + kl0 + 16 * kt, out_lane_off, to_h4(acc));
                }
            }
            RFA_TICK_AT(13, kDqTick);
            wg_sync();
            RFA_TICK_AT(14, kDqTick);
        };
        wg_sync();      // the first iteration: the loader group stages the last chunk
        wg_sync();
        chunk_body(std::true_type{}, 1);
        for (int i = 2; i <= n_chunks; ++i) chunk_body(std::false_type{}, i);
    } else {
        half_t* dkb = dk + (int64_t)n * KD + koff;
        f4 RT[2][NCT], racc[2];
#pragma unroll
        for (int kt = 0; kt < 2; ++kt) {
            racc[kt] = f4_zero();
#pragma unroll
            for (int ct = 0; ct < NCT; ++ct) RT[kt][ct] = f4_zero();
        }
        auto chunk_body = [&](auto ragged_tag, int i) __attribute__((always_inline)) {
            constexpr bool RAGGED = decltype(ragged_tag)::value;
            const int t0 = (n_chunks - i) * C;
            const Stage st = stage_of(i - 1);
            // dK^T tiles (m = k, n = j), then R += G^T Q, r += Q^T gz
            h8 qf[2][2];    // Q column fragments: Q[i = 32is + 8G + e][k = kl0 + 16kt + lane i]
#pragma unroll
            for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                for (int is = 0; is < 2; ++is) qf[kt][is] = col8(st.Qs, LDK, is * 32, kl0 + 16 * kt, lane);
            f4 dkacc[2][4];
#pragma unroll
            for (int jt = 0; jt < 4; ++jt) {
                const h8 pc1 = col8(st.Ps, LDA, 32, 16 * jt, lane);
                h8 pc0 = pc1;
                if (jt < 2) pc0 = col8(st.Ps, LDA, 0, 16 * jt, lane);
#pragma unroll
                for (int kt = 0; kt < 2; ++kt) {
                    f4 acc = racc[kt];
                    if (jt < 2) acc = mfma32(qf[kt][0], pc0, acc);
                    acc = mfma32(qf[kt][1], pc1, acc);
                    dkacc[kt][jt] = acc;
                }
            }
#pragma unroll
            for (int cs = 0; cs < DH / 32; ++cs) {
                h8 bvv[4];
#pragma unroll
                for (int jt = 0; jt < 4; ++jt) bvv[jt] = row_split8(st.Vs, LDV, 16 * jt + row, cs * 32, G);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int kt = 0; kt < 2; ++kt) {
                    const h8 rh = acc_to_operand_rn(RT[kt][2 * cs], RT[kt][2 * cs + 1]);
#pragma unroll
                    for (int jt = 0; jt < 4; ++jt) dkacc[kt][jt] = mfma32(rh, bvv[jt], dkacc[kt][jt]);
                }
            }
            wg_sync();
#pragma unroll
            for (int jt = 0; jt < 4; ++jt) {
                const int jj = 16 * jt + row;
#pragma unroll
                for (int kt = 0; kt < 2; ++kt)
                    if (!RAGGED || t0 + jj < T)
                        store_lane(dkb + (int64_t)(t0 + 16 * jt) * k_stride + kl0 + 16 * kt, out_lane_off, to_h4(dkacc[kt][jt]));
            }
#pragma unroll
            for (int is = 0; is < 2; ++is) {
                h8 ghi, glo;
                f8_to_operand(*reinterpret_cast<const f4*>(st.gzs + is * 32 + 8 * G),
                              *reinterpret_cast<const f4*>(st.gzs + is * 32 + 8 * G + 4), ghi, glo);
                h8 gc[NCT];
#pragma unroll
                for (int ct = 0; ct < NCT; ++ct) gc[ct] = col8(st.Gs, LDV, is * 32, 16 * ct, lane);
#pragma unroll
                for (int kt = 0; kt < 2; ++kt) {
                    racc[kt] = mfma32(qf[kt][is], ghi, racc[kt]);
                    racc[kt] = mfma32(qf[kt][is], glo, racc[kt]);
#pragma unroll
                    for (int ct = 0; ct < NCT; ++ct) RT[kt][ct] = mfma32(gc[ct], qf[kt][is], RT[kt][ct]);
                }
            }
            wg_sync();
        };
        wg_sync();
        wg_sync();
        chunk_body(std::true_type{}, 1);
        for (int i = 2; i <= n_chunks; ++i) chunk_body(std::false_type{}, i);
    }
}

// ---------------------------------------------------------------------------
// dV for value columns [coff, coff + 64) of one sequence.
//   loader group: stages Q, K (all KD features) and the G^ slice, then A^T = tril(Q K^T)^T
//   dV groups jh = 0, 1: wave (jh, wc) owns columns cw = coff + 16 wc .. + 15 and produces the dV
//             rows of the 16-step tiles 2jh, 2jh + 1 of every chunk; RR[kt] = R tile
//             (k = 16kt + 4G + e, c = cw + i), all KD feature rows, is kept by both waves of a
//             column tile (the same updates in the same order: identical bits).
// ---------------------------------------------------------------------------
template <int KD, int DH, int SW>
__device__ __forceinline__ void sliced_bwd_dv(
    unsigned char* smem, int n, int coff, const half_t* __restrict__ q, const half_t* __restrict__ k,
    const half_t* __restrict__ g, const float* __restrict__ den_raw, half_t* __restrict__ dv, int T, int N) {
    using Cfg = SlicedBwdCfg<KD, DH, SW>;
    constexpr int NT = kGroupThreads, C = Cfg::C, CSL = Cfg::CSL;
    constexpr int LDQ = Cfg::LDQ, LDG = Cfg::LDG_, LDA = Cfg::LDA;
    constexpr int NKT = KD / 16;
    constexpr int PPR = CSL / 8, VP = ChunkRegs<CSL, NT>::kPieces;
    constexpr size_t kStage = Cfg::kLds / 2;

    const int lane = threadIdx.x & 63;
    if ((threadIdx.x >> 6) >= 8) return;        // the role has 8 waves; the launch may carry more for the other role
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int grp = w >> 2, wc = w & 3;         // loader: column block of the A^T tiles
    const int tid = (w & 3) * 64 + lane;
    const int row = lane & 15, G = lane >> 4;
    const int jh = (w >> 1) & 1;                // product waves 4..7: half of the chunk's rows ...
    const int cl0 = 32 * (w & 1);               // ... and first of this wave's 32 columns, local to the slice array
    const unsigned out_lane_off = (unsigned)row * (unsigned)(N * DH * 2) + 8u * G;
    const int64_t k_stride = (int64_t)N * KD, v_stride = (int64_t)N * DH;
    const int n_chunks = (T + C - 1) / C;
    RFA_TICK_INIT();

    struct Stage { half_t *Qs, *Ks, *Gs, *ATs; };
    auto stage_of = [&](int i) __attribute__((always_inline)) {
        Stage st;
        st.Qs = reinterpret_cast<half_t*>(smem + (i & 1) * kStage);
        st.Ks = st.Qs + C * LDQ;
        st.Gs = st.Ks + C * LDQ;                 // G / den, this slice's columns
        st.ATs = st.Gs + C * LDG;                // AT[j][i] = A[i][j]
        return st;
    };

    if (grp == 0) {
        const half_t* qb = q + (int64_t)n * KD;
        const half_t* kb = k + (int64_t)n * KD;
        const half_t* gb = g + (int64_t)n * DH + coff;
        RowPtrs<KD, NT> pq, pk;
        RowPtrs<CSL, NT> pg;
        pq.init(qb, k_stride, tid);
        pk.init(kb, k_stride, tid);
        pg.init(gb, v_stride, tid);
        struct RowSet {
            ChunkRegs<KD, NT> rq, rk;
            ChunkRegs<CSL, NT> rg;
            float den[VP];
        };
        RowSet s0, s1;
        // which halves of this lane's A^T elements are kept: element (j = 16wc + row, i = 16it + 4G + e) when i >= j
        uint2 tril_mask[4];
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            auto keep = [&](int e) { return (16 * it + 4 * G + e >= 16 * wc + row) ? 0xffffu : 0u; };
            tril_mask[it].x = keep(0) | (keep(1) << 16);
            tril_mask[it].y = keep(2) | (keep(3) << 16);
        }
        auto prefetch_ragged = [&](RowSet& r, int c) __attribute__((always_inline)) {
            const int t0 = c * C, rows = T - t0;
            chunk_g2r<KD, NT>(r.rk, kb + (int64_t)t0 * k_stride, k_stride, rows, tid);
            chunk_g2r<KD, NT>(r.rq, qb + (int64_t)t0 * k_stride, k_stride, rows, tid);
            chunk_g2r<CSL, NT>(r.rg, gb + (int64_t)t0 * v_stride, v_stride, rows, tid);
#pragma unroll
            for (int it = 0; it < VP; ++it) {
                const int r_ = min((tid + NT * it) / PPR, r.rg.rows - 1);
                r.den[it] = den_raw[(int64_t)(t0 + r_) * N + n];
            }
        };
        auto prefetch = [&](RowSet& r, int c) __attribute__((always_inline)) {
            const int64_t t0 = (int64_t)c * C;
            pk.load_full(r.rk, t0 * k_stride);
            pq.load_full(r.rq, t0 * k_stride);
            pg.load_full(r.rg, t0 * v_stride);
#pragma unroll
            for (int it = 0; it < VP; ++it) r.den[it] = den_raw[(t0 + (tid + NT * it) / PPR) * N + n];
        };
        auto stage_chunk = [&](int i, RowSet& r, int c_next, bool do_prefetch) __attribute__((always_inline)) {
            const Stage st = stage_of(i);
            chunk_r2s<KD, NT>(r.rk, st.Ks, LDQ, tid);
            chunk_r2s<KD, NT>(r.rq, st.Qs, LDQ, tid);
            float inv_den[VP];
#pragma unroll
            for (int it = 0; it < VP; ++it) inv_den[it] = rcp_nr(fmaxf(r.den[it], 1.0f));
            chunk_r2s_scaled<CSL, NT>(r.rg, inv_den, st.Gs, LDG, tid);
            RFA_TICK_AT(1, 0);
            wg_sync();
            RFA_TICK_AT(2, 0);
            if (do_prefetch) prefetch(r, c_next);
            RFA_TICK_AT(3, 0);
            // A = tril(Q K^T) tiles (m = i, n = j), stored transposed: column block wc, all four row
            // tiles, no branch around the products
            {
                const int j = 16 * wc + row;
                f4 a_[4];
#pragma unroll
                for (int it = 0; it < 4; ++it) a_[it] = f4_zero();
#pragma unroll
                for (int ks = 0; ks < KD / 32; ++ks) {
                    const h8 bk = row8(st.Ks, LDQ, j, ks * 32, G);
#pragma unroll
                    for (int it = 0; it < 4; ++it) a_[it] = mfma32(row8(st.Qs, LDQ, 16 * it + row, ks * 32, G), bk, a_[it]);
                }
#pragma unroll
                for (int it = 0; it < 4; ++it) {
                    uint2 av;
                    av.x = pack_h2(a_[it][0], a_[it][1]) & tril_mask[it].x;
                    av.y = pack_h2(a_[it][2], a_[it][3]) & tril_mask[it].y;
                    *reinterpret_cast<uint2*>(st.ATs + j * LDA + 16 * it + 4 * G) = av;
                }
            }
            RFA_TICK_AT(4, 0);
            wg_sync();
            RFA_TICK_AT(5, 0);
        };

        const bool multi = n_chunks > 1;
        prefetch_ragged(s0, n_chunks - 1);
        if (multi) prefetch(s1, n_chunks - 2);
        stage_chunk(0, s0, max(n_chunks - 3, 0), multi);
        for (int i = 1; i < n_chunks; i += 2) {
            stage_chunk(i, s1, max(n_chunks - 3 - i, 0), true);
            if (i + 1 >= n_chunks) break;
            stage_chunk(i + 1, s0, max(n_chunks - 4 - i, 0), true);
        }
        wg_sync();
        wg_sync();
    } else {
        half_t* dvb = dv + (int64_t)n * DH + coff;
        f4 RR[2][NKT];
#pragma unroll
        for (int cc = 0; cc < 2; ++cc)
#pragma unroll
            for (int kt = 0; kt < NKT; ++kt) RR[cc][kt] = f4_zero();
        auto chunk_body = [&](auto ragged_tag, int i) __attribute__((always_inline)) {
            constexpr bool RAGGED = decltype(ragged_tag)::value;
            const int t0 = (n_chunks - i) * C;
            const Stage st = stage_of(i - 1);
            // dV^T tiles (m = c, n = j) for j tiles 2jh, 2jh + 1, then R += Q^T G^; every operand
            // read from LDS serves both column tiles of the wave
            h8 gf[2][2];     // G^ column fragments: G^[i = 32is + 8G + e][c = cl0 + 16cc + lane i]
#pragma unroll
            for (int cc = 0; cc < 2; ++cc)
#pragma unroll
                for (int is = 0; is < 2; ++is) gf[cc][is] = col8(st.Gs, LDG, is * 32, cl0 + 16 * cc, lane);
            f4 dvacc[2][2];
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const int jr = 16 * (2 * jh + u) + row;
                // rows i < 32 of A^T only reach the first two j tiles: their operand is all zero
                // for the other half, and multiplying by zeros keeps both halves on one code path
                const h8 a0 = row8(st.ATs, LDA, jr, 0, G), a1 = row8(st.ATs, LDA, jr, 32, G);
#pragma unroll
                for (int cc = 0; cc < 2; ++cc) {
                    f4 acc = mfma32(gf[cc][0], a0, f4_zero());
                    acc = mfma32(gf[cc][1], a1, acc);
                    dvacc[cc][u] = acc;
                }
            }
#pragma unroll
            for (int ks = 0; ks < KD / 32; ++ks) {
                h8 bkk[2];
#pragma unroll
                for (int u = 0; u < 2; ++u) bkk[u] = row_split8(st.Ks, LDQ, 16 * (2 * jh + u) + row, ks * 32, G);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int cc = 0; cc < 2; ++cc) {
                    const h8 rh = acc_to_operand_rn(RR[cc][2 * ks], RR[cc][2 * ks + 1]);
#pragma unroll
                    for (int u = 0; u < 2; ++u) dvacc[cc][u] = mfma32(rh, bkk[u], dvacc[cc][u]);
                }
            }
            RFA_TICK_AT(11, 256);
            wg_sync();
            RFA_TICK_AT(12, 256);
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const int jj = 16 * (2 * jh + u) + row;
#pragma unroll
                for (int cc = 0; cc < 2; ++cc)
                    if (!RAGGED || t0 + jj < T)
                        store_lane(dvb + (int64_t)(t0 + 16 * (2 * jh + u)) * v_stride + cl0 + 16 * cc, out_lane_off, to_h4(dvacc[cc][u]));
            }
#pragma unroll
            for (int is = 0; is < 2; ++is)
#pragma unroll
                for (int kt = 0; kt < NKT; ++kt) {
                    const h8 qc = col8(st.Qs, LDQ, is * 32, 16 * kt, lane);
#pragma unroll
                    for (int cc = 0; cc < 2; ++cc) RR[cc][kt] = mfma32(qc, gf[cc][is], RR[cc][kt]);
                }
            RFA_TICK_AT(13, 256);
            wg_sync();
            RFA_TICK_AT(14, 256);
        };
        wg_sync();
        wg_sync();
        chunk_body(std::true_type{}, 1);
        for (int i = 2; i <= n_chunks; ++i) chunk_body(std::false_type{}, i);
    }
}

// grid = kXcds * ceil(N / kXcds) * (NA + NB); Cfg::kThreads threads.  hdr_in / plan: see plan_matches.
template <int KD, int DH, int SW>
__global__ __launch_bounds__(sliced_threads(SW)) void k_sliced_bwd(
    const half_t* __restrict__ q, const half_t* __restrict__ k, const half_t* __restrict__ v,
    const half_t* __restrict__ g, const half_t* __restrict__ o, const float* __restrict__ den_raw,
    const float* __restrict__ final_s, const float* __restrict__ final_z, half_t* __restrict__ dq,
    half_t* __restrict__ dk, half_t* __restrict__ dv, int T, int N, const int* __restrict__ hdr_in, PlanWords plan) {
    using Cfg = SlicedBwdCfg<KD, DH, SW>;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    int n, role;
    seq_role_of_block(blockIdx.x, Cfg::NA + Cfg::NB, n, role);
    if (n >= N) return;
    if (!plan_matches(hdr_in, plan)) {
        if (role < Cfg::NA) {
            poison_rows<SW>(dq + (int64_t)n * KD + role * SW, (int64_t)N * KD, 0, T);
            poison_rows<SW>(dk + (int64_t)n * KD + role * SW, (int64_t)N * KD, 0, T);
        } else {
            poison_rows<kSliceWidth>(dv + (int64_t)n * DH + (role - Cfg::NA) * kSliceWidth, (int64_t)N * DH, 0, T);
        }
        return;
    }
    if (role < Cfg::NA)
        sliced_bwd_dqdk<KD, DH, SW>(smem_raw, n, role * SW, q, k, v, g, o, den_raw, dq, dk, final_s, final_z, T, N);
    else
        sliced_bwd_dv<KD, DH, SW>(smem_raw, n, (role - Cfg::NA) * kSliceWidth, q, k, g, den_raw, dv, T, N);
}

}  // namespace rfa
