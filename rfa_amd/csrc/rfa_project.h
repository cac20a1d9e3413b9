// Linear projection to heads with the feature map in the epilogue (gfx950).
//
// The attention modules project their input with torch.nn.Linear layers, view the result
// as heads and push the q and k projections through the feature map
// (random_feature_attention/causal_attention.py:228-247, cross_attention.py:66-76,:279-283,
// utils.py:100-120).  Here one launch computes up to three projections of the same input
//     y_p[r, h, :] = x[r, :] . W_p[h*DH .. h*DH+DH, :]^T + b_p[h*DH ..]        (fp16, fp32 accumulate)
// and, for the projections that ask for it, phi(y_p) = scale * [sin(W' y^), cos(W' y^)] with
// y^ = y / (||y|| + 1e-3), from the tile while it is still in registers.  y is rounded to
// fp16 first, exactly as the unfused chain sees it, and is written out as well (the backward
// of the feature map needs it).
//
// Layouts:  x  [R, E] fp16 row-major          W_p [H*DH, E] fp16 row-major (nn.Linear.weight)
//           b_p [H*DH] fp16 or NULL           y_p [R, H, DH] fp16
//           w' [H, D, DH] fp16                phi_p [R, H, 2D] fp16 (sin block first)
#pragma once
#include "rfa_common.h"
#include "rfa_featuremap.h"

namespace rfa {

constexpr int kMaxProjections = 3;

struct ProjectArgs {
    const half_t* w[kMaxProjections];
    const half_t* b[kMaxProjections];
    half_t* y[kMaxProjections];
    half_t* phi[kMaxProjections];     // NULL: no feature map for this projection
};

// element p of a kernel-argument array without indexing it dynamically (which would copy the
// struct to private memory)
template <typename T>
__device__ __forceinline__ T pick3(T const (&a)[kMaxProjections], int p) {
    return p == 0 ? a[0] : (p == 1 ? a[1] : a[2]);
}

template <int D, int DH>
struct ProjectCfg {
    static_assert(D % 32 == 0 && DH % 64 == 0, "D multiple of 32, DH multiple of 64");
    static constexpr int BM = 128;                 // rows of x per workgroup
    static constexpr int BK = 64;                  // contraction step
    static constexpr int LDX = BK + lds_pad(BK);
    static constexpr int LDW = DH + lds_pad(DH);   // rows of w'
    static constexpr int LDP = (2 * D > DH ? 2 * D : DH) + 16;   // staging rows of y / phi
    static constexpr int kStageHalves = (BM + DH) * LDX;         // x tile, then W tile
    static constexpr size_t kLoopLds = (size_t)2 * kStageHalves * 2;
    static constexpr size_t kEpiLds = (size_t)(D * LDW + 4 * 16 * LDP) * 2;
    static constexpr size_t kLds = kLoopLds > kEpiLds ? kLoopLds : kEpiLds;
};

// One contraction step of the operands: [rows][BK] sub-tiles of x (clamped to the last row) and
// of W, 16-byte pieces, piece -> (row, 16-byte column); global -> registers -> LDS.
template <int XP, int WP, int BK>
__device__ __forceinline__ void project_load_stage(uint4 (&xr)[XP], uint4 (&wr)[WP], const half_t* __restrict__ x,
                                                   const half_t* __restrict__ wp, int row0, int R, int E, int k0,
                                                   int tid) {
#pragma unroll
    for (int it = 0; it < XP; ++it) {
        const int pc = tid + kThreads * it;
        const int r = min(row0 + pc / (BK / 8), R - 1);
        xr[it] = *reinterpret_cast<const uint4*>(x + (int64_t)r * E + k0 + (pc % (BK / 8)) * 8);
    }
#pragma unroll
    for (int it = 0; it < WP; ++it) {
        const int pc = tid + kThreads * it;
        wr[it] = *reinterpret_cast<const uint4*>(wp + (int64_t)(pc / (BK / 8)) * E + k0 + (pc % (BK / 8)) * 8);
    }
}

template <int XP, int WP, int BK, int BM, int LDX>
__device__ __forceinline__ void project_store_stage(const uint4 (&xr)[XP], const uint4 (&wr)[WP], half_t* Xs, int tid) {
    half_t* Wsm = Xs + BM * LDX;
#pragma unroll
    for (int it = 0; it < XP; ++it) {
        const int pc = tid + kThreads * it;
        *reinterpret_cast<uint4*>(Xs + (pc / (BK / 8)) * LDX + (pc % (BK / 8)) * 8) = xr[it];
    }
#pragma unroll
    for (int it = 0; it < WP; ++it) {
        const int pc = tid + kThreads * it;
        *reinterpret_cast<uint4*>(Wsm + (pc / (BK / 8)) * LDX + (pc % (BK / 8)) * 8) = wr[it];
    }
}

// Workgroup -> (row tile, head, projection).  Workgroups are dealt to the 8 XCDs round-robin
// by their index; the mapping gives each XCD its own row tiles, so that the H * np workgroups
// that share a tile of x find it in that XCD's L2, while the (small) weights are read by all.
// grid = 8 * ceil(nrt / 8) * H * np.
template <int D, int DH>
__global__ __launch_bounds__(kThreads) void k_project_phi(
    const half_t* __restrict__ x, ProjectArgs pa, const half_t* __restrict__ wf, int R, int E, int H, int np,
    float scale) {
    using Cfg = ProjectCfg<D, DH>;
    constexpr int BM = Cfg::BM, BK = Cfg::BK, LDX = Cfg::LDX, LDW = Cfg::LDW, LDP = Cfg::LDP;
    constexpr int NCT = DH / 16;                       // column tiles of the output
    constexpr int XP = BM * BK / 8 / kThreads;         // 16-byte pieces per thread and stage: x
    constexpr int WP = DH * BK / 8 / kThreads;         //                                      W
    extern __shared__ __align__(16) unsigned char smem_raw[];
    half_t* smem = reinterpret_cast<half_t*>(smem_raw);

    const int tid = threadIdx.x, lane = tid & 63;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int i = lane & 15, G = lane >> 4;

    const int per_tile = H * np;
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int rt_idx = xcd + 8 * (slot / per_tile);
    const int hp = slot % per_tile;
    const int h = hp % H, p = hp / H;
    const int row0 = rt_idx * BM;
    if (row0 >= R) return;                             // whole workgroup: padding of the grid

    const half_t* __restrict__ wp = pick3(pa.w, p) + (int64_t)h * DH * E;

    uint4 xr[XP], wr[WP];
    // y^T tiles (m = output column, n = row): wave wv owns rows [32 wv, +32) of the tile
    f4 acc[2][NCT];
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int c = 0; c < NCT; ++c) acc[a][c] = f4_zero();

    const int nk = E / BK;
    project_load_stage<XP, WP, BK>(xr, wr, x, wp, row0, R, E, 0, tid);
    project_store_stage<XP, WP, BK, BM, LDX>(xr, wr, smem, tid);
    __syncthreads();
    for (int kk = 0; kk < nk; ++kk) {
        // branch-free prefetch: the last step re-reads its own operands and stores them to the idle buffer
        project_load_stage<XP, WP, BK>(xr, wr, x, wp, row0, R, E, min((kk + 1) * BK, E - BK), tid);
        const half_t* Xs = smem + (kk & 1) * Cfg::kStageHalves;
        const half_t* Wsm = Xs + BM * LDX;
#pragma unroll
        for (int ks = 0; ks < BK / 32; ++ks) {
            const h8 xb0 = row8(Xs, LDX, 32 * wv + i, 32 * ks, G);
            const h8 xb1 = row8(Xs, LDX, 32 * wv + 16 + i, 32 * ks, G);
#pragma unroll
            for (int ct = 0; ct < NCT; ++ct) {
                const h8 wa = row8(Wsm, LDX, 16 * ct + i, 32 * ks, G);
                acc[0][ct] = mfma32(wa, xb0, acc[0][ct]);
                acc[1][ct] = mfma32(wa, xb1, acc[1][ct]);
            }
        }
        project_store_stage<XP, WP, BK, BM, LDX>(xr, wr, smem + ((kk + 1) & 1) * Cfg::kStageHalves, tid);
        __syncthreads();
    }

    // ---- epilogue: the stage buffers are free now
    half_t* Wfs = smem;                                   // w' of this head
    half_t* Ps = smem + D * LDW + wv * 16 * LDP;          // this wave's 16 staging rows
    half_t* phi = pick3(pa.phi, p);
    if (phi) {
        load_w_to_lds<D, DH>(Wfs, wf + (int64_t)h * D * DH, tid);
        __syncthreads();
    }
    const half_t* bias = pick3(pa.b, p);
    half_t* y = pick3(pa.y, p);
#pragma unroll
    for (int a = 0; a < 2; ++a) {
        const int r0 = row0 + 32 * wv + 16 * a;
        h8 op[DH / 32];      // the rounded tile as the B operand of the feature projection, split slot order
        float ss = 0.f;
#pragma unroll
        for (int ct = 0; ct < NCT; ++ct) {
            f4 t = acc[a][ct];
            if (bias) {
                const h4 bv = *reinterpret_cast<const h4*>(bias + h * DH + 16 * ct + 4 * G);
#pragma unroll
                for (int e = 0; e < 4; ++e) t[e] += (float)bv[e];
            }
            const h4 yh = to_h4(t);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                ss += (float)yh[e] * (float)yh[e];
                op[ct / 2][4 * (ct % 2) + e] = yh[e];
            }
            if (y) *reinterpret_cast<h4*>(Ps + i * LDP + 16 * ct + 4 * G) = yh;
        }
        if (y) {        // NULL: the caller keeps only phi(y) (no backward pass will ask for y)
            wave_lds_order();
            wave_rows_s2g<DH>(Ps, LDP, y, r0, R, H, h, lane);
            wave_lds_order();
        }
        if (phi) {
            ss = sum_over_groups(ss);
            const float inv = 1.0f / (sqrtf(ss) + 1e-3f);
#pragma unroll
            for (int jt = 0; jt < D / 16; ++jt) {
                f4 u = f4_zero();     // u^T tile (m = feature j, n = row); contraction in split slot order
#pragma unroll
                for (int pr = 0; pr < DH / 32; ++pr) {
                    u = mfma32(row_split8(Wfs, LDW, 16 * jt + i, 32 * pr, G), op[pr], u);
                }
                h4 sv, cv;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float s_, c_;
                    fast_sincos(u[e] * inv, s_, c_);
                    sv[e] = (half_t)(scale * s_);
                    cv[e] = (half_t)(scale * c_);
                }
                *reinterpret_cast<h4*>(Ps + i * LDP + 16 * jt + 4 * G) = sv;
                *reinterpret_cast<h4*>(Ps + i * LDP + D + 16 * jt + 4 * G) = cv;
            }
            wave_lds_order();
            wave_rows_s2g<2 * D>(Ps, LDP, phi, r0, R, H, h, lane);
            wave_lds_order();
        }
    }
}

// ---------------------------------------------------------------------------
// Same computation for narrow inputs (E = 32 * NKS <= 512, DH = 64): a workgroup keeps its 128
// rows of x in registers for its whole life -- wave w holds rows [32w, 32w + 32) as MFMA B
// operands, 2 * NKS registers of 8 halves -- and walks a list of (head, projection) pairs whose
// weight rows ([DH][E] each) arrive whole in a two-buffer LDS ring, one pair ahead.  No barrier
// inside a pair's contraction or its epilogue.
//   grid = 8 * ceil(nrt / 8) * ngroups; group g of a row tile takes pairs [g * ppg, (g + 1) * ppg)
//   of the H * np pairs, pair index hp -> head hp / np, projection hp % np.
// LDS: [ring: 2 x DH x (E + 8); first used to stage the x tile][staging rows of the waves][w' of the head]
// ---------------------------------------------------------------------------
// 16 bytes as a native vector: assignments are plain vector loads and stores (the uint4 class
// is copied with memcpy, which keeps registers that stay in flight across loop iterations in
// private memory)
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

template <int D, int DH, int NKS>
struct ProjectRowCfg {
    static_assert(DH == 64, "one 64-wide head per pair");
    static constexpr int BM = 128, E = 32 * NKS;
    static constexpr int LDE = E + 8;
    static constexpr int LDW = DH + lds_pad(DH);
    static constexpr int LDP = (2 * D > DH ? 2 * D : DH) + 16;
    static constexpr int kSliceHalves = DH * LDE;
    static constexpr int SP = DH * E / 8 / kThreads;        // 16-byte pieces per thread and slice
    static constexpr size_t kLds = (size_t)(2 * kSliceHalves + 4 * 16 * LDP + D * LDW) * 2;
    static_assert(2 * kSliceHalves >= BM * LDE, "the x tile is staged in the ring");
    static_assert(kLds <= 160 * 1024, "LDS budget");
};

template <int D, int DH, int NKS>
__global__ __launch_bounds__(kThreads) void k_project_phi_rows(
    const half_t* __restrict__ x, ProjectArgs pa, const half_t* __restrict__ wf, int R, int H, int np,
    int ngroups, int ppg, float scale) {
    using Cfg = ProjectRowCfg<D, DH, NKS>;
    constexpr int BM = Cfg::BM, E = Cfg::E, LDE = Cfg::LDE, LDW = Cfg::LDW, LDP = Cfg::LDP, SP = Cfg::SP;
    constexpr int NCT = DH / 16, PPR = E / 8;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    half_t* ring = reinterpret_cast<half_t*>(smem_raw);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int i = lane & 15, G = lane >> 4;
    half_t* Ps = ring + 2 * Cfg::kSliceHalves + wv * 16 * LDP;
    half_t* Wfs = ring + 2 * Cfg::kSliceHalves + 4 * 16 * LDP;

    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int row0 = (xcd + 8 * (slot / ngroups)) * BM;
    const int grp = slot % ngroups;
    const int pairs = H * np;
    const int hp_begin = grp * ppg, hp_end = min(hp_begin + ppg, pairs);
    if (row0 >= R || hp_begin >= hp_end) return;
    RFA_TICK_INIT();

    // weight rows of pair hp: piece -> (row, 16-byte column)
    u32x4 wr[SP];
    auto slice_g2r = [&](int hp) {
        const half_t* __restrict__ src = pick3(pa.w, hp % np) + (int64_t)(hp / np) * DH * E;
#pragma unroll
        for (int it = 0; it < SP; ++it) wr[it] = *reinterpret_cast<const u32x4*>(src + (int64_t)(tid + kThreads * it) * 8);
    };
    auto slice_r2s = [&](half_t* buf) {
#pragma unroll
        for (int it = 0; it < SP; ++it) {
            const int pc = tid + kThreads * it;
            *reinterpret_cast<u32x4*>(buf + (pc / PPR) * LDE + (pc % PPR) * 8) = wr[it];
        }
    };
    // Workgroups of different row tiles walk their pairs in rotated order, so that the CUs of an
    // XCD do not all ask the L2 for the same weight rows at the same time.
    const int cnt = hp_end - hp_begin;
    const int rot = (row0 / BM) % cnt;
    auto pair_at = [&](int j) { return hp_begin + (j + rot) % cnt; };
    slice_g2r(pair_at(0));

    // x tile -> ring (coalesced rows) -> this wave's rows as B operands
    {
        constexpr int XP = BM * PPR / kThreads, BATCH = XP % 16 == 0 ? 16 : 8;
        static_assert(XP % BATCH == 0, "x tile pieces");
#pragma unroll
        for (int base = 0; base < XP; base += BATCH) {
            u32x4 v[BATCH];
#pragma unroll
            for (int b = 0; b < BATCH; ++b) {
                const int pc = tid + kThreads * (base + b);
                const int r = min(row0 + pc / PPR, R - 1);
                v[b] = *reinterpret_cast<const u32x4*>(x + (int64_t)r * E + (pc % PPR) * 8);
            }
#pragma unroll
            for (int b = 0; b < BATCH; ++b) {
                const int pc = tid + kThreads * (base + b);
                *reinterpret_cast<u32x4*>(ring + (pc / PPR) * LDE + (pc % PPR) * 8) = v[b];
            }
        }
    }
    __syncthreads();
    h8 xb[2][NKS];
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) xb[a][ks] = row8(ring, LDE, 32 * wv + 16 * a + i, 32 * ks, G);
    __syncthreads();
    slice_r2s(ring);
    // wf is NULL when no projection asks for phi
    int h_loaded = pair_at(0) / np;
    if (wf) load_w_to_lds<D, DH>(Wfs, wf + (int64_t)h_loaded * D * DH, tid);
    __syncthreads();
    RFA_TICK(0);

    for (int j = 0; j < cnt; ++j) {
        const int hp = pair_at(j);
        const int h = hp / np, p = hp % np;
        const half_t* Ws = ring + (j & 1) * Cfg::kSliceHalves;
        // the bias before the weight prefetch: loads return in order, and the epilogue must not
        // have to wait for the next pair's weights to see its bias
        const half_t* bias = pick3(pa.b, p);
        h4 bv[NCT];
#pragma unroll
        for (int ct = 0; ct < NCT; ++ct) {
#pragma unroll
            for (int e = 0; e < 4; ++e) bv[ct][e] = (half_t)0.f;
            if (bias) bv[ct] = *reinterpret_cast<const h4*>(bias + h * DH + 16 * ct + 4 * G);
        }
        const int hp_next = pair_at(min(j + 1, cnt - 1));     // the last pair re-reads its own rows
        slice_g2r(hp_next);

        f4 acc[2][NCT];
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int c = 0; c < NCT; ++c) acc[a][c] = f4_zero();
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks)
#pragma unroll
            for (int ct = 0; ct < NCT; ++ct) {
                const h8 wa = row8(Ws, LDE, 16 * ct + i, 32 * ks, G);
                acc[0][ct] = mfma32(wa, xb[0][ks], acc[0][ct]);
                acc[1][ct] = mfma32(wa, xb[1][ks], acc[1][ct]);
            }
        RFA_TICK(1);

        half_t* phi = pick3(pa.phi, p);
        half_t* y = pick3(pa.y, p);
#pragma unroll
        for (int a = 0; a < 2; ++a) {
            const int r0 = row0 + 32 * wv + 16 * a;
            h8 op[DH / 32];
            float ss = 0.f;
#pragma unroll
            for (int ct = 0; ct < NCT; ++ct) {
                f4 t = acc[a][ct];
#pragma unroll
                for (int e = 0; e < 4; ++e) t[e] += (float)bv[ct][e];
                const h4 yh = to_h4(t);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    ss += (float)yh[e] * (float)yh[e];
                    op[ct / 2][4 * (ct % 2) + e] = yh[e];
                }
                if (y) *reinterpret_cast<h4*>(Ps + i * LDP + 16 * ct + 4 * G) = yh;
            }
            if (y) {
                wave_lds_order();
                wave_rows_s2g<DH>(Ps, LDP, y, r0, R, H, h, lane);
                wave_lds_order();
            }
            if (phi) {
                ss = sum_over_groups(ss);
                const float inv = 1.0f / (sqrtf(ss) + 1e-3f);
#pragma unroll
                for (int jt = 0; jt < D / 16; ++jt) {
                    f4 u = f4_zero();
#pragma unroll
                    for (int pr = 0; pr < DH / 32; ++pr)
                        u = mfma32(row_split8(Wfs, LDW, 16 * jt + i, 32 * pr, G), op[pr], u);
                    h4 sv, cv;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        float s_, c_;
                        fast_sincos(u[e] * inv, s_, c_);
                        sv[e] = (half_t)(scale * s_);
                        cv[e] = (half_t)(scale * c_);
                    }
                    *reinterpret_cast<h4*>(Ps + i * LDP + 16 * jt + 4 * G) = sv;
                    *reinterpret_cast<h4*>(Ps + i * LDP + D + 16 * jt + 4 * G) = cv;
                }
                wave_lds_order();
                wave_rows_s2g<2 * D>(Ps, LDP, phi, r0, R, H, h, lane);
                wave_lds_order();
            }
        }
        RFA_TICK(2);
        __syncthreads();                              // everyone is done with this pair's buffer and w'
        const int h_next = hp_next / np;
        if (h_next != h_loaded) {
            h_loaded = h_next;
            if (wf) load_w_to_lds<D, DH>(Wfs, wf + (int64_t)h_next * D * DH, tid);
        }
        slice_r2s(ring + ((j + 1) & 1) * Cfg::kSliceHalves);
        __syncthreads();
        RFA_TICK(3);
    }
}

// ---------------------------------------------------------------------------
// Weight and bias gradients of those Linear layers:
//     dW_p[o][c] = sum_r dy_p[r][o] * x[r][c],      db_p[o] = sum_r dy_p[r][o]
// (what autograd computes for torch.nn.Linear).  The contraction runs over the R rows, far
// longer than either output side, so it is split: workgroup (split s, projection p, tile)
// sums a 128 x 128 tile of dW_p over the rows of split s into an fp32 partial, and
// k_weight_grad_reduce adds the partials.  Both operands are contracted over their row index,
// i.e. read from their row-major LDS tiles with the transposing read.
// Layouts: x [R, Ei], dy_p [R, Eo] fp16 row-major; part [nsplit][np][Eo][Ei], bpart
// [nsplit][np][Eo] fp32; dW_p [Eo, Ei], db_p [Eo] fp16.
// ---------------------------------------------------------------------------
struct WeightGradArgs {
    const half_t* dy[kMaxProjections];
    half_t* dw[kMaxProjections];
    half_t* db[kMaxProjections];      // NULL: no bias gradient for this projection
};

struct WeightGradCfg {
    static constexpr int TO = 128, TI = 128, C = 64;       // tile of dW, rows per step
    static constexpr int LD = 128 + lds_pad(128);
    static constexpr int kTile = C * LD;                   // halves
    static constexpr size_t kLds = (size_t)2 * 2 * kTile * 2;
    static constexpr int kPieces = C * 128 / 8 / kThreads; // 16-byte pieces per thread and tile
};

// rows [r0, r0 + 64) x columns [c0, c0 + 128) of a [R, E] matrix -> registers; rows at or past
// r_end are read from row r_end - 1 (always a valid row) and zeroed on the way to LDS
__device__ __forceinline__ void wgrad_g2r(uint4 (&v)[WeightGradCfg::kPieces], const half_t* __restrict__ src, int E,
                                          int r0, int r_end, int c0, int tid) {
#pragma unroll
    for (int it = 0; it < WeightGradCfg::kPieces; ++it) {
        const int pc = tid + kThreads * it;
        const int r = min(r0 + pc / 16, r_end - 1);
        v[it] = *reinterpret_cast<const uint4*>(src + (int64_t)r * E + c0 + (pc % 16) * 8);
    }
}

__device__ __forceinline__ void wgrad_r2s(const uint4 (&v)[WeightGradCfg::kPieces], half_t* Xs, int r0, int r_end,
                                          int tid) {
#pragma unroll
    for (int it = 0; it < WeightGradCfg::kPieces; ++it) {
        const int pc = tid + kThreads * it;
        const bool keep = r0 + pc / 16 < r_end;
        uint4 x = v[it];
        x.x = keep ? x.x : 0u; x.y = keep ? x.y : 0u; x.z = keep ? x.z : 0u; x.w = keep ? x.w : 0u;
        *reinterpret_cast<uint4*>(Xs + (pc / 16) * WeightGradCfg::LD + (pc % 16) * 8) = x;
    }
}

// grid = 8 * ceil(nsplit / 8) * np * (Eo / 128) * (Ei / 128): the workgroups of one split (which
// share its rows of x and dy) are dealt to one XCD.  rows_per_split is a multiple of 64.
__global__ __launch_bounds__(kThreads) void k_weight_grad_partial(
    const half_t* __restrict__ x, WeightGradArgs wa, float* __restrict__ part, float* __restrict__ bpart, int R,
    int Eo, int Ei, int np, int nsplit, int rows_per_split) {
    using Cfg = WeightGradCfg;
    constexpr int LD = Cfg::LD, C = Cfg::C;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    half_t* smem = reinterpret_cast<half_t*>(smem_raw);

    const int tid = threadIdx.x, lane = tid & 63;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int i = lane & 15, G = lane >> 4;
    const int wo = wv >> 1, wi = wv & 1;                  // wave -> 64 x 64 quadrant of the tile

    const int tiles_i = Ei / Cfg::TI, tiles_o = Eo / Cfg::TO;
    const int per_split = np * tiles_o * tiles_i;
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int s = xcd + 8 * (slot / per_split);
    if (s >= nsplit) return;
    int idx = slot % per_split;
    const int ti = idx % tiles_i; idx /= tiles_i;
    const int to = idx % tiles_o;
    const int p = idx / tiles_o;
    const int r_begin = s * rows_per_split, r_end = min(r_begin + rows_per_split, R);
    const int o0 = to * Cfg::TO, c0 = ti * Cfg::TI;
    const half_t* __restrict__ dy = pick3(wa.dy, p);
    const bool with_bias = ti == 0 && wi == 0 && pick3(wa.db, p) != nullptr;   // wave-uniform

    f4 acc[4][4];        // (m = o, n = c) tiles of this wave's quadrant
    f4 accb[4];          // column sums of dy: every column n holds the same sum
#pragma unroll
    for (int a = 0; a < 4; ++a) {
        accb[a] = f4_zero();
#pragma unroll
        for (int b = 0; b < 4; ++b) acc[a][b] = f4_zero();
    }
    h8 ones;
#pragma unroll
    for (int e = 0; e < 8; ++e) ones[e] = (half_t)1.0f;

    if (r_begin < r_end) {
        uint4 yr[Cfg::kPieces], xr[Cfg::kPieces];
        wgrad_g2r(yr, dy, Eo, r_begin, r_end, o0, tid);
        wgrad_g2r(xr, x, Ei, r_begin, r_end, c0, tid);
        wgrad_r2s(yr, smem, r_begin, r_end, tid);
        wgrad_r2s(xr, smem + Cfg::kTile, r_begin, r_end, tid);
        __syncthreads();
        int buf = 0;
        for (int r0 = r_begin; r0 < r_end; r0 += C) {
            // branch-free prefetch of the next step (the last one re-reads valid rows and zeroes them)
            wgrad_g2r(yr, dy, Eo, r0 + C, r_end, o0, tid);
            wgrad_g2r(xr, x, Ei, r0 + C, r_end, c0, tid);
            const half_t* Ys = smem + buf * 2 * Cfg::kTile;
            const half_t* Xs = Ys + Cfg::kTile;
#pragma unroll
            for (int rs = 0; rs < C / 32; ++rs) {
                h8 xa[4];
#pragma unroll
                for (int b = 0; b < 4; ++b) xa[b] = col8(Xs, LD, 32 * rs, 64 * wi + 16 * b, lane);
#pragma unroll
                for (int a = 0; a < 4; ++a) {
                    const h8 ya = col8(Ys, LD, 32 * rs, 64 * wo + 16 * a, lane);
#pragma unroll
                    for (int b = 0; b < 4; ++b) acc[a][b] = mfma32(ya, xa[b], acc[a][b]);
                    if (with_bias) accb[a] = mfma32(ya, ones, accb[a]);
                }
            }
            buf ^= 1;
            wgrad_r2s(yr, smem + buf * 2 * Cfg::kTile, r0 + C, r_end, tid);
            wgrad_r2s(xr, smem + buf * 2 * Cfg::kTile + Cfg::kTile, r0 + C, r_end, tid);
            __syncthreads();
        }
    }
    float* po = part + ((int64_t)(s * np + p) * Eo + o0 + 64 * wo) * Ei + c0 + 64 * wi;
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 4; ++b)
#pragma unroll
            for (int e = 0; e < 4; ++e) po[(int64_t)(16 * a + 4 * G + e) * Ei + 16 * b + i] = acc[a][b][e];
    if (with_bias && i == 0) {
        float* pb = bpart + (int64_t)(s * np + p) * Eo + o0 + 64 * wo;
#pragma unroll
        for (int a = 0; a < 4; ++a) *reinterpret_cast<f4*>(pb + 16 * a + 4 * G) = accb[a];
    }
}

// dW_p = sum of the partials (4 elements per thread), then db_p; grid = ceil(np * (Eo * Ei + Eo) / 4 / 256)
__global__ __launch_bounds__(kThreads) void k_weight_grad_reduce(
    const float* __restrict__ part, const float* __restrict__ bpart, WeightGradArgs wa, int Eo, int Ei, int np,
    int nsplit) {
    const int64_t per_w = (int64_t)Eo * Ei / 4, per_b = Eo / 4;
    const int64_t t = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (t < per_w * np) {
        const int p = (int)(t / per_w);
        const int64_t q = t % per_w;
        f4 sum = f4_zero();
        for (int s = 0; s < nsplit; ++s) {
            const f4 v = *reinterpret_cast<const f4*>(part + ((int64_t)(s * np + p) * per_w + q) * 4);
            sum[0] += v[0]; sum[1] += v[1]; sum[2] += v[2]; sum[3] += v[3];
        }
        *reinterpret_cast<h4*>(pick3(wa.dw, p) + q * 4) = to_h4(sum);
    } else if (t < (per_w + per_b) * np) {
        const int64_t u = t - per_w * np;
        const int p = (int)(u / per_b);
        const int64_t q = u % per_b;
        half_t* db = pick3(wa.db, p);
        if (!db) return;
        f4 sum = f4_zero();
        for (int s = 0; s < nsplit; ++s) {
            const f4 v = *reinterpret_cast<const f4*>(bpart + ((int64_t)(s * np + p) * per_b + q) * 4);
            sum[0] += v[0]; sum[1] += v[1]; sum[2] += v[2]; sum[3] += v[3];
        }
        *reinterpret_cast<h4*>(db + q * 4) = to_h4(sum);
    }
}

}  // namespace rfa
