// Device-side building blocks shared by the RFA kernels (gfx950 / CDNA4 only).
//
// Conventions used everywhere in this directory
//   * a workgroup is 256 threads = 4 wavefronts of 64 lanes;
//   * lane = 16*G + i  (G = lane/16 in 0..3, i = lane%16);
//   * MFMA v_mfma_f32_16x16x32_f16 computes  D[m][n] += sum_r A[m][r] * B[n][r]
//     with, per lane,  A operand = 8 halves A[m=i][r=8G..8G+7],
//                      B operand = 8 halves B[n=i][r=8G..8G+7],
//                      D         = 4 floats D[m=4G+e][n=i], e=0..3.
//     (layout checked on hardware by tests/test_gpu_mfma_layout.py)
//   * consequence used throughout: an accumulator tile D is itself a valid A or
//     B operand for a later MFMA that contracts over D's *row* index m, with the
//     "split" slot order  slots 0..3 <-> m = 4G+e of tile t,
//                         slots 4..7 <-> m = 4G+e of tile t+1;
//     the other operand is then read with the same slot order (row_split8).
#pragma once
#include <type_traits>
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace rfa {

typedef _Float16 half_t;
typedef half_t h2 __attribute__((ext_vector_type(2)));
typedef half_t h4 __attribute__((ext_vector_type(4)));
typedef half_t h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));

// Phase timing for kernel tuning: compile with -DRFA_PHASE_TIMING to make thread 0 of
// one workgroup add the core-clock cycles spent between consecutive RFA_TICK marks to
// g_phase_ticks (read back with rfa_debug_phase_ticks).  Compiled out otherwise.
#ifdef RFA_PHASE_TIMING
__device__ unsigned long long g_phase_ticks[32];
#define RFA_TICK_INIT() long long tick_last_ = clock64()
#define RFA_TICK(i) RFA_TICK_AT(i, 0)
#define RFA_TICK_AT(i, thr)                                                                \
    do {                                                                                   \
        if (blockIdx.x == RFA_PHASE_TIMING && threadIdx.x == (thr)) {                      \
            const long long now_ = clock64();                                              \
            atomicAdd(&g_phase_ticks[i], (unsigned long long)(now_ - tick_last_));         \
            tick_last_ = now_;                                                             \
        }                                                                                  \
    } while (0)
#else
#define RFA_TICK_INIT() do { } while (0)
#define RFA_TICK(i) do { } while (0)
#define RFA_TICK_AT(i, thr) do { } while (0)
#endif

// Row padding (in halves) of an LDS array with F halves per row.  With 64 banks of 4
// bytes the row stride in dwords must be 4*odd mod 64 for conflict-free 16-byte row
// reads and leave 8-dword gaps between 4 consecutive rows for the transposing reads:
// stride = 12 (mod 64) dwords for F = 128, 256 and 36 for F = 64.
constexpr int lds_pad(int F) { return (F % 128 == 0) ? 24 : 8; }

constexpr int kThreads = 256;   // threads per workgroup
constexpr int kChunk = 64;      // time steps per chunk
constexpr int kXcds = 8;        // accelerator dies of an MI355X; workgroups are dealt to them round-robin by index

// Description of the forward pass that filled a saved-state buffer: the first 16 ints of the
// buffer.  The forward kernel writes it, the backward kernels compare it with the plan they were
// launched for and, if the two differ, fill their outputs with NaN instead of reading segment
// totals laid out for another plan.
struct PlanWords {
    int w[16];   // magic, version, layout, K, d, nseg, seg_len, prefixed, T lo, T hi, N lo, N hi, 0...
};
constexpr int kPlanMagic = 0x52464153;   // "RFAS"

__device__ __forceinline__ void plan_write(int* __restrict__ hdr, const PlanWords& p) {
    if (hdr && blockIdx.x == 0 && threadIdx.x < 16) hdr[threadIdx.x] = p.w[threadIdx.x];
}

// same answer in every wave of the workgroup
__device__ __forceinline__ bool plan_matches(const int* __restrict__ hdr, const PlanWords& p) {
    if (!hdr) return true;
    const int lane = threadIdx.x & 63;
    const bool bad = lane < 16 && hdr[lane] != p.w[lane];
    return !__any(bad);
}

// rows [t_begin, t_end) of one sequence of a time-major fp16 tensor <- NaN
template <int F>
__device__ __forceinline__ void poison_rows(_Float16* __restrict__ base, int64_t row_stride, int t_begin, int t_end) {
    const unsigned short nan16 = 0x7E00;
    unsigned short* b = reinterpret_cast<unsigned short*>(base);
    for (int64_t e = threadIdx.x; e < (int64_t)(t_end - t_begin) * F; e += blockDim.x)
        b[(int64_t)(t_begin + e / F) * row_stride + e % F] = nan16;
}

__device__ __forceinline__ f4 mfma32(h8 a, h8 b, f4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ f4 f4_zero() { f4 z = {0.f, 0.f, 0.f, 0.f}; return z; }

// 8 consecutive halves of one LDS row: X[row][c0 + 8G .. +7]   ("natural" slot order)
__device__ __forceinline__ h8 row8(const half_t* X, int ld, int row, int c0, int G) {
    return *reinterpret_cast<const h8*>(X + row * ld + c0 + 8 * G);
}

// "split" slot order: X[row][c0 + 4G + e] (e=0..3) then X[row][c0 + 16 + 4G + e]
__device__ __forceinline__ h8 row_split8(const half_t* X, int ld, int row, int c0, int G) {
    const half_t* p = X + row * ld + c0 + 4 * G;
    h4 a = *reinterpret_cast<const h4*>(p);
    h4 b = *reinterpret_cast<const h4*>(p + 16);
    return __builtin_shufflevector(a, b, 0, 1, 2, 3, 4, 5, 6, 7);
}

// LDS transposing read (ds_read_b64_tr_b16).  Within each group of 16 lanes the
// hardware returns  out[lane i][e] = in[lane 4e + i/4][i%4]; with the address
// pattern below lane (G,i) receives the column fragment
//     X[r0 + 4G' + e][c0 + i],  e = 0..3,   where r0 already includes 4G' .
__device__ __forceinline__ h4 tr_read4(const half_t* p) {
    typedef __attribute__((__vector_size__(4 * sizeof(__fp16)))) __fp16 fp16x4;
    typedef __attribute__((address_space(3))) fp16x4 lds_fp16x4;
    union { fp16x4 v; h4 h; } u;
    u.v = __builtin_amdgcn_ds_read_tr16_b64_v4f16((lds_fp16x4*)(p));
    return u.h;
}

// Column fragment in natural slot order: X[r0 + 8G + e][c0 + i], e = 0..7, from a
// row-major LDS array (ld in halves, multiple of 4).  This is how an operand whose
// contraction index is the *row* index of X is fed to the MFMA without keeping a
// transposed copy of X.
__device__ __forceinline__ h8 col8(const half_t* X, int ld, int r0, int c0, int lane) {
    const int s = lane & 15, G = lane >> 4;
    const half_t* p = X + (r0 + 8 * G + (s >> 2)) * ld + c0 + 4 * (s & 3);
    h4 a = tr_read4(p);
    h4 b = tr_read4(p + 4 * ld);
    return __builtin_shufflevector(a, b, 0, 1, 2, 3, 4, 5, 6, 7);
}

// "Pair order" of the rows of an MFMA operand matrix: row pair_pos(f) holds index f, so that tile t
// of 16 rows is made of the indices 32 (t / 2) + 8 G + 4 (t % 2) + e at accumulator position
// m = 4 G + e, and the accumulators of tiles 2p and 2p + 1 together give lane (i, G) the 8
// consecutive indices 32 p + 8 G .. + 7: 16 bytes per lane and row, ready for one store.
__host__ __device__ constexpr int pair_pos(int f) { return (f & ~31) | ((f & 4) << 2) | ((f & 24) >> 1) | (f & 3); }

// Two fp32 values -> packed fp16 hi and lo with hi + lo carrying ~22 bits of each.  The
// residual x - float(hi) is exact in fp32 and is formed as fma(hi, -1, x): with the -1 and the
// packed hi opaque to the optimiser the compiler selects the mixed-precision fma that reads the
// fp16 half in place (v_fma_mix*), two VALU instructions per value instead of four.
__device__ __forceinline__ void split_pair(float a, float b, h2& hi, h2& lo) {
    float m1 = -1.0f;
    asm("" : "+s"(m1));
    h2 t;
    t[0] = (half_t)a;
    t[1] = (half_t)b;
    unsigned int p = __builtin_bit_cast(unsigned int, t);
    asm("" : "+v"(p));
    hi = __builtin_bit_cast(h2, p);
    lo[0] = (half_t)__builtin_fmaf((float)hi[0], m1, a);
    lo[1] = (half_t)__builtin_fmaf((float)hi[1], m1, b);
}

// eight fp32 values (two f4) -> fp16 operand pair hi + lo, natural slot order
__device__ __forceinline__ void f8_to_operand(const f4& a, const f4& b, h8& hi, h8& lo) {
    h2 h[4], l[4];
    split_pair(a[0], a[1], h[0], l[0]);
    split_pair(a[2], a[3], h[1], l[1]);
    split_pair(b[0], b[1], h[2], l[2]);
    split_pair(b[2], b[3], h[3], l[3]);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        hi[2 * i] = h[i][0]; hi[2 * i + 1] = h[i][1];
        lo[2 * i] = l[i][0]; lo[2 * i + 1] = l[i][1];
    }
}

// Two accumulator tiles as one fp16 operand in the same (split) slot order, rounded to nearest.
// For products that only *use* a carried fp32 state: the state itself stays fp32 in its
// accumulator, so the rounding is that of any other fp16 operand and does not build up over steps.
__device__ __forceinline__ h8 acc_to_operand_rn(const f4& t0, const f4& t1) {
    h8 r;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        r[e] = (half_t)t0[e];
        r[4 + e] = (half_t)t1[e];
    }
    return r;
}

// two floats rounded to nearest into one register of two halves (a in the low half)
__device__ __forceinline__ unsigned pack_h2(float a, float b) {
    typedef _Float16 hh2 __attribute__((ext_vector_type(2)));
    hh2 r;
    r[0] = (half_t)a; r[1] = (half_t)b;
    return __builtin_bit_cast(unsigned, r);
}

__device__ __forceinline__ h4 to_h4(const f4& x) {
    h4 r;
    r[0] = (half_t)x[0]; r[1] = (half_t)x[1]; r[2] = (half_t)x[2]; r[3] = (half_t)x[3];
    return r;
}

__device__ __forceinline__ h4 h4_zero() {
    h4 r; r[0] = (half_t)0.f; r[1] = (half_t)0.f; r[2] = (half_t)0.f; r[3] = (half_t)0.f; return r;
}

__device__ __forceinline__ h8 h8_ones() {
    h8 r;
#pragma unroll
    for (int e = 0; e < 8; ++e) r[e] = (half_t)1.0f;
    return r;
}


// sin and cos of x (radians) on the hardware transcendental unit: v_sin_f32 / v_cos_f32
// take their argument in turns.  The argument of the feature map is u = w . x^ with
// |u| rarely above 10; the error of x * (1/2pi) in fp32 (2^-24 relative) and of the unit
// itself stay below 1e-6 absolute there, far inside the fp16 resolution of the outputs
// (3e-4 relative at |phi| ~ 0.1).  About ten times fewer instructions than sincosf.
//
// sin and cos of 2 pi t.  The hardware functions take their argument in turns and are valid on
// [-256, 256]: the fractional part (one instruction) keeps any t inside.
__device__ __forceinline__ void sincos_turns(float t, float& s, float& c) {
    t = __builtin_amdgcn_fractf(t);
    s = __builtin_amdgcn_sinf(t);
    c = __builtin_amdgcn_cosf(t);
}

__device__ __forceinline__ void fast_sincos(float x, float& s, float& c) { sincos_turns(x * 0.15915494309189535f, s, c); }

// sum over the four 16-lane groups (lanes i, i+16, i+32, i+48)
// Sum of the per-segment slots [s_first, s_last) of a carried state.  A loop that loads and adds one
// slot per iteration pays one full memory latency per slot (the slots were written by other
// workgroups of the previous kernel: they come from memory, about 1 us each).  Here GRP slots
// are requested before the first one is added, branch-free: a slot index past the end is clamped
// to the last slot and its values are multiplied by 0 (a load under a branch would make the
// compiler wait for everything outstanding at the join).  The additions keep the slot order of
// the plain loop.  load(s, slot) fills a Slot; add(slot, keep) accumulates keep * slot, keep = 1 or 0.
template <int GRP, typename Slot, typename Load, typename Add>
__device__ __forceinline__ void sum_slots(int s_first, int s_last, Load load, Add add) {
    if (s_last - s_first == 1) {      // one slot (scanned totals, or the segment next to the end): no spare loads
        Slot t;
        load(s_first, t);
        add(t, 1.0f);
        return;
    }
    for (int s0 = s_first; s0 < s_last; s0 += GRP) {
        Slot t[GRP];
#pragma unroll
        for (int u = 0; u < GRP; ++u) load(min(s0 + u, s_last - 1), t[u]);
#pragma unroll
        for (int u = 0; u < GRP; ++u) add(t[u], (s0 + u < s_last) ? 1.0f : 0.0f);
    }
}

// Workgroup index -> (sequence, segment) of the scan kernels.  Workgroups are dealt to the 8 XCDs
// round-robin by index, and the work of a workgroup grows with its segment number (it reads one
// fp32 state total per earlier -- or, in the reverse sweep, later -- segment).  With the segments
// of a sequence on consecutive indices and a segment count of 2, 4 or 8, every workgroup of the
// heaviest kind lands on the same one, two or four XCDs, whose share of the memory fabric then
// sets the kernel time.  Here the 8 sequences of a group go to the 8 XCDs and the segments of a
// sequence stay on one XCD: every XCD gets the same mix, and the totals that several segments
// of a sequence read are fetched into that XCD's L2 once.
__device__ __forceinline__ void seq_seg_of_block(int b, int N, int nseg, int& n, int& seg) {
    const int per_group = 8 * nseg, full = N / 8;
    const int g = b / per_group;
    if (g < full) {
        const int r = b - g * per_group;
        n = 8 * g + (r & 7);
        seg = r >> 3;
    } else {                       // the last N % 8 sequences
        const int m = N - 8 * full, r = b - full * per_group;
        n = 8 * full + r % m;
        seg = r / m;
    }
}

__device__ __forceinline__ float sum_over_groups(float x) {
    x += __shfl_xor(x, 16, 64);
    x += __shfl_xor(x, 32, 64);
    return x;
}

// ---------------------------------------------------------------------------
// chunk movement: a chunk is 64 consecutive time steps of one (batch, head)
// sequence, F halves per step; in HBM consecutive steps are `row_stride` halves
// apart ([T, N, F] time-major layout).
// ---------------------------------------------------------------------------
// Loads never depend on control flow: a row past the end of the chunk is read from the
// last valid row (clamped address) and replaced by zeros when the registers are written
// to LDS, i.e. after the data has arrived.  A load under a lane- or row-dependent branch
// makes the compiler wait for all outstanding loads at the join, which serialises the
// prefetch of a chunk into several memory round trips.
template <int F, int NT = kThreads>
struct ChunkRegs {
    static constexpr int kPieces = kChunk * F / 8 / NT;   // 16-byte pieces per thread
    static_assert(kPieces >= 1, "feature width too small for this many threads");
    uint4 v[kPieces];
    unsigned char drop[kPieces];   // non-zero: the piece's row is masked out (chunk_mask_rows)
    int rows;                      // rows of the chunk that exist
};

// rows_valid >= 1
template <int F, int NT = kThreads>
__device__ __forceinline__ void chunk_g2r(ChunkRegs<F, NT>& r, const half_t* __restrict__ base,
                                          int64_t row_stride, int rows_valid, int tid) {
    constexpr int PPR = F / 8;
    r.rows = min(rows_valid, kChunk);
#pragma unroll
    for (int it = 0; it < ChunkRegs<F, NT>::kPieces; ++it) {
        const int p = tid + NT * it;
        const int row = min(p / PPR, r.rows - 1), c8 = p % PPR;
        r.v[it] = *reinterpret_cast<const uint4*>(base + (int64_t)row * row_stride + c8 * 8);
        r.drop[it] = 0;
    }
}

// 64 rows x F halves of a full chunk.  The address of a piece is a base that is the same for the
// whole wave (tensor + sequence + chunk + piece index * rows per pass: scalar registers and scalar
// arithmetic) plus one 32-bit byte offset per lane, set up once: a load costs no vector
// arithmetic and the row addresses take one register per tensor.  64 rows of a tensor must span
// less than 4 GiB (the launchers check).
template <int F, int NT = kThreads>
struct RowPtrs {
    static constexpr int kPieces = ChunkRegs<F, NT>::kPieces;
    static constexpr int PPR = F / 8;                       // 16-byte pieces per row
    static constexpr int kRowsPerPass = NT / PPR;
    const char* base;       // wave-uniform
    int64_t pass_bytes;     // wave-uniform: kRowsPerPass rows
    unsigned lane_off;
    __device__ __forceinline__ void init(const half_t* tensor, int64_t row_stride, int tid) {
        base = reinterpret_cast<const char*>(tensor);
        pass_bytes = (int64_t)kRowsPerPass * row_stride * 2;
        lane_off = (unsigned)(tid / PPR) * (unsigned)(row_stride * 2) + (unsigned)(tid % PPR) * 16u;
    }
    __device__ __forceinline__ void load_full(ChunkRegs<F, NT>& r, int64_t chunk_off) const {
        r.rows = kChunk;
        const char* b = base + chunk_off * 2;
#pragma unroll
        for (int it = 0; it < kPieces; ++it) {
            r.v[it] = *reinterpret_cast<const uint4*>(b + it * pass_bytes + lane_off);
            r.drop[it] = 0;
        }
    }
};

// store through a wave-uniform base (scalar registers, scalar address arithmetic) plus one 32-bit
// byte offset per lane that is set up once: no vector arithmetic per store
template <typename V>
__device__ __forceinline__ void store_lane(half_t* uniform_base, unsigned lane_off_bytes, const V& value) {
    *reinterpret_cast<V*>(reinterpret_cast<char*>(uniform_base) + lane_off_bytes) = value;
}

// mark the rows whose mask byte is non-zero (mask already offset to the chunk's first
// step); they are written to LDS as zeros.  Call after chunk_g2r.
template <int F, int NT = kThreads>
__device__ __forceinline__ void chunk_mask_rows(ChunkRegs<F, NT>& r, const uint8_t* __restrict__ mask, int tid) {
    constexpr int PPR = F / 8;
#pragma unroll
    for (int it = 0; it < ChunkRegs<F, NT>::kPieces; ++it) {
        const int row = min((tid + NT * it) / PPR, r.rows - 1);
        r.drop[it] = mask[row];
    }
}

template <int F, int NT = kThreads>
__device__ __forceinline__ void chunk_r2s(const ChunkRegs<F, NT>& r, half_t* Xs, int ld, int tid) {
    constexpr int PPR = F / 8;
#pragma unroll
    for (int it = 0; it < ChunkRegs<F, NT>::kPieces; ++it) {
        const int p = tid + NT * it;
        const int row = p / PPR, c8 = p % PPR;
        const bool keep = row < r.rows && !r.drop[it];
        uint4 x = r.v[it];
        x.x = keep ? x.x : 0u; x.y = keep ? x.y : 0u; x.z = keep ? x.z : 0u; x.w = keep ? x.w : 0u;
        *reinterpret_cast<uint4*>(Xs + row * ld + c8 * 8) = x;
    }
}

// 1 / x for x >= 1 (denominators): the hardware approximation and one Newton step, 3 vector
// instructions where the correctly rounded quotient takes about ten; the result differs from
// it by at most one unit in the last place, far below the fp16 rounding of whatever it scales.
__device__ __forceinline__ float rcp_nr(float x) {
    const float y = __builtin_amdgcn_rcpf(x);
    return __builtin_fmaf(__builtin_fmaf(-x, y, 1.0f), y, y);
}

// Eight halves times one fp32 factor, each product formed in fp32 and rounded once to fp16:
// the mixed-precision multiply-add reads the half in place and writes the rounded half, one
// instruction per element (convert, multiply, convert and pack take 2.5).
__device__ __forceinline__ uint4 scale_h8(uint4 x, float f) {
    uint4 y;
    const unsigned in[4] = {x.x, x.y, x.z, x.w};
    unsigned out[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        unsigned r;
        asm("v_fma_mixlo_f16 %0, %1, %2, 0 op_sel_hi:[1,0,0]" : "=v"(r) : "v"(in[i]), "v"(f));
        asm("v_fma_mixhi_f16 %0, %1, %2, 0 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "+v"(r) : "v"(in[i]), "v"(f));
        out[i] = r;
    }
    y.x = out[0]; y.y = out[1]; y.z = out[2]; y.w = out[3];
    return y;
}

// dot product of two rows of eight halves, accumulated in fp32 (v_dot2_f32_f16: 4 instructions)
__device__ __forceinline__ float dot_h8(uint4 a, uint4 b) {
    typedef _Float16 hh2 __attribute__((ext_vector_type(2)));
    const unsigned ua[4] = {a.x, a.y, a.z, a.w}, ub[4] = {b.x, b.y, b.z, b.w};
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i)
        acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(hh2, ua[i]), __builtin_bit_cast(hh2, ub[i]), acc, false);
    return acc;
}

// Sum of x over groups of W adjacent lanes (W = 4, 8 or 16, groups aligned to W), result in every
// lane of the group: data-parallel-primitive moves inside the vector unit (quad permutes, then the
// mirror of a half row / of a row, which for lanes that already hold their quad's / half row's
// sum fetches the other one), no trip through the LDS crossbar.  Same pairing of the additions
// as a butterfly over lane ^ 1, ^ 2, ^ 4, ^ 8.
template <int W>
__device__ __forceinline__ float sum_adjacent(float x) {
    static_assert(W == 4 || W == 8 || W == 16, "group width");
    auto dpp = [](float v, auto ctrl) {
        return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), decltype(ctrl)::value,
                                                                     0xf, 0xf, true));
    };
    x += dpp(x, std::integral_constant<int, 0xB1>{});                       // quad_perm [1, 0, 3, 2]
    x += dpp(x, std::integral_constant<int, 0x4E>{});                       // quad_perm [2, 3, 0, 1]
    if constexpr (W >= 8) x += dpp(x, std::integral_constant<int, 0x141>{});    // row_half_mirror
    if constexpr (W >= 16) x += dpp(x, std::integral_constant<int, 0x140>{});   // row_mirror
    return x;
}

// same, each row multiplied by scale[piece] (fp32) before the store
template <int F, int NT = kThreads>
__device__ __forceinline__ void chunk_r2s_scaled(const ChunkRegs<F, NT>& r, const float* scale,
                                                 half_t* Xs, int ld, int tid) {
    constexpr int PPR = F / 8;
#pragma unroll
    for (int it = 0; it < ChunkRegs<F, NT>::kPieces; ++it) {
        const int p = tid + NT * it;
        const int row = p / PPR, c8 = p % PPR;
        const float sc = row < r.rows ? scale[it] : 0.f;
        *reinterpret_cast<uint4*>(Xs + row * ld + c8 * 8) = scale_h8(r.v[it], sc);
    }
}

}  // namespace rfa
