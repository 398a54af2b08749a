// Fused QKV projection for gfx950 (MI355X, CDNA4): the front end of the attention forward.
//
//   qkv[m][n] = sum_k x[m][k] w[k][n] (+ bias[n]),   m < M = B L,  n < N = 3 F,  F = R H
// written as the packed [B, L, 3, R H] tensor whose three slices fa_fwd_strided reads as q, k and v
// without a copy, with an optional rotary position encoding (rotate-half form) applied to the q and
// k slices before the one rounding to 16 bits.  The reference lists this front end as not done
// (reference README.md:137); its attention kernel takes q, k, v as three separate tensors
// (reference src/fused_attn_extention.cu:15-22).
//
// One kernel, one pass: a workgroup of eight wave64s owns a 256 x 256 tile of the output and walks
// the contraction in slices of 64.  The x and w slices are written into LDS by the loads themselves
// (direct-to-LDS loads: no staging registers, no LDS store instructions), into a ring of two
// 64 KB slots.  One load instruction of a wave fills 1 KB of consecutive LDS, lane l the 16 bytes
// at 16 l, and each lane is free to fetch any 16-byte chunk: the tiles stay row-major without
// padding, whole cache lines per wave on the global side, and the chunks of a row are permuted
// (XOR with a few bits of the row index) so that the operand reads touch every bank once:
//   x slot [256 rows][8 chunks]:  chunk c of row r sits at position c ^ ((r >> 1) & 7)
//          (16 consecutive rows of one logical chunk cover the 16 bank groups of 16 bytes);
//   w slot [64 rows][32 chunks]:  chunk c of contraction row k sits at c ^ (((k & 3) << 2) | (((k >> 3) & 1) << 1))
//          (the four rows a transpose read touches land in the four 64-byte quarters of the banks,
//          rows eight apart in different halves of a quarter).
// The products are computed transposed, C^T = W^T X^T, with v_mfma_f32_16x16x32_f16: the A operand
// W^T (16 outputs n x 32 k) comes from the row-major w slice through the LDS transpose read
// (ds_read_b64_tr_b16), the B operand X^T (32 k x 16 rows m) is a plain 16-byte read of a row of x.
// In the accumulator a lane then owns one output row m and, per 16 x 16 block, a run of four output
// features n: bias and rotation are applied in registers (the partner feature n + H/2 of a
// rotation sits in the same lane, or 32 lanes away at head_dim 16); the rounded rows then pass
// through a small per-wave LDS tile and leave as whole 256-byte row segments with streaming stores.
// The 16 x 16 x 32 instruction has the flops per clock of the 32 x 32 x 16 one with half the
// accumulator traffic per flop; on this chip, whose clock follows the switching activity, the
// same kernel written on 32 x 32 x 16 tiles measured 8.7 to 15 % slower on the same box.
//
// A wave owns 64 rows x 128 features (8 x 4 blocks of 16 x 16, 128 accumulator registers); its
// 128 features are whole heads for every head_dim up to 128.
#pragma once

#include "fused_attn_kernel.hpp"

namespace fa {
namespace qkv {

constexpr int kTileM = 256;
constexpr int kTileN = 256;
constexpr int kTileK = 64;    // contraction steps per slice (one ring slot)
constexpr int kWaves = 8;
constexpr int kBand = 4;      // row tiles per band of the tile order
constexpr int kSlots = 2;     // ring slots: one is read while the other is filled
constexpr int kRingHalves = kSlots * (kTileM + kTileN) * kTileK;                           // 128 KB
constexpr int kStageHalves = 16 * 128;      // per wave: 16 output rows of the wave's 128 features (4 KB)
constexpr int kLdsBytes = (kRingHalves + kWaves * kStageHalves) * (int)sizeof(_Float16);   // 160 KB

struct Params {
    const _Float16* x;       // [M, K]
    const _Float16* w;       // [K, N]
    const _Float16* bias;    // [N] or nullptr
    _Float16* out;           // [M, N]
    const float* rope_cos;   // [L, H / 2] or nullptr
    const float* rope_sin;
    int M, K, N;
    int F;                   // features per slice (N = 3 F)
    int L;                   // sequence length: position of row m is m % L
    int tiles_n;             // ceil(N / 256)
    int total_tiles;         // tiles_m * tiles_n
    int total_wgs;           // workgroups that take tiles: min(total_tiles, one per compute unit)
    int wgs_per_xcd;         // ceil(total_wgs / 8): the grid is 8 times this
};

__device__ __forceinline__ void dma16(uint32_t lds_addr, const void* base, uint32_t voff) {
    // M0 holds the LDS address of lane 0's 16 bytes.  Written in assembly so that the compiler
    // does not see an LDS write (it would wait for the load before the wave's next LDS read).
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :: "s"(lds_addr), "v"(voff), "s"(base) : "memory", "m0");
}
template <int N>
__device__ __forceinline__ void wait_loads() { asm volatile("s_waitcnt vmcnt(%0)" :: "n"(N) : "memory"); }

template <int N>
using I = std::integral_constant<int, N>;

// HR = head_dim of the rotation (16, 32, 64, 128), or 0 for none.
template <int HR, bool BF>
__global__ __launch_bounds__(kWaves * 64, 2) void qkv_proj_kernel(const Params p) {
    constexpr int KS = kTileK;
    constexpr int NSLOT = kSlots;
    constexpr int CPRX = KS / 8;                        // 16-byte chunks per row of an x slot
    constexpr int LX = CPRX / 2;                        // x loads per wave and step
    constexpr int LW = KS / 16;                         // w loads per wave and step
    constexpr int XSLOT = kTileM * KS;                  // halves
    constexpr int WSLOT = KS * kTileN;
    constexpr int NSUB = KS / 32;                       // 32-wide contraction sub-steps per step
    extern __shared__ __attribute__((aligned(16))) _Float16 smem[];
    _Float16* const xs = smem;
    _Float16* const ws = smem + NSLOT * XSLOT;
    typedef short short8v __attribute__((ext_vector_type(8)));

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c16 = lane & 15;
    const int g4 = lane >> 4;
    const int wm = wave >> 1;
    const int wn = wave & 1;
    _Float16* const stage = smem + kRingHalves + wave * kStageHalves;     // this wave's output staging tile

    // A resident grid: workgroup `logical` takes the tiles logical, logical + G, logical + 2 G, ...
    // Workgroups are dealt round-robin to the XCDs, so they are renumbered first: one XCD (one L2)
    // then works on consecutive tiles, and the tiles are ordered in bands of four row tiles, feature
    // tile by feature tile inside a band: the 32 workgroups of an XCD cover about 4 x 8 tiles at a
    // time and share 4 row blocks of x and 8 column blocks of w in L2, instead of 1 and 32.
    const int wg = blockIdx.x;
    const int logical = (wg % kNumXcd) * p.wgs_per_xcd + wg / kNumXcd;
    if (logical >= p.total_wgs) return;
    const int tiles_m = p.total_tiles / p.tiles_n;
    auto tile_origin = [&](int tile, int& m0, int& n0) __attribute__((always_inline)) {
        const int band = tile / (kBand * p.tiles_n);
        const int in_band = tile - band * (kBand * p.tiles_n);
        const int band_rows = min(kBand, tiles_m - band * kBand);
        m0 = (band * kBand + in_band % band_rows) * kTileM;
        n0 = (in_band / band_rows) * kTileN;
    };

    // ---- the load stream -----------------------------------------------------------------------
    // Load instruction i of wave w fills the LDS positions (16-byte units) (w L + i) 64 + lane of a
    // slot; the lane fetches the chunk that belongs there: x position = row * 8 + (chunk ^ fx(row)),
    // w position = contraction row * 32 + (chunk ^ fw(row)).  Rows of x beyond M are read from row
    // M - 1 and feature chunks of w beyond N from chunk 0 (their results are never stored).  The
    // stream runs over all (tile, slice) pairs of the workgroup: the first slices of the next tile
    // are on their way while this one is finished.
    uint32_t xvo[LX], wvo[LW];
    const char* xsrc = nullptr;
    const char* wsrc = nullptr;
    int fetch_tile = logical, fetch_kt = 0;
    const int ksteps = p.K / KS;
    auto aim = [&]() __attribute__((always_inline)) {
        int m0, n0;
        tile_origin(fetch_tile, m0, n0);
#pragma unroll
        for (int i = 0; i < LX; ++i) {
            const int pos = (wave * LX + i) * 64 + lane;
            const int row = pos / CPRX;
            const int c = (pos % CPRX) ^ ((row >> 1) & 7);
            const int grow = min(m0 + row, p.M - 1) - m0;       // rows beyond M: never stored
            xvo[i] = ((uint32_t)grow * (uint32_t)p.K + (uint32_t)c * 8u) * 2u;
        }
#pragma unroll
        for (int i = 0; i < LW; ++i) {
            const int pos = (wave * LW + i) * 64 + lane;
            const int krow = pos >> 5;
            int c = (pos & 31) ^ (((krow & 3) << 2) | (((krow >> 3) & 1) << 1));
            if (n0 + c * 8 >= p.N) c = 0;                        // features beyond N: never stored
            wvo[i] = ((uint32_t)krow * (uint32_t)p.N + (uint32_t)c * 8u) * 2u;
        }
        xsrc = reinterpret_cast<const char*>(p.x + (int64_t)m0 * p.K);
        wsrc = reinterpret_cast<const char*>(p.w + n0);
    };
    const uint32_t xs_lds = (uint32_t)(uintptr_t)(FA_LDS void*)xs + (uint32_t)(wave * LX) * 1024u;
    const uint32_t ws_lds = (uint32_t)(uintptr_t)(FA_LDS void*)ws + (uint32_t)(wave * LW) * 1024u;
    // The LX + LW loads of a step are issued in two parts, one sub-step apart: 64 KB per step and
    // compute unit keep the texture path busy for half the step, and a wave that issues all its
    // loads at once waits at the issue port while the queue drains (measured: +3.5 % for two
    // parts; four parts, one per sub-step, lose that again because the last ones are issued too
    // late to land before the step ends).
    constexpr int NP = 2;
    constexpr int LPP = (LX + LW) / NP;              // loads per part
    static_assert((LX + LW) % NP == 0 && NP <= NSUB, "whole loads per part, at most one part per sub-step");
    auto issue_part = [&](int slot, auto part_c) __attribute__((always_inline)) {
        constexpr int PART = decltype(part_c)::value;
#pragma unroll
        for (int j = PART * LPP; j < (PART + 1) * LPP; ++j) {
            if (j < LX)
                dma16(xs_lds + (uint32_t)(slot * XSLOT * 2 + j * 1024), xsrc, xvo[j]);
            else
                dma16(ws_lds + (uint32_t)(slot * WSLOT * 2 + (j - LX) * 1024), wsrc, wvo[j - LX]);
        }
        if constexpr (PART == NP - 1) {
            xsrc += KS * 2;
            wsrc += (int64_t)KS * p.N * 2;
            if (++fetch_kt == ksteps) {
                fetch_kt = 0;
                fetch_tile += p.total_wgs;
                if (fetch_tile < p.total_tiles) aim();
            }
        }
    };
    auto issue = [&](int slot) __attribute__((always_inline)) {
        issue_part(slot, std::integral_constant<int, 0>{});
        issue_part(slot, std::integral_constant<int, 1>{});
    };

    // acc[nt][mt][r]: row m = m0 + wm 64 + mt 16 + c16, feature n = n0 + wn 128 + nt 16 + 4 g4 + r
    floatx4 acc[8][4];
#pragma unroll
    for (int nt = 0; nt < 8; ++nt)
#pragma unroll
        for (int mt = 0; mt < 4; ++mt) acc[nt][mt] = floatx4{0.f, 0.f, 0.f, 0.f};

    // ---- per-lane parts of the operand addresses (halves inside a slot) ---------------------------
    // B operand (x): row wm 64 + mt 16 + c16, logical chunk 4 s + g4 (k-slots 8 g4 ... of sub-step s are
    // contraction indices 32 s + 8 g4 ...).  The LDS serves the 16-byte reads of lanes 0-3, 12-15, 20-23
    // and 24-27 together (and 4-7, 8-11, 16-19, 28-31): with the chunk of row r at c ^ ((r >> 1) & 7)
    // and neighbouring chunks for g4 and g4 ^ 1 each such set of 16 lanes covers all banks once.
    int xrd[NSUB];
    {
        const int r0 = wm * 64 + c16;
        const int fx = (c16 >> 1) & 7;     // wm 64 and mt 16 do not reach these bits
#pragma unroll
        for (int s = 0; s < NSUB; ++s) xrd[s] = (r0 * CPRX + ((4 * s + g4) ^ fx)) * 8;
    }
    // A operand (w^T), transpose reads: lane s16 of the 16-lane group g4 points at contraction row
    // 32 s + 8 g4 + s16 / 4 (+ 4 for the second read), features 4 (s16 % 4) ... of the 16 of feature
    // block nt; lane j of the group receives four consecutive contraction rows of feature j, so the
    // two reads fill the k-slots 8 g4 ... 8 g4 + 7.  Chunk c of contraction row k sits at
    // c ^ (((k & 3) << 2) | (((k >> 3) & 1) << 1)): the four rows of a read land in the four 64-byte
    // quarters of the banks, and the rows of g4 and g4 ^ 1, eight apart, in different halves of a
    // quarter.  Feature block nt adds 2 nt to the chunk index, which commutes with that XOR: the
    // address of block nt is the address of block 0 XOR 16 nt (in halves).
    int wrd0;
    {
        const int kk = c16 >> 2;
        const int swz = (kk << 2) | ((g4 & 1) << 1);
        const int krow = 8 * g4 + kk;
        wrd0 = krow * kTileN + (wn * 16 + (swz | ((c16 & 3) >> 1))) * 8 + 4 * (c16 & 1);
    }

    // ---- end of a tile: bias, rotation, one rounding, whole-row stores; the accumulators start over ---
    // The accumulators are only read here (results are formed in temporaries): modifying them in
    // place inside the step loop makes the compiler carry a second copy of all of them.
    auto finish_tile = [&](int done_tile) __attribute__((always_inline)) {
        int m0, n0;
        tile_origin(done_tile, m0, n0);
        const int nw = n0 + wn * 128;
        // one run of four features of one row with the bias added
        auto biased = [&](int nt, int mt, int n) __attribute__((always_inline)) {
            floatx4 v = acc[nt][mt];
            if (p.bias != nullptr && n < p.N) {
                const u16x4 b4 = *reinterpret_cast<const u16x4*>(p.bias + n);
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] += BF ? bf16::elem_to_float(b4[e]) : elem_to_float(b4[e]);
            }
            return v;
        };
        // The results leave through a private LDS tile of 16 rows x 128 features per wave, so that
        // every store instruction writes whole rows (16 lanes x 16 bytes = the wave's 256 bytes of a
        // row) as streaming stores.  A lane holds one row of a 16-row block and runs of four features;
        // chunk c (16 bytes) of stage row r sits at c ^ r.
        auto store_run = [&](floatx4 v, int nt) __attribute__((always_inline)) {
            u16x4 hv;
#pragma unroll
            for (int e = 0; e < 4; ++e) hv[e] = BF ? bf16::float_to_elem(v[e]) : float_to_elem(v[e]);
            // (the row index is made opaque per run: otherwise the swizzled addresses of a row are all
            // computed ahead and held in registers through the whole epilogue)
            int r = c16;
            asm volatile("" : "+v"(r));
            *reinterpret_cast<u32x2*>(stage + r * 128 + (((2 * nt + (g4 >> 1)) ^ r) * 8) + 4 * (g4 & 1)) = __builtin_bit_cast(u32x2, hv);
        };
#pragma unroll
        for (int mt = 0; mt < 4; ++mt) {
            const int m = m0 + wm * 64 + mt * 16 + c16;
            if constexpr (HR > 0) {
                // rotate-half: within a head, feature i < HR / 2 pairs with feature i + HR / 2:
                //   out[i] = y[i] cos_i - y[i + HR/2] sin_i,  out[i + HR/2] = y[i + HR/2] cos_i + y[i] sin_i
                // with cos_i, sin_i taken at the row's position m % L.  Only the q and k slices (n < 2 F).
                const int pos = (m < p.M ? m : p.M - 1) % p.L;
                const float* const cs = p.rope_cos + (int64_t)pos * (HR / 2);
                const float* const sn = p.rope_sin + (int64_t)pos * (HR / 2);
                if constexpr (HR >= 32) {
                    // the partner run sits in the same lane, HR / 32 feature blocks on
                    constexpr int D = HR / 32;
#pragma unroll
                    for (int pr = 0; pr < 4; ++pr) {
                        const int nt_a = (pr / D) * 2 * D + pr % D, nt_b = nt_a + D;
                        const int n_a = nw + nt_a * 16 + 4 * g4, n_b = nw + nt_b * 16 + 4 * g4;
                        floatx4 a = biased(nt_a, mt, n_a);
                        floatx4 b = biased(nt_b, mt, n_b);
                        if (n_a < 2 * p.F) {
                            const int i0 = n_a % (HR / 2);      // index inside the half head
                            const floatx4 c4 = *reinterpret_cast<const floatx4*>(cs + i0);
                            const floatx4 s4 = *reinterpret_cast<const floatx4*>(sn + i0);
                            const floatx4 ra = a * c4 - b * s4;
                            const floatx4 rb = b * c4 + a * s4;
                            a = ra;
                            b = rb;
                        }
                        store_run(a, nt_a);
                        store_run(b, nt_b);
                        // one pair at a time: all table loads at once would not fit in the registers
                        __builtin_amdgcn_sched_barrier(0);
                    }
                } else {
                    // head_dim 16: a head is one feature block and the partner of a run sits 32 lanes away
#pragma unroll
                    for (int nt = 0; nt < 8; ++nt) {
                        const int n = nw + nt * 16 + 4 * g4;
                        floatx4 a = biased(nt, mt, n);
                        floatx4 b;
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const float ae = a[e];      // (a bit cast taken straight from a vector element reads element 0)
                            b[e] = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((lane ^ 32) << 2, __builtin_bit_cast(int, ae)));
                        }
                        if (n < 2 * p.F) {
                            const int i0 = n % 8;
                            const floatx4 c4 = *reinterpret_cast<const floatx4*>(cs + i0);
                            const floatx4 s4 = *reinterpret_cast<const floatx4*>(sn + i0);
                            a = g4 < 2 ? a * c4 - b * s4 : a * c4 + b * s4;
                        }
                        store_run(a, nt);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            } else {
#pragma unroll
                for (int nt = 0; nt < 8; ++nt) store_run(biased(nt, mt, nw + nt * 16 + 4 * g4), nt);
            }
            // LDS operations of one wave complete in order; the waits keep the compiler from moving
            // the reads above the writes (and the next block's writes above these reads)
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int r = 4 * i + (lane >> 4), ch = lane & 15;
                const u32x4 w = *reinterpret_cast<const u32x4*>(stage + r * 128 + ((ch ^ r) * 8));
                const int mr = m0 + wm * 64 + mt * 16 + r;
                const int n = nw + ch * 8;
                if (mr < p.M && n < p.N)
                    __builtin_nontemporal_store(w, reinterpret_cast<u32x4*>(p.out + (int64_t)mr * p.N + n));
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        }
#pragma unroll
        for (int nt = 0; nt < 8; ++nt)
#pragma unroll
            for (int mt = 0; mt < 4; ++mt) acc[nt][mt] = floatx4{0.f, 0.f, 0.f, 0.f};
    };

    const int my_tiles = (p.total_tiles - logical + p.total_wgs - 1) / p.total_wgs;
    const int total_steps = my_tiles * ksteps;
    int tile = logical, kt = 0;

    // Operand registers.  B (rows of x): the four fragments of a 32-wide sub-step, two sets.  A (w^T): the
    // eight fragments of a sub-step are used pair by pair (one unit = 2 A fragments x 4 B fragments = 8
    // matrix instructions), two pairs of registers: the reads of a pair are issued before the matrix
    // instructions of the pair before it, the B fragments of the next sub-step two units ahead.
    half8 wop[2][2], xop[2][4];
    auto load_a = [&](auto set_c, int slot, auto s_c, auto pair_c) __attribute__((always_inline)) {
        constexpr int SET = decltype(set_c)::value;
        constexpr int S = decltype(s_c)::value;
        constexpr int PAIR = decltype(pair_c)::value;
        const _Float16* const wb = ws + slot * WSLOT;
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const _Float16* p0 = wb + (wrd0 ^ (16 * (2 * PAIR + e))) + (32 * S) * kTileN;
            const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((FA_LDS short4v*)(p0));
            const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((FA_LDS short4v*)(p0 + 4 * kTileN));
            const short8v both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            wop[SET][e] = __builtin_bit_cast(half8, both);
        }
    };
    auto load_b = [&](auto set_c, int slot, auto s_c) __attribute__((always_inline)) {
        constexpr int SET = decltype(set_c)::value;
        constexpr int S = decltype(s_c)::value;
        const _Float16* const xb = xs + slot * XSLOT;
#pragma unroll
        for (int mt = 0; mt < 4; ++mt)
            xop[SET][mt] = *reinterpret_cast<const half8*>(xb + xrd[S] + mt * 16 * CPRX * 8);
    };
    auto multiply = [&](auto aset_c, auto bset_c, auto pair_c) __attribute__((always_inline)) {
        constexpr int ASET = decltype(aset_c)::value;
        constexpr int BSET = decltype(bset_c)::value;
        constexpr int PAIR = decltype(pair_c)::value;
#pragma unroll
        for (int e = 0; e < 2; ++e)
#pragma unroll
            for (int mt = 0; mt < 4; ++mt) {
                if constexpr (BF)
                    acc[2 * PAIR + e][mt] = bf16::mfma16(wop[ASET][e], xop[BSET][mt], acc[2 * PAIR + e][mt]);
                else
                    acc[2 * PAIR + e][mt] = mfma16(wop[ASET][e], xop[BSET][mt], acc[2 * PAIR + e][mt]);
            }
    };

    // Step u reads slot u % 2 while the loads of step u + 1 fill the other one.  One barrier per
    // step, placed before the matrix instructions of the step's last unit: by then every wave has
    // the operands of that unit in registers, so the slot is free for the loads of step u + 2, and
    // the data of step u + 1 (each wave has waited for its own part) are visible to everybody, so
    // the operands of its first unit are requested before the last matrix instructions of step u
    // are issued.
    static_assert(NSLOT == 2, "the waits below assume that only the next step's loads are in flight");
    static_assert(NSUB == 2, "eight units per step");
    aim();
    issue(0);
    if (total_steps > 1) {
        issue(1);
        wait_loads<LX + LW>();      // loads complete in order: all but the second step's have landed
    } else {
        wait_loads<0>();
    }
    ring_barrier();
    load_a(I<0>{}, 0, I<0>{}, I<0>{});
    load_b(I<0>{}, 0, I<0>{});

    bool pending = false;      // the second part of the loads into the previous step's slot is still to be issued
    auto step = [&](int u, auto slot_c) __attribute__((always_inline)) {
        constexpr int SLOT = decltype(slot_c)::value;
        constexpr int PREV = (SLOT + NSLOT - 1) % NSLOT;
        // unit t (sub-step t / 4, fragment pair t % 4) uses A set t % 2 and B set (t / 4) % 2
        auto unit = [&](auto t_c) __attribute__((always_inline)) {
            constexpr int T = decltype(t_c)::value;
            load_a(I<(T + 1) & 1>{}, SLOT, I<(T + 1) / 4>{}, I<(T + 1) % 4>{});
            if constexpr (T == 1) load_b(I<1>{}, SLOT, I<1>{});
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (T == 1) {
                if (pending) issue_part(PREV, I<1>{});
            }
            multiply(I<T & 1>{}, I<(T / 4) & 1>{}, I<T % 4>{});
            __builtin_amdgcn_sched_barrier(0);
        };
        unit(I<0>{});
        unit(I<1>{});
        unit(I<2>{});
        unit(I<3>{});
        unit(I<4>{});
        unit(I<5>{});
        unit(I<6>{});
        // this wave's loads of step u + 1 have landed (the stores of an epilogue are waited for
        // with them), its reads of this step's slot have all returned
        wait_loads<0>();
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        ring_barrier();
        pending = u + NSLOT < total_steps;
        if (pending) issue_part(SLOT, I<0>{});
        // (at the end of a tile the operands of the next step are requested behind the epilogue, which
        // needs the registers)
        const bool last = kt + 1 == ksteps;
        if (u + 1 < total_steps && !last) {
            load_a(I<0>{}, (SLOT + 1) % NSLOT, I<0>{}, I<0>{});
            load_b(I<0>{}, (SLOT + 1) % NSLOT, I<0>{});
        }
        __builtin_amdgcn_sched_barrier(0);
        multiply(I<1>{}, I<1>{}, I<3>{});
        __builtin_amdgcn_sched_barrier(0);
        if (last) {
            finish_tile(tile);
            kt = 0;
            tile += p.total_wgs;
            __builtin_amdgcn_sched_barrier(0);
            if (u + 1 < total_steps) {
                load_a(I<0>{}, (SLOT + 1) % NSLOT, I<0>{}, I<0>{});
                load_b(I<0>{}, (SLOT + 1) % NSLOT, I<0>{});
            }
        } else {
            ++kt;
        }
    };
    for (int u = 0; u < total_steps; u += NSLOT) {
        step(u, I<0>{});
        if (u + 1 < total_steps) step(u + 1, I<1>{});
    }
}

}  // namespace qkv
}  // namespace fa
