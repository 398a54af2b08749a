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
//   w slot [64 rows][32 chunks]:  chunk c of contraction row k sits at c ^ ((k & 3) << 2)
//          (the four rows a transpose read touches land in the four 64-byte quarters of the banks).
// The products are computed transposed, C^T = W^T X^T, with v_mfma_f32_32x32x16_f16: the A operand
// W^T (32 outputs n x 16 k) comes from the row-major w slice through the LDS transpose read
// (ds_read_b64_tr_b16), the B operand X^T (16 k x 32 rows m) is a plain 16-byte read of a row of x.
// In the accumulator a lane then owns one output row m and, per 32 x 32 block, 16 output features
// n in runs of four: bias and rotation are applied in registers (the partner feature n + H/2 of a
// rotation sits in the same lane); the rounded rows then pass through a small per-wave LDS tile
// and leave as whole 256-byte row segments with streaming stores.
//
// A wave owns 64 rows x 128 features (4 x 2 blocks of 32 x 32, 128 accumulator registers); its
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
    constexpr int NSUB = KS / 16;                       // 16-wide contraction sub-steps per step
    extern __shared__ __attribute__((aligned(16))) _Float16 smem[];
    _Float16* const xs = smem;
    _Float16* const ws = smem + NSLOT * XSLOT;
    typedef short short8v __attribute__((ext_vector_type(8)));

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = lane >> 5;
    const int ln = lane & 31;
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
            int c = (pos & 31) ^ ((krow & 3) << 2);
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

    floatx16 acc[4][2];
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[nt][mt][r] = 0.f;

    // ---- per-lane parts of the operand addresses (halves inside a slot) ---------------------------
    // B operand (x): row wm 64 + mt 32 + ln, logical chunk 2 s + g
    int xrd[NSUB];
    {
        const int r0 = wm * 64 + ln;
        const int fx = (ln >> 1) & 7;      // wm 64 and mt 32 do not reach these bits
#pragma unroll
        for (int s = 0; s < NSUB; ++s) xrd[s] = (r0 * CPRX + ((2 * s + g) ^ fx)) * 8;
    }
    // A operand (w^T), transpose read: lane s16 of a 16-lane group points at contraction row
    // 8 g + s16 / 4 (+ 4 for the second read), features 4 (s16 % 4) ... of the 16 that start at
    // 16 * ((lane / 16) % 2) of feature block nt; lane j of the group receives four consecutive
    // contraction rows of feature j: slot (g, i) of the operand is contraction index 16 s + 8 g + i,
    // the order in which the 16-byte read of x delivers them.
    int wrd[4];
    {
        const int s16 = lane & 15;
        const int kk = (s16 >> 2) & 3;
        const int krow = 8 * g + (s16 >> 2);
#pragma unroll
        for (int nt = 0; nt < 4; ++nt) {
            const int c = wn * 16 + ((nt ^ kk) << 2) + 2 * ((lane >> 4) & 1) + ((s16 & 3) >> 1);
            wrd[nt] = krow * kTileN + c * 8 + 4 * (s16 & 1);
        }
    }

    // ---- end of a tile: bias, rotation, one rounding, whole-row stores; the accumulators start over ---
    // acc[nt][mt][r]: row m = m0 + wm 64 + mt 32 + ln, feature n = n0 + wn 128 + nt 32 + 8 (r / 4) + 4 g + r % 4.
    // The accumulators are only read here (results are formed in temporaries): modifying them in
    // place inside the step loop makes the compiler carry a second copy of all of them.
    auto finish_tile = [&](int done_tile) __attribute__((always_inline)) {
        int m0, n0;
        tile_origin(done_tile, m0, n0);
        const int nw = n0 + wn * 128;
        // one run of four features of one row: bias added, rounded, stored
        auto biased = [&](int nt, int mt, int r4, int n) __attribute__((always_inline)) {
            floatx4 v = {acc[nt][mt][4 * r4], acc[nt][mt][4 * r4 + 1], acc[nt][mt][4 * r4 + 2], acc[nt][mt][4 * r4 + 3]};
            if (p.bias != nullptr && n < p.N) {
                const u16x4 b4 = *reinterpret_cast<const u16x4*>(p.bias + n);
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] += BF ? bf16::elem_to_float(b4[e]) : elem_to_float(b4[e]);
            }
            return v;
        };
        // The results leave through a private LDS tile of 16 rows x 128 features per wave, so that
        // every store instruction writes whole rows (16 lanes x 16 bytes = the wave's 256 bytes of a
        // row) as streaming stores, instead of 8 bytes into each of 32 rows.  A lane holds one row
        // of a 32-row block: the block goes out in two halves of 16 rows, the lanes of the other half
        // sitting the pass out.  Chunk c (16 bytes) of stage row r sits at c ^ r: the 16
        // rows of one chunk column and the 16 chunks of one row both cover all banks.
        auto store_run = [&](floatx4 v, int nt, int r4) __attribute__((always_inline)) {
            {
                u16x4 hv;
#pragma unroll
                for (int e = 0; e < 4; ++e) hv[e] = BF ? bf16::float_to_elem(v[e]) : float_to_elem(v[e]);
                // (the row index is made opaque per run: otherwise the 16 swizzled addresses of a row
                // are all computed ahead and held in registers through the whole epilogue)
                int r = ln & 15;
                asm volatile("" : "+v"(r));
                *reinterpret_cast<u32x2*>(stage + r * 128 + (((nt * 4 + r4) ^ r) * 8) + 4 * g) = __builtin_bit_cast(u32x2, hv);
            }
        };
#pragma unroll
        for (int mh = 0; mh < 4; ++mh) {
            const int mt = mh >> 1, half = mh & 1;
            const int m = m0 + wm * 64 + mt * 32 + ln;
            if ((ln >> 4) == half) {        // the other half of the lanes sits this pass out (no table or bias loads)
            if constexpr (HR > 0) {
                // rotate-half: within a head, feature i < HR / 2 pairs with feature i + HR / 2:
                //   out[i] = y[i] cos_i - y[i + HR/2] sin_i,  out[i + HR/2] = y[i + HR/2] cos_i + y[i] sin_i
                // with cos_i, sin_i taken at the row's position m % L.  Only the q and k slices (n < 2 F).
                const int pos = (m < p.M ? m : p.M - 1) % p.L;
                const float* const cs = p.rope_cos + (int64_t)pos * (HR / 2);
                const float* const sn = p.rope_sin + (int64_t)pos * (HR / 2);
#pragma unroll
                for (int pr = 0; pr < 8; ++pr) {       // the 16 runs a lane holds per row form 8 pairs
                    int nt_a, r4_a, nt_b, r4_b;
                    if constexpr (HR == 128) {          // head = the wave's 128 features: block nt pairs with nt + 2
                        nt_a = pr >> 2; r4_a = pr & 3; nt_b = nt_a + 2; r4_b = r4_a;
                    } else if constexpr (HR == 64) {    // head = two blocks: nt pairs with nt + 1
                        nt_a = 2 * (pr >> 2); r4_a = pr & 3; nt_b = nt_a + 1; r4_b = r4_a;
                    } else if constexpr (HR == 32) {    // head = one block: register group r4 pairs with r4 + 2
                        nt_a = pr >> 1; r4_a = pr & 1; nt_b = nt_a; r4_b = r4_a + 2;
                    } else {                            // head = half a block: register group r4 pairs with r4 + 1
                        nt_a = pr >> 1; r4_a = 2 * (pr & 1); nt_b = nt_a; r4_b = r4_a + 1;
                    }
                    const int n_a = nw + nt_a * 32 + 8 * r4_a + 4 * g;      // first features of the two runs
                    const int n_b = nw + nt_b * 32 + 8 * r4_b + 4 * g;
                    floatx4 a = biased(nt_a, mt, r4_a, n_a);
                    floatx4 b = biased(nt_b, mt, r4_b, n_b);
                    if (n_a < 2 * p.F) {
                        const int i0 = n_a % (HR / 2);      // index inside the half head
                        const floatx4 c4 = *reinterpret_cast<const floatx4*>(cs + i0);
                        const floatx4 s4 = *reinterpret_cast<const floatx4*>(sn + i0);
                        const floatx4 ra = a * c4 - b * s4;
                        const floatx4 rb = b * c4 + a * s4;
                        a = ra;
                        b = rb;
                    }
                    store_run(a, nt_a, r4_a);
                    store_run(b, nt_b, r4_b);
                    // one pair at a time: all table loads at once would not fit in the registers
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else {
#pragma unroll
                for (int nt = 0; nt < 4; ++nt)
#pragma unroll
                    for (int r4 = 0; r4 < 4; ++r4) {
                        const int n = nw + nt * 32 + 8 * r4 + 4 * g;
                        store_run(biased(nt, mt, r4, n), nt, r4);
                    }
            }
            }
            // LDS operations of one wave complete in order; the waits keep the compiler from moving
            // the reads above the writes (and the next half's writes above these reads)
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int r = 4 * i + (lane >> 4), ch = lane & 15;
                const u32x4 w = *reinterpret_cast<const u32x4*>(stage + r * 128 + ((ch ^ r) * 8));
                const int mr = m0 + wm * 64 + mt * 32 + half * 16 + r;
                const int n = nw + ch * 8;
                if (mr < p.M && n < p.N)
                    __builtin_nontemporal_store(w, reinterpret_cast<u32x4*>(p.out + (int64_t)mr * p.N + n));
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        }
#pragma unroll
        for (int nt = 0; nt < 4; ++nt)
#pragma unroll
            for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[nt][mt][r] = 0.f;
    };

    const int my_tiles = (p.total_tiles - logical + p.total_wgs - 1) / p.total_wgs;
    const int total_steps = my_tiles * ksteps;
    int tile = logical, kt = 0;

    // Operand registers, two sets: the reads of a sub-step are issued before the matrix
    // instructions of the sub-step before it.
    half8 wop[2][4], xop[2][2];
    auto load_ops = [&](auto set_c, int slot, int s) __attribute__((always_inline)) {
        constexpr int SET = decltype(set_c)::value;
        const _Float16* const xb = xs + slot * XSLOT;
        const _Float16* const wb = ws + slot * WSLOT;
#pragma unroll
        for (int nt = 0; nt < 4; ++nt) {
            const _Float16* p0 = wb + wrd[nt] + (16 * s) * kTileN;
            const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((FA_LDS short4v*)(p0));
            const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((FA_LDS short4v*)(p0 + 4 * kTileN));
            const short8v both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            wop[SET][nt] = __builtin_bit_cast(half8, both);
        }
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
            xop[SET][mt] = *reinterpret_cast<const half8*>(xb + xrd[s] + mt * 32 * CPRX * 8);
    };
    auto multiply = [&](auto set_c) __attribute__((always_inline)) {
        constexpr int SET = decltype(set_c)::value;
#pragma unroll
        for (int nt = 0; nt < 4; ++nt)
#pragma unroll
            for (int mt = 0; mt < 2; ++mt) {
                if constexpr (BF)
                    acc[nt][mt] = bf16::mfma32(wop[SET][nt], xop[SET][mt], acc[nt][mt]);
                else
                    acc[nt][mt] = mfma32(wop[SET][nt], xop[SET][mt], acc[nt][mt]);
            }
    };
    using set0 = std::integral_constant<int, 0>;
    using set1 = std::integral_constant<int, 1>;

    // Step u reads slot u % 2 while the loads of step u + 1 fill the other one.  One barrier per
    // step, placed before the matrix instructions of the step's last sub-step: by then every wave
    // has the operands of that sub-step in registers, so the slot is free for the loads of step
    // u + 2, and the data of step u + 1 (each wave has waited for its own part) are visible to
    // everybody, so the operands of its first sub-step are requested before the last matrix
    // instructions of step u are issued.  The matrix pipe never waits for LDS at a step boundary.
    static_assert(NSLOT == 2, "the waits below assume that only the next step's loads are in flight");
    aim();
    issue(0);
    if (total_steps > 1) {
        issue(1);
        wait_loads<LX + LW>();      // loads complete in order: all but the second step's have landed
    } else {
        wait_loads<0>();
    }
    ring_barrier();
    load_ops(set0{}, 0, 0);

    bool pending = false;      // the second part of the loads into the previous step's slot is still to be issued
    auto step = [&](int u, auto slot_c) __attribute__((always_inline)) {
        constexpr int SLOT = decltype(slot_c)::value;
        constexpr int PREV = (SLOT + NSLOT - 1) % NSLOT;
        // NSUB is even: sub-step s uses register set s % 2, the next step starts with set 0 again
        auto substep = [&](auto s_c) __attribute__((always_inline)) {
            constexpr int S = decltype(s_c)::value;
            load_ops(std::integral_constant<int, (S + 1) & 1>{}, SLOT, S + 1);
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (S + 1 < NP) {
                if (pending) issue_part(PREV, std::integral_constant<int, S + 1>{});
            }
            multiply(std::integral_constant<int, S & 1>{});
            __builtin_amdgcn_sched_barrier(0);
        };
        static_assert(NSUB == 4, "three sub-steps before the barrier, one behind it");
        substep(std::integral_constant<int, 0>{});
        substep(std::integral_constant<int, 1>{});
        substep(std::integral_constant<int, 2>{});
        // this wave's loads of step u + 1 have landed (the stores of an epilogue are waited for
        // with them), its reads of this step's slot have all returned
        wait_loads<0>();
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        ring_barrier();
        pending = u + NSLOT < total_steps;
        if (pending) issue_part(SLOT, std::integral_constant<int, 0>{});
        // (at the end of a tile the operands of the next step are requested behind the epilogue, which
        // needs the registers)
        const bool last = kt + 1 == ksteps;
        if (u + 1 < total_steps && !last) load_ops(set0{}, (SLOT + 1) % NSLOT, 0);
        __builtin_amdgcn_sched_barrier(0);
        multiply(set1{});
        __builtin_amdgcn_sched_barrier(0);
        if (last) {
            finish_tile(tile);
            kt = 0;
            tile += p.total_wgs;
            __builtin_amdgcn_sched_barrier(0);
            if (u + 1 < total_steps) load_ops(set0{}, (SLOT + 1) % NSLOT, 0);
        } else {
            ++kt;
        }
    };
    for (int u = 0; u < total_steps; u += NSLOT) {
        step(u, std::integral_constant<int, 0>{});
        if (u + 1 < total_steps) step(u + 1, std::integral_constant<int, 1>{});
    }
}

}  // namespace qkv
}  // namespace fa
