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
// the contraction in steps of 64.  x and w tiles go global -> registers -> LDS with 16-byte
// accesses, whole cache lines per wave on the global side, into two LDS stages of row-major tiles
// with padded rows (the loads of the next step are in flight while this one is consumed).  The
// products are computed
// transposed, C^T = W^T X^T, with v_mfma_f32_32x32x16_f16: the A operand W^T (32 outputs n x 16 k)
// comes from the row-major w tile through the LDS transpose read (ds_read_b64_tr_b16), the B
// operand X^T (16 k x 32 rows m) is a plain 16-byte read of a row of x.  In the accumulator a lane
// then owns one output row m and, per 32 x 32 block, 16 output features n in runs of four: bias
// and rotation are applied in registers (the partner feature n + H/2 of a rotation sits in the
// same lane), and a run is stored with one 8-byte store.
//
// A wave owns 64 rows x 128 features (4 x 2 blocks of 32 x 32, 128 accumulator registers); its
// 128 features are whole heads for every head_dim up to 128.
#pragma once

#include "fused_attn_kernel.hpp"

namespace fa {
namespace qkv {

constexpr int kTileM = 256;
constexpr int kTileN = 256;
constexpr int kTileK = 64;
constexpr int kWaves = 8;
constexpr int kBand = 4;      // row tiles per band of the tile order
// LDS tiles are row-major with padded rows, so that the 16-byte operand reads of x (32 consecutive
// rows per half-wave) and the transpose reads of w (four contraction rows x 32 bytes per 16 lanes)
// touch every bank once: 144-byte rows of x put 16 consecutive rows on distinct 16-byte bank
// groups, 576-byte rows of w put four consecutive rows 16 banks apart.
constexpr int kXStr = kTileK + 8;                   // halves per row of the x tile [256][64]
constexpr int kWStr = kTileN + 32;                  // halves per row of the w tile [64][256]
constexpr int kXTile = kTileM * kXStr;
constexpr int kWTile = kTileK * kWStr;
constexpr int kLdsBytes = 2 * (kXTile + kWTile) * (int)sizeof(_Float16);

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

// HR = head_dim of the rotation (16, 32, 64, 128), or 0 for none.
template <int HR, bool BF>
__global__ __launch_bounds__(kWaves * 64, 2) void qkv_proj_kernel(const Params p) {
    extern __shared__ __attribute__((aligned(16))) _Float16 smem[];
    _Float16* const xs = smem;                   // two x tiles
    _Float16* const ws = smem + 2 * kXTile;      // two w tiles
    typedef short short8v __attribute__((ext_vector_type(8)));

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = lane >> 5;
    const int ln = lane & 31;
    const int wm = wave >> 1;          // which 64 rows of the tile
    const int wn = wave & 1;           // which 128 features of the tile

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

    // ---- loads: global -> registers -> LDS, 16 bytes per lane ------------------------------------
    // x tile: chunk idx = tid + 512 i is row idx / 8, 16-byte chunk idx % 8: eight lanes read the 128
    // bytes of one row, a wave reads eight whole cache lines per instruction.  Rows beyond M are
    // read from row M - 1 (their results are never stored).  w tile: chunk idx is contraction row
    // idx / 32, feature chunk idx % 32: 32 lanes read 512 contiguous bytes of a row; chunks beyond N
    // are not fetched and hold zeros.
    // The loads run ahead of the arithmetic as one stream over all (tile, contraction step) pairs of
    // the workgroup: the first steps of the next tile are on their way while this one is finished.
    constexpr int NP = 4;      // chunks per thread and tile, of x and of w
    uint32_t xoff[NP], woff[NP], xdst[NP], wdst[NP];
    bool wvalid[NP];
    const char* xsrc = nullptr;
    const char* wsrc = nullptr;
    int fetch_tile = logical, fetch_kt = 0;
    auto aim = [&]() __attribute__((always_inline)) {      // point the loads at the first step of fetch_tile
        int m0, n0;
        tile_origin(fetch_tile, m0, n0);
#pragma unroll
        for (int i = 0; i < NP; ++i) {
            const int idx = tid + i * (kWaves * 64);
            const int row = min(m0 + (idx >> 3), p.M - 1) - m0;
            xoff[i] = ((uint32_t)row * (uint32_t)p.K + (uint32_t)(idx & 7) * 8u) * 2u;
            wvalid[i] = n0 + (idx & 31) * 8 < p.N;
        }
        xsrc = reinterpret_cast<const char*>(p.x + (int64_t)m0 * p.K);
        wsrc = reinterpret_cast<const char*>(p.w + n0);
    };
#pragma unroll
    for (int i = 0; i < NP; ++i) {
        const int idx = tid + i * (kWaves * 64);
        xdst[i] = (uint32_t)((idx >> 3) * kXStr + (idx & 7) * 8);
        woff[i] = ((uint32_t)(idx >> 5) * (uint32_t)p.N + (uint32_t)(idx & 31) * 8u) * 2u;
        wdst[i] = (uint32_t)((idx >> 5) * kWStr + (idx & 31) * 8);
    }
    aim();
    const int ksteps = p.K / kTileK;
    // two sets of staging registers: a step's data is fetched two steps before it is consumed
    u32x4 xreg[2][NP], wreg[2][NP];
    auto fetch = [&](auto set_c) __attribute__((always_inline)) {
        constexpr int SET = decltype(set_c)::value;
#pragma unroll
        for (int i = 0; i < NP; ++i) xreg[SET][i] = *reinterpret_cast<const u32x4*>(xsrc + xoff[i]);
#pragma unroll
        for (int i = 0; i < NP; ++i) {
            wreg[SET][i] = u32x4{0u, 0u, 0u, 0u};
            if (wvalid[i]) wreg[SET][i] = *reinterpret_cast<const u32x4*>(wsrc + woff[i]);
        }
        xsrc += kTileK * 2;
        wsrc += (int64_t)kTileK * p.N * 2;
        if (++fetch_kt == ksteps) {
            fetch_kt = 0;
            fetch_tile += p.total_wgs;
            if (fetch_tile < p.total_tiles) aim();
        }
    };
    auto stash = [&](auto set_c, int stage) __attribute__((always_inline)) {
        constexpr int SET = decltype(set_c)::value;
#pragma unroll
        for (int i = 0; i < NP; ++i) *reinterpret_cast<u32x4*>(xs + stage * kXTile + xdst[i]) = xreg[SET][i];
#pragma unroll
        for (int i = 0; i < NP; ++i) *reinterpret_cast<u32x4*>(ws + stage * kWTile + wdst[i]) = wreg[SET][i];
    };

    floatx16 acc[4][2];
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[nt][mt][r] = 0.f;

    // per-lane parts of the operand addresses
    // B operand (x): row wm 64 + mt 32 + ln, contraction chunk 2 s + g
    const _Float16* const xop_base = xs + (wm * 64 + ln) * kXStr + 8 * g;
    // A operand (w^T), transpose read: lane s16 of a 16-lane group points at contraction row
    // 8 g + s16 / 4 (+ 4 for the second read), features 4 (s16 % 4) ... of the 16 that start at
    // 16 * ((lane / 16) % 2); feature block nt adds 32.  Lane j of the group receives four
    // consecutive contraction rows of feature j: slot (g, i) of the operand is contraction index
    // 16 s + 8 g + i, the order in which the 16-byte read of x delivers them.
    const int s16 = lane & 15;
    const _Float16* const wop_base = ws + (8 * g + (s16 >> 2)) * kWStr + wn * 128 + 16 * ((lane >> 4) & 1) +
                                     4 * (s16 & 3);

    // ---- end of a tile: bias, rotation, one rounding, 8-byte stores; the accumulators start over ---
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
        auto store_run = [&](floatx4 v, int m, int n) __attribute__((always_inline)) {
            if (m < p.M && n < p.N) {
                u16x4 hv;
#pragma unroll
                for (int e = 0; e < 4; ++e) hv[e] = BF ? bf16::float_to_elem(v[e]) : float_to_elem(v[e]);
                *reinterpret_cast<u32x2*>(p.out + (int64_t)m * p.N + n) = __builtin_bit_cast(u32x2, hv);
            }
        };
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) {
            const int m = m0 + wm * 64 + mt * 32 + ln;
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
                    store_run(a, m, n_a);
                    store_run(b, m, n_b);
                    // one pair at a time: all table loads at once would not fit in the registers
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else {
#pragma unroll
                for (int nt = 0; nt < 4; ++nt)
#pragma unroll
                    for (int r4 = 0; r4 < 4; ++r4) {
                        const int n = nw + nt * 32 + 8 * r4 + 4 * g;
                        store_run(biased(nt, mt, r4, n), m, n);
                    }
            }
        }
#pragma unroll
        for (int nt = 0; nt < 4; ++nt)
#pragma unroll
            for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[nt][mt][r] = 0.f;
    };

    // Two LDS stages, two register sets.  Step t of the workgroup's stream consumes its data from LDS
    // stage t % 2; the loads of step t + 2 are sent off at its start into register set t % 2, and at
    // its end the data of step t + 1 (requested one step earlier) moves from the other set to the
    // other stage, which everybody finished reading before the barrier that ended step t - 1.
    const int my_tiles = (p.total_tiles - logical + p.total_wgs - 1) / p.total_wgs;
    const int total_steps = my_tiles * ksteps;
    int tile = logical, kt = 0;
    auto step = [&](int t, auto par_c) __attribute__((always_inline)) {
        constexpr int PAR = decltype(par_c)::value;
        // (at the last step of a tile the loads are sent off behind the epilogue instead, so that no
        // staging register is live while the epilogue needs registers of its own)
        const bool last = kt + 1 == ksteps;
        if (!last && t + 2 < total_steps) fetch(std::integral_constant<int, PAR>{});
        const _Float16* const xb = xop_base + PAR * kXTile;
        const _Float16* const wb = wop_base + PAR * kWTile;
#pragma unroll
        for (int s = 0; s < kTileK / 16; ++s) {
            half8 wop[4], xop[2];
#pragma unroll
            for (int nt = 0; nt < 4; ++nt) {
                const _Float16* p0 = wb + (16 * s) * kWStr + nt * 32;
                const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((FA_LDS short4v*)(p0));
                const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((FA_LDS short4v*)(p0 + 4 * kWStr));
                const short8v both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                wop[nt] = __builtin_bit_cast(half8, both);
            }
#pragma unroll
            for (int mt = 0; mt < 2; ++mt)
                xop[mt] = *reinterpret_cast<const half8*>(xb + mt * 32 * kXStr + s * 16);
#pragma unroll
            for (int nt = 0; nt < 4; ++nt)
#pragma unroll
                for (int mt = 0; mt < 2; ++mt) {
                    if constexpr (BF)
                        acc[nt][mt] = bf16::mfma32(wop[nt], xop[mt], acc[nt][mt]);
                    else
                        acc[nt][mt] = mfma32(wop[nt], xop[mt], acc[nt][mt]);
                }
        }
        if (t + 1 < total_steps) stash(std::integral_constant<int, 1 - PAR>{}, 1 - PAR);
        __syncthreads();
        if (last) {
            finish_tile(tile);
            kt = 0;
            tile += p.total_wgs;
            if (t + 2 < total_steps) fetch(std::integral_constant<int, PAR>{});
        } else {
            ++kt;
        }
    };
    fetch(std::integral_constant<int, 0>{});
    stash(std::integral_constant<int, 0>{}, 0);
    if (total_steps > 1) fetch(std::integral_constant<int, 1>{});
    __syncthreads();
    for (int t = 0; t < total_steps; t += 2) {
        step(t, std::integral_constant<int, 0>{});
        if (t + 1 < total_steps) step(t + 1, std::integral_constant<int, 1>{});
    }
}

}  // namespace qkv
}  // namespace fa
