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
// the contraction in steps of 64.  x and w tiles stream through a two-stage LDS ring written by
// direct-to-LDS loads (16 bytes per lane, no staging registers), laid out column-major in 16-byte
// chunks like the K/V rings of the attention kernel (kColStride).  The products are computed
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
// one 64-row x 16-byte block of a ring tile, in halves (1 KB plus the pad of the attention rings)
constexpr int kBlk = kColStride;
constexpr int kXTile = (kTileK / 8) * (kTileM / 64) * kBlk;   // chunk c, row block rb at (c * 4 + rb) * kBlk
constexpr int kWTile = (kTileN / 8) * kBlk;                   // feature chunk cn at cn * kBlk, 64 k rows each
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
    int total_wgs;           // tiles_m * tiles_n
    int wgs_per_xcd;
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

    // Workgroups are dealt round-robin to the XCDs: renumber so that one XCD receives consecutive
    // tiles, which share their rows of x (the feature tiles of one row tile follow each other).
    const int wg = blockIdx.x;
    const int logical = (wg % kNumXcd) * p.wgs_per_xcd + wg / kNumXcd;
    if (logical >= p.total_wgs) return;
    const int m0 = (logical / p.tiles_n) * kTileM;
    const int n0 = (logical % p.tiles_n) * kTileN;

    // ---- loads: every wave fetches four x blocks and four w blocks of a stage -------------------
    // x block (c, rb): lane l = row m0 + rb 64 + l, 16 bytes at k chunk c.  Rows beyond M are read
    // from row M - 1 (their results are never stored).  w block cn: lane l = contraction row
    // k0 + l, 16 bytes at feature chunk cn; chunks beyond N are not fetched (their LDS block then
    // holds stale data that only reaches output features which are never stored).
    uint32_t xoff[4], woff[4];
    uint32_t xlds[4], wlds[4];
    bool wvalid[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int blk = wave * 4 + i;               // 0..31
        const int c = blk >> 2, rb = blk & 3;
        const int row = min(m0 + rb * 64 + lane, p.M - 1) - m0;
        xoff[i] = ((uint32_t)row * (uint32_t)p.K + (uint32_t)c * 8u) * 2u;
        xlds[i] = (uint32_t)(c * 4 + rb) * (kBlk * 2);
        const int cn = blk;
        woff[i] = ((uint32_t)lane * (uint32_t)p.N + (uint32_t)cn * 8u) * 2u;
        wlds[i] = (uint32_t)cn * (kBlk * 2);
        wvalid[i] = n0 + cn * 8 < p.N;
    }
    const _Float16* xsrc = p.x + (int64_t)m0 * p.K;                 // k0 = 0
    const _Float16* wsrc = p.w + n0;
    const uint32_t xs_addr = (uint32_t)(uintptr_t)(FA_LDS void*)xs;
    const uint32_t ws_addr = (uint32_t)(uintptr_t)(FA_LDS void*)ws;
    auto issue = [&](int stage) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            RingLoader<64, 4>::dma16(xs_addr + stage * (kXTile * 2) + xlds[i], xsrc, xoff[i]);
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (wvalid[i]) RingLoader<64, 4>::dma16(ws_addr + stage * (kWTile * 2) + wlds[i], wsrc, woff[i]);
    };

    floatx16 acc[4][2];
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[nt][mt][r] = 0.f;

    // per-lane parts of the operand addresses
    // B operand (x): row wm 64 + mt 32 + ln of chunk 2 s + g
    const int xrow = wm * 64 + ln;
    const _Float16* const xop_base = xs + (g * 4 + (xrow >> 6)) * kBlk + (xrow & 63) * 8;
    // A operand (w^T), transpose read: lane s16 of a 16-lane group points at contraction row
    // 8 g + s16 / 4 (+ 4 for the second read), halves 4 (s16 % 4) ... of the 32-byte span of features
    // that starts at chunk 2 * ((lane / 16) % 2); feature block nt adds 4 chunks.  Lane j of the
    // group receives four consecutive contraction rows of feature j: slot (g, i) of the operand is
    // contraction index 16 s + 8 g + i, the order in which the 16-byte read of x delivers them.
    const int s16 = lane & 15;
    const _Float16* const wop_base = ws + (wn * 16 + 2 * ((lane >> 4) & 1) + ((s16 & 3) >> 1)) * kBlk +
                                     (8 * g + (s16 >> 2)) * 8 + 4 * (s16 & 1);

    const int ksteps = p.K / kTileK;
    issue(0);
    wait_ring_loads();
    __syncthreads();
    for (int kt = 0; kt < ksteps; ++kt) {
        const int stage = kt & 1;
        if (kt + 1 < ksteps) {
            xsrc += kTileK;
            wsrc += (int64_t)kTileK * p.N;
            issue(stage ^ 1);
        }
        const _Float16* const xb = xop_base + stage * kXTile;
        const _Float16* const wb = wop_base + stage * kWTile;
#pragma unroll
        for (int s = 0; s < kTileK / 16; ++s) {
            half8 wop[4], xop[2];
#pragma unroll
            for (int nt = 0; nt < 4; ++nt) {
                const _Float16* p0 = wb + nt * 4 * kBlk + (16 * s) * 8;
                const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((FA_LDS short4v*)(p0));
                const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((FA_LDS short4v*)(p0 + 4 * 8));
                const short8v both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                wop[nt] = __builtin_bit_cast(half8, both);
            }
#pragma unroll
            for (int mt = 0; mt < 2; ++mt)
                xop[mt] = *reinterpret_cast<const half8*>(xb + (2 * s) * 4 * kBlk + mt * 32 * 8);
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
        // this wave's loads of the next stage have landed; after the barrier everybody's have, and
        // everybody is done reading the stage that the loads after next will overwrite
        wait_ring_loads();
        __syncthreads();
    }

    // ---- epilogue: bias, rotation, one rounding, 8-byte stores ------------------------------------
    // acc[nt][mt][r]: row m = m0 + wm 64 + mt 32 + ln, feature n = n0 + wn 128 + nt 32 + 8 (r / 4) + 4 g + r % 4
    const int nw = n0 + wn * 128;
#pragma unroll
    for (int mt = 0; mt < 2; ++mt) {
        const int m = m0 + wm * 64 + mt * 32 + ln;
        if (p.bias != nullptr) {
#pragma unroll
            for (int nt = 0; nt < 4; ++nt)
#pragma unroll
                for (int r4 = 0; r4 < 4; ++r4) {
                    const int n = nw + nt * 32 + 8 * r4 + 4 * g;
                    if (n < p.N) {
                        const u16x4 b4 = *reinterpret_cast<const u16x4*>(p.bias + n);
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            acc[nt][mt][4 * r4 + e] += BF ? bf16::elem_to_float(b4[e]) : elem_to_float(b4[e]);
                    }
                }
        }
        if constexpr (HR > 0) {
            // rotate-half: within a head, feature i < HR / 2 pairs with feature i + HR / 2:
            //   out[i] = x[i] cos_i - x[i + HR/2] sin_i,  out[i + HR/2] = x[i + HR/2] cos_i + x[i] sin_i
            // with cos_i, sin_i taken at the row's position m % L.  Only the q and k slices (n < 2 F).
            const int pos = (m < p.M ? m : p.M - 1) % p.L;
            const float* const cs = p.rope_cos + (int64_t)pos * (HR / 2);
            const float* const sn = p.rope_sin + (int64_t)pos * (HR / 2);
            // (block, register group) of the first half and of its partner, by head_dim
            constexpr int NPAIR = 8;   // the 16 runs of four features a lane holds per row form 8 pairs
#pragma unroll
            for (int pr = 0; pr < NPAIR; ++pr) {
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
                const int n_a = nw + nt_a * 32 + 8 * r4_a + 4 * g;      // first feature of the run in the first half
                if (n_a < 2 * p.F) {
                    const int i0 = n_a % (HR / 2);      // index inside the half head
                    const floatx4 c4 = *reinterpret_cast<const floatx4*>(cs + i0);
                    const floatx4 s4 = *reinterpret_cast<const floatx4*>(sn + i0);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float a = acc[nt_a][mt][4 * r4_a + e];
                        const float b = acc[nt_b][mt][4 * r4_b + e];
                        acc[nt_a][mt][4 * r4_a + e] = a * c4[e] - b * s4[e];
                        acc[nt_b][mt][4 * r4_b + e] = b * c4[e] + a * s4[e];
                    }
                }
            }
        }
        if (m < p.M) {
            _Float16* const orow = p.out + (int64_t)m * p.N;
#pragma unroll
            for (int nt = 0; nt < 4; ++nt)
#pragma unroll
                for (int r4 = 0; r4 < 4; ++r4) {
                    const int n = nw + nt * 32 + 8 * r4 + 4 * g;
                    if (n < p.N) {
                        u16x4 hv;
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            hv[e] = BF ? bf16::float_to_elem(acc[nt][mt][4 * r4 + e]) : float_to_elem(acc[nt][mt][4 * r4 + e]);
                        *reinterpret_cast<u32x2*>(orow + n) = __builtin_bit_cast(u32x2, hv);
                    }
                }
        }
    }
}

}  // namespace qkv
}  // namespace fa
