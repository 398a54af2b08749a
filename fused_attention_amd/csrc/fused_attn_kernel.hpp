// Fused multi-head attention forward for gfx950 (MI355X, CDNA4).
//
// One kernel computes O = softmax(Q K^T * scale) V per (batch, head) without ever
// writing the L x L score matrix to memory.  It replaces, as a single pass, the
// reference's attention_kernel and every threadblock_* helper it calls
// (reference include/fused_attn.cuh:48-538 and :605-858).
//
// Work decomposition
//   workgroup  = NW wave64s, each wave owns 64 query rows (two 32-row blocks)
//   K/V        = streamed in BK-key tiles, global -> registers -> LDS, double buffered
//   per 32 keys: S^T = K_sub * Q^T        v_mfma_f32_32x32x16_f16, Q held in registers
//                online softmax on S^T     f32, state (m, l) per lane
//                O^T += V_sub^T * P^T      same MFMA, V^T fetched with ds_read_b64_tr_b16
//
// Why the transposed products: in the 32x32 accumulator layout lane l owns column
// (l % 32) -- one query -- and 16 of the 32 rows (keys); lane l^32 owns the other 16.
// A softmax row therefore lives in one lane pair, so row max / row sum need 15 in-lane
// ops and a single v_permlane32_swap.  The f16-packed P^T registers are, as they stand,
// a valid B operand of the second product provided the A operand (V^T) enumerates keys
// in the same order, which the transpose-read from a row-major V tile provides.
//
// MFMA operand maps used below (g = lane / 32, ln = lane % 32):
//   A (32 x 16): lane holds row ln,   k = 8 g + i          (i = 0..7)
//   B (16 x 32): lane holds col ln,   k = 8 g + i
//   C (32 x 32): lane holds col ln,   row = 8 (r / 4) + 4 g + r % 4   (r = 0..15)
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fa {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

#define FA_LDS __attribute__((address_space(3)))

struct FwdParams {
    const _Float16* q;
    const _Float16* k;
    const _Float16* v;
    const _Float16* mask;  // additive [B, L, L] or nullptr
    _Float16* o;
    int64_t stride_b;      // elements between batches
    int64_t stride_h;      // elements between heads
    int64_t stride_l;      // elements between sequence positions
    int B, R, L;
    int n_qtiles;          // ceil(L / queries per workgroup)
    int total_wgs;         // B * R * n_qtiles
    int wgs_per_xcd;       // ceil(total_wgs / 8)
    float scale_log2e;     // scale * log2(e)
};

constexpr int kNumXcd = 8;

template <int H>
struct Geometry {
    static constexpr int KS = H / 16;                    // k-steps of the QK^T product
    static constexpr int HV = H < 32 ? 32 : H;           // V columns held in LDS (zero padded)
    static constexpr int DB = HV / 32;                   // 32-row blocks of O^T
    // Row strides (in f16) chosen so that the 16 rows touched by one quarter-wave of a
    // ds_read_b128 (K) and the 4 rows touched by a 16-lane transpose read (V) fall into
    // disjoint LDS banks.
    static constexpr int KSTR = H + 8;
    static constexpr int VSTR = HV == 32 ? 32 : HV + 32;
};

template <int H, int NW, int BK>
constexpr int lds_bytes() {
    using G = Geometry<H>;
    return 2 * BK * (G::KSTR + G::VSTR) * (int)sizeof(_Float16);
}

// NaN-propagating maximum: lowers to v_maximum3_f32 without the input canonicalisation that
// fmaxf needs in IEEE mode.
__device__ __forceinline__ float fmax2(float a, float b) { return __builtin_elementwise_maximum(a, b); }

// Exchanges a value between lanes l and l^32.  v_permlane32_swap(a, b) leaves, in lanes < 32,
// (a[l], a[l + 32]) and, in lanes >= 32, (b[l - 32], b[l]); with a = b = x every lane holds its own
// value and its partner's.  The two results are copied to scalars before the bit cast: applying
// __builtin_bit_cast directly to a vector element reads element 0 for both.
__device__ __forceinline__ float pair_max(float x) {
    const uint32_t xb = __builtin_bit_cast(uint32_t, x);
    const u32x2 r = __builtin_amdgcn_permlane32_swap(xb, xb, false, false);
    const uint32_t r0 = r[0], r1 = r[1];
    return fmax2(__builtin_bit_cast(float, r0), __builtin_bit_cast(float, r1));
}

__device__ __forceinline__ float pair_sum(float x) {
    const uint32_t xb = __builtin_bit_cast(uint32_t, x);
    const u32x2 r = __builtin_amdgcn_permlane32_swap(xb, xb, false, false);
    const uint32_t r0 = r[0], r1 = r[1];
    return __builtin_bit_cast(float, r0) + __builtin_bit_cast(float, r1);
}

__device__ __forceinline__ uint32_t pack_rtz(float a, float b) {
    return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(a, b));
}

// Streams one K/V tile from global memory into registers, and from registers into LDS.
template <int H, int NW, int BK>
struct TileLoader {
    using G = Geometry<H>;
    static constexpr int CPR = H / 8;                       // 16-byte chunks per row
    static constexpr int NCHUNK = BK * CPR;
    static constexpr int NT = NW * 64;
    static constexpr int NP = (NCHUNK + NT - 1) / NT;       // chunks per thread
    u32x4 kreg[NP];
    u32x4 vreg[NP];

    __device__ __forceinline__ void load(const _Float16* kbase, const _Float16* vbase,
                                         int64_t stride_l, int key0, int L, int tid) {
#pragma unroll
        for (int i = 0; i < NP; ++i) {
            const int idx = tid + i * NT;
            const int row = idx / CPR;
            const int chunk = idx % CPR;
            const int key = key0 + row;
            u32x4 kk = {0u, 0u, 0u, 0u};
            u32x4 vv = {0u, 0u, 0u, 0u};
            if ((NCHUNK % NT == 0 || idx < NCHUNK) && key < L) {
                const int64_t off = (int64_t)key * stride_l + chunk * 8;
                kk = *reinterpret_cast<const u32x4*>(kbase + off);
                vv = *reinterpret_cast<const u32x4*>(vbase + off);
            }
            kreg[i] = kk;
            vreg[i] = vv;
        }
    }

    __device__ __forceinline__ void store(_Float16* ks, _Float16* vs, int tid) const {
#pragma unroll
        for (int i = 0; i < NP; ++i) {
            const int idx = tid + i * NT;
            const int row = idx / CPR;
            const int chunk = idx % CPR;
            if (NCHUNK % NT == 0 || idx < NCHUNK) {
                *reinterpret_cast<u32x4*>(ks + row * G::KSTR + chunk * 8) = kreg[i];
                *reinterpret_cast<u32x4*>(vs + row * G::VSTR + chunk * 8) = vreg[i];
            }
        }
    }
};

// Largest partial row sum (16 terms) the fast path of the online softmax accepts.
constexpr float kTrip = 16384.f;

// p = exp2(s * c + mc) for the 2 x 16 scores of a sub-tile, rounded to fp16 pairs (round toward
// zero), and the per-lane sums of the rounded values.  The sums are taken over the rounded
// probabilities that enter the second product, so numerator and denominator see the same rounding.
__device__ __forceinline__ void exp_pack_sum(const floatx16 (&s)[2], float c, const float (&mc)[2],
                                             uint32_t (&pk)[2][8], float (&ts)[2]) {
    const half2v ones = {(_Float16)1.0f, (_Float16)1.0f};
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
        float acc = 0.f;
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
            const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[nb][r], c, mc[nb]));
            const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[nb][r + 1], c, mc[nb]));
            const uint32_t pp = pack_rtz(p0, p1);
            pk[nb][r >> 1] = pp;
            acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, pp), ones, acc, false);
        }
        ts[nb] = acc;
    }
}

// O^T[.][nb] *= alpha, in place.  Written as one instruction per register with the register tied
// as input and output, so that the rarely taken rescale does not make the compiler keep a second
// copy of the accumulators (and copy them on the common path).  The leading wait covers the
// matrix-core results the multiplies read.
template <int DB>
__device__ __forceinline__ void scale_accumulators(floatx16 (&o)[DB][2], int nb, float alpha) {
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#pragma unroll
    for (int db = 0; db < DB; ++db) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            float e = o[db][nb][r];
            asm volatile("v_mul_f32 %0, %1, %0" : "+v"(e) : "v"(alpha));
            o[db][nb][r] = e;
        }
    }
}

// Per-wave state: Q^T as B operands, O^T accumulators, online-softmax (m, l).
template <int H>
struct WaveState {
    using G = Geometry<H>;
    half8 q[2][G::KS];
    floatx16 o[G::DB][2];
    float m[2];   // reference row maximum of the raw (unscaled) scores, identical in lanes l and l^32
    float mc[2];  // -m * c, the additive term of the exponent; +inf while no reference exists yet
    float l[2];   // running sum of exp over the keys this lane has seen (half of each tile)
};

// Processes 32 keys (one sub-tile) for the wave's 64 queries.
//   ks/vs : LDS tile base for the current buffer
//   sub   : sub-tile index inside the tile
//   nvalid: number of valid keys in this sub-tile (only read when MASKED)
template <int H, bool MASKED, bool HAS_MASK>
__device__ __forceinline__ void process_subtile(WaveState<H>& st, const _Float16* ks,
                                                const _Float16* vs, int sub, int nvalid,
                                                float c, int lane,
                                                const _Float16* mask_row0, const _Float16* mask_row1,
                                                int key_base, int L) {
    using G = Geometry<H>;
    const int g = lane >> 5;
    const int ln = lane & 31;

    // ---- S^T = K_sub * Q^T -------------------------------------------------------------
    floatx16 s[2];
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
        for (int r = 0; r < 16; ++r) s[nb][r] = 0.f;

    const _Float16* krow = ks + (sub * 32 + ln) * G::KSTR + 8 * g;
#pragma unroll
    for (int kk = 0; kk < G::KS; ++kk) {
        const half8 a = *reinterpret_cast<const half8*>(krow + kk * 16);
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
            s[nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, st.q[nb][kk], s[nb], 0, 0, 0);
    }

    // ---- optional additive mask (log2 domain is applied later, so pre-divide by c) -------
    if constexpr (HAS_MASK) {
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
            const _Float16* mrow = nb == 0 ? mask_row0 : mask_row1;
            if (mrow != nullptr) {
#pragma unroll
                for (int r4 = 0; r4 < 4; ++r4) {
                    const int key = key_base + 8 * r4 + 4 * g;
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        if (key + j < L) {
                            // The mask is added to the scaled score; S holds raw scores, so the
                            // mask is brought to raw units: (s*scale + mask) = scale*(s + mask/scale).
                            s[nb][4 * r4 + j] += (float)mrow[key + j] * (1.4426950408889634f / c);
                        }
                    }
                }
            }
        }
    }

    // ---- tail masking --------------------------------------------------------------------
    if constexpr (MASKED) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int key = 8 * (r >> 2) + 4 * g + (r & 3);
            if (key >= nvalid) {
                s[0][r] = -__builtin_inff();
                s[1][r] = -__builtin_inff();
            }
        }
    }

    // ---- online softmax ------------------------------------------------------------------
    // Fast path: exponentiate against the reference maximum of the rows seen so far, without
    // looking at this sub-tile's maximum.  Any reference works as long as numerator and
    // denominator share it; it only has to keep exp2 inside the fp16 range.  Each lane checks
    // that with its own partial row sum: 16 non-negative terms whose sum is <= kTrip are each
    // <= kTrip, and anything that overflowed (inf) or was computed from an undefined reference
    // (NaN) fails the comparison.  Only then the wave takes the slow path, which brings the
    // reference up to the true running maximum and rescales O and l.
    uint32_t pk[2][8];
    float ts[2];
    exp_pack_sum(s, c, st.mc, pk, ts);
    const bool ok = (ts[0] <= kTrip) & (ts[1] <= kTrip);
    if (__builtin_expect(__builtin_amdgcn_ballot_w64(!ok) != 0, 0)) {
        float mcu[2];
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
            float mx = fmax2(s[nb][0], s[nb][1]);
#pragma unroll
            for (int r = 2; r < 16; r += 2) mx = fmax2(mx, fmax2(s[nb][r], s[nb][r + 1]));
            mx = pair_max(mx);
            const float m_old = st.m[nb];
            const float m_new = fmax2(m_old, mx);
            // m_new == -inf: every key so far carried a -inf additive mask.  Nothing has been
            // accumulated yet, this sub-tile contributes zeros, and the stored reference stays
            // undefined (+inf) so that the next sub-tile comes back here.
            const bool empty = m_new == -__builtin_inff();
            const float alpha = empty ? 1.f : __builtin_amdgcn_exp2f((m_old - m_new) * c);
            st.l[nb] *= alpha;
            scale_accumulators<G::DB>(st.o, nb, alpha);
            st.m[nb] = m_new;
            st.mc[nb] = empty ? __builtin_inff() : -m_new * c;
            mcu[nb] = empty ? 0.f : -m_new * c;
        }
        exp_pack_sum(s, c, mcu, pk, ts);
    }
    st.l[0] += ts[0];
    st.l[1] += ts[1];

    // ---- O^T += V_sub^T * P^T ------------------------------------------------------------
    // Transpose read: inside each group of 16 lanes, lane j receives, for i = 0..3, element
    // (j % 4) of the 8-byte row fetched by lane 4 i + j / 4.  With lane s of a group pointing at
    // V[key0 + s / 4][d0 + 4 (s % 4) ...], lane j ends up with V[key0 + i][d0 + j], i = 0..3.
    const int s16 = lane & 15;
    const _Float16* vrow = vs + (sub * 32 + 4 * g + (s16 >> 2)) * G::VSTR + 16 * ((lane >> 4) & 1) +
                           4 * (s16 & 3);
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        half8 pb[2];
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
            u32x4 w = {pk[nb][4 * t], pk[nb][4 * t + 1], pk[nb][4 * t + 2], pk[nb][4 * t + 3]};
            pb[nb] = __builtin_bit_cast(half8, w);
        }
#pragma unroll
        for (int db = 0; db < G::DB; ++db) {
            const _Float16* p0 = vrow + (16 * t) * G::VSTR + db * 32;
            const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((FA_LDS short4v*)(p0));
            const short4v hi =
                __builtin_amdgcn_ds_read_tr16_b64_v4i16((FA_LDS short4v*)(p0 + 8 * G::VSTR));
            typedef short short8v __attribute__((ext_vector_type(8)));
            const short8v both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            const half8 a = __builtin_bit_cast(half8, both);
#pragma unroll
            for (int nb = 0; nb < 2; ++nb)
                st.o[db][nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, pb[nb], st.o[db][nb], 0, 0, 0);
        }
    }
}

template <int H, int NW, int BK, bool HAS_MASK>
__global__ __launch_bounds__(NW * 64, (H <= 64 ? 2 : 1)) void fwd_kernel(const FwdParams p) {
    using G = Geometry<H>;
    constexpr int BQ = NW * 64;
    constexpr int NSUB = BK / 32;

    extern __shared__ __attribute__((aligned(16))) _Float16 smem[];
    _Float16* const ks_base = smem;                                // [2][BK][KSTR]
    _Float16* const vs_base = smem + 2 * BK * G::KSTR;             // [2][BK][VSTR]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = lane >> 5;
    const int ln = lane & 31;

    // Workgroups are dealt round-robin to the 8 XCDs; renumber so that one XCD (one L2)
    // receives a contiguous run of tiles, i.e. all query tiles of a (batch, head) share K/V in L2.
    const int wg = blockIdx.x;
    const int logical = (wg % kNumXcd) * p.wgs_per_xcd + wg / kNumXcd;
    if (logical >= p.total_wgs) return;
    const int bh = logical / p.n_qtiles;
    const int qt = logical % p.n_qtiles;
    const int b = bh / p.R;
    const int h = bh % p.R;
    const int L = p.L;

    const int64_t head_off = (int64_t)b * p.stride_b + (int64_t)h * p.stride_h;
    const _Float16* qbase = p.q + head_off;
    const _Float16* kbase = p.k + head_off;
    const _Float16* vbase = p.v + head_off;
    _Float16* obase = p.o + head_off;
    const int q0 = qt * BQ + wave * 64;

    // V columns beyond H (only when H = 16) stay zero for the whole kernel.
    if constexpr (G::HV != H) {
        for (int i = tid; i < 2 * BK * G::VSTR; i += BQ) vs_base[i] = (_Float16)0.f;
        __syncthreads();
    }

    WaveState<H> st;
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
        const int row = q0 + nb * 32 + ln;
#pragma unroll
        for (int kk = 0; kk < G::KS; ++kk) {
            u32x4 w = {0u, 0u, 0u, 0u};
            if (row < L)
                w = *reinterpret_cast<const u32x4*>(qbase + (int64_t)row * p.stride_l + kk * 16 + 8 * g);
            st.q[nb][kk] = __builtin_bit_cast(half8, w);
        }
        st.m[nb] = -__builtin_inff();
        st.mc[nb] = __builtin_inff();
        st.l[nb] = 0.f;
#pragma unroll
        for (int db = 0; db < G::DB; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) st.o[db][nb][r] = 0.f;
    }

    const _Float16* mask_row0 = nullptr;
    const _Float16* mask_row1 = nullptr;
    if constexpr (HAS_MASK) {
        const _Float16* mb = p.mask + (int64_t)b * L * L;
        if (q0 + ln < L) mask_row0 = mb + (int64_t)(q0 + ln) * L;
        if (q0 + 32 + ln < L) mask_row1 = mb + (int64_t)(q0 + 32 + ln) * L;
    }

    const int ntiles = (L + BK - 1) / BK;
    const float c = p.scale_log2e;

    TileLoader<H, NW, BK> loader;
    loader.load(kbase, vbase, p.stride_l, 0, L, tid);
    loader.store(ks_base, vs_base, tid);
    __syncthreads();

    // Full tiles: one straight path per iteration.  The ragged last tile, if any, is peeled off so
    // that its masking code does not share a loop (and register assignment) with the hot path.
    const int nfull = L / BK;
    for (int t = 0; t < nfull; ++t) {
        const int buf = t & 1;
        const _Float16* ks = ks_base + buf * BK * G::KSTR;
        const _Float16* vs = vs_base + buf * BK * G::VSTR;
        const bool has_next = t + 1 < ntiles;
        if (has_next) loader.load(kbase, vbase, p.stride_l, (t + 1) * BK, L, tid);
#pragma unroll
        for (int sub = 0; sub < NSUB; ++sub)
            process_subtile<H, false, HAS_MASK>(st, ks, vs, sub, 32, c, lane, mask_row0, mask_row1,
                                                t * BK + sub * 32, L);
        if (has_next) loader.store(ks_base + (buf ^ 1) * BK * G::KSTR, vs_base + (buf ^ 1) * BK * G::VSTR, tid);
        __syncthreads();
    }
    if (nfull < ntiles) {
        const int buf = nfull & 1;
        const _Float16* ks = ks_base + buf * BK * G::KSTR;
        const _Float16* vs = vs_base + buf * BK * G::VSTR;
        const int key0 = nfull * BK;
#pragma unroll
        for (int sub = 0; sub < NSUB; ++sub) {
            const int nvalid = L - key0 - sub * 32;
            if (nvalid > 0)
                process_subtile<H, true, HAS_MASK>(st, ks, vs, sub, nvalid, c, lane, mask_row0, mask_row1,
                                                   key0 + sub * 32, L);
        }
    }

    // ---- epilogue: O = O^T / l, f16, 8-byte stores ------------------------------------------
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
        const float lt = pair_sum(st.l[nb]);
        // A row whose every key carried a -inf mask has l = 0: emit zeros rather than NaN.
        const float inv = lt > 0.f ? 1.0f / lt : 0.f;
        const int row = q0 + nb * 32 + ln;
        if (row < L) {
            _Float16* orow = obase + (int64_t)row * p.stride_l;
#pragma unroll
            for (int db = 0; db < G::DB; ++db) {
#pragma unroll
                for (int r4 = 0; r4 < 4; ++r4) {
                    const int d = db * 32 + 8 * r4 + 4 * g;
                    if (G::HV == H || d < H) {
                        half4 hv;
#pragma unroll
                        for (int j = 0; j < 4; ++j) hv[j] = (_Float16)(st.o[db][nb][4 * r4 + j] * inv);
                        *reinterpret_cast<u32x2*>(orow + d) = __builtin_bit_cast(u32x2, hv);
                    }
                }
            }
        }
    }
}

}  // namespace fa
