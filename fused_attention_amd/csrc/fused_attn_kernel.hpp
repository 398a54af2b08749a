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
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

#define FA_LDS __attribute__((address_space(3)))

struct FwdParams {
    const _Float16* q;
    const _Float16* k;
    const _Float16* v;
    const _Float16* mask;  // additive [B, L, L] or nullptr
    _Float16* o;
    float* lse;            // optional [B, R, L] natural-log row sums of exp(scores), or nullptr
    int64_t stride_b;      // elements between batches
    int64_t stride_h;      // elements between heads
    int64_t stride_l;      // elements between sequence positions
    int B, R, L;
    int n_qtiles;          // workgroups per (batch, head): ceil(L / queries per workgroup), or half of
                           // that (rounded up) when a causal workgroup takes a pair of query tiles
    int total_wgs;         // B * R * n_qtiles
    int wgs_per_xcd;       // ceil(total_wgs / 8)
    float scale_log2e;     // scale * log2(e)
};

constexpr int kNumXcd = 8;

// Kernel variants of the non-ping-pong kernel.
constexpr int kPlain = 0;    // no mask: software-pipelined loop
constexpr int kAdditive = 1; // additive [B, L, L] mask
constexpr int kCausal = 2;   // key index <= query index, key tiles above the diagonal skipped

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

// Streams K/V tiles from global memory into registers, and from registers into LDS.  K and V are
// handled separately because the pipelined loop keeps K one tile ahead of V.
template <int H, int NW, int BK>
struct TileLoader {
    using G = Geometry<H>;
    static constexpr int CPR = H / 8;                       // 16-byte chunks per row
    static constexpr int NCHUNK = BK * CPR;
    static constexpr int NT = NW * 64;
    static constexpr int NP = (NCHUNK + NT - 1) / NT;       // chunks per thread
    static constexpr bool EXACT = NCHUNK % NT == 0;
    u32x4 kreg[NP];
    u32x4 vreg[NP];
    uint32_t goff[NP];   // byte offset of this thread's chunk i from the first key of a tile

    __device__ __forceinline__ void init(int64_t stride_l, int tid) {
#pragma unroll
        for (int i = 0; i < NP; ++i) {
            const int idx = EXACT ? tid + i * NT : min(tid + i * NT, NCHUNK - 1);
            goff[i] = (uint32_t)(((int64_t)(idx / CPR) * stride_l + (idx % CPR) * 8) * 2);
        }
    }

    // A full tile is fetched with one uniform base address plus the per-thread byte offsets (no
    // vector address arithmetic inside the key loop).  In the ragged last tile, rows at or beyond
    // L are read from row L - 1 instead of being predicated off (a predicated load into a zeroed
    // register makes every load wait for the one before it).  Such keys are masked to -inf before
    // the softmax, and a probability of exactly zero times a finite V row contributes nothing.
    __device__ __forceinline__ void load(u32x4 (&reg)[NP], const _Float16* base, int64_t stride_l,
                                         int key0, int L, int tid) const {
        if (key0 >= L) return;
        if (key0 + BK <= L) {
            const char* tile = reinterpret_cast<const char*>(base + (int64_t)key0 * stride_l);
#pragma unroll
            for (int i = 0; i < NP; ++i) reg[i] = *reinterpret_cast<const u32x4*>(tile + goff[i]);
        } else {
#pragma unroll
            for (int i = 0; i < NP; ++i) {
                const int idx = EXACT ? tid + i * NT : min(tid + i * NT, NCHUNK - 1);
                const int key = min(key0 + idx / CPR, L - 1);
                reg[i] = *reinterpret_cast<const u32x4*>(base + (int64_t)key * stride_l + (idx % CPR) * 8);
            }
        }
    }
    template <int STR>
    static __device__ __forceinline__ void store(const u32x4 (&reg)[NP], _Float16* dst, int tid) {
#pragma unroll
        for (int i = 0; i < NP; ++i) {
            const int idx = tid + i * NT;
            if (EXACT || idx < NCHUNK)
                *reinterpret_cast<u32x4*>(dst + (idx / CPR) * STR + (idx % CPR) * 8) = reg[i];
        }
    }
    __device__ __forceinline__ void load_k(const _Float16* kbase, int64_t sl, int key0, int L, int tid) {
        load(kreg, kbase, sl, key0, L, tid);
    }
    __device__ __forceinline__ void load_v(const _Float16* vbase, int64_t sl, int key0, int L, int tid) {
        load(vreg, vbase, sl, key0, L, tid);
    }
    __device__ __forceinline__ void store_k(_Float16* ks, int tid) const { store<G::KSTR>(kreg, ks, tid); }
    __device__ __forceinline__ void store_v(_Float16* vs, int tid) const { store<G::VSTR>(vreg, vs, tid); }
};

// Largest partial row sum (16 terms) the fast path of the online softmax accepts.
constexpr float kTrip = 16384.f;

// p = exp2(s * c + mc) for the NQB x 16 scores of a sub-tile, rounded to fp16 pairs (round toward
// zero), and the per-lane sums of the rounded values.  The sums are taken over the rounded
// probabilities that enter the second product, so numerator and denominator see the same rounding.
template <int NQB>
__device__ __forceinline__ void exp_pack_sum(const floatx16 (&s)[NQB], float c, const float (&mc)[NQB],
                                             uint32_t (&pk)[NQB][8], float (&ts)[NQB]) {
    const half2v ones = {(_Float16)1.0f, (_Float16)1.0f};
#pragma unroll
    for (int nb = 0; nb < NQB; ++nb) {
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

// Same exponentials without the sums: returns the bitwise OR of all packed fp16 pairs of the
// sub-tile.  A non-negative fp16 value is below 2.0 exactly when bit 14 is clear (inf and NaN have
// it set), so the OR tells whether any probability of the sub-tile reached 2.0.  The reference the
// exponentials are taken against carries a bias of kBias (log2 units) on top of the running row
// maximum: probabilities normally stay below 2^-kBias, and the fast path tolerates a reference
// that lags the true maximum by up to kBias + 1.  The factor 2^-kBias cancels between O and l; the
// smallest probabilities lose kBias bits of fp16 sub-normal range, far below the rounding of O.
constexpr float kBias = 6.0f;
constexpr uint32_t kTripBits = 0x40004000u;
template <int NQB>
__device__ __forceinline__ uint32_t exp_pack_or(const floatx16 (&s)[NQB], float c, const float (&mc)[NQB],
                                                uint32_t (&pk)[NQB][8]) {
    uint32_t orv = 0u;
#pragma unroll
    for (int nb = 0; nb < NQB; ++nb) {
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
            const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[nb][r], c, mc[nb]));
            const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[nb][r + 1], c, mc[nb]));
            const uint32_t pp = pack_rtz(p0, p1);
            pk[nb][r >> 1] = pp;
            orv |= pp;
        }
    }
    return orv;
}
__device__ __forceinline__ bool trips(uint32_t orv) { return (orv & kTripBits) != 0u; }

// A operand that makes v_mfma_f32_16x16x32_f16 add up the packed P^T registers of one k-step per
// query.  In that instruction lane l holds A[l % 16][8 (l / 16) + i] and B[8 (l / 16) + i][l % 16],
// and D[m][n] lands in lane n + 16 (m / 4), register m % 4.  Read as its B operand, the P^T registers
// of lane l hold eight keys of query l % 32, i.e. column n = l % 16 carries query n in k-blocks 0
// and 2 and query n + 16 in k-blocks 1 and 3.  With row 0 of A selecting k-blocks 0 and 2 and row 4
// selecting k-blocks 1 and 3, register 0 of lane q (q < 32) receives the sum over the 16 keys of
// query q: the lane that owns the query.  Lanes 32..63 receive zeros.
__device__ __forceinline__ half8 row_sum_operand(int lane) {
    const _Float16 v = (lane == 0 || lane == 32 || lane == 20 || lane == 52) ? (_Float16)1.0f : (_Float16)0.f;
    const half8 a = {v, v, v, v, v, v, v, v};
    return a;
}
template <int NQB>
__device__ __forceinline__ void row_sum_mfma(floatx4 (&lacc)[NQB], half8 sel, const uint32_t (&pk)[NQB][8]) {
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int nb = 0; nb < NQB; ++nb) {
            const u32x4 w = {pk[nb][4 * t], pk[nb][4 * t + 1], pk[nb][4 * t + 2], pk[nb][4 * t + 3]};
            lacc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(sel, __builtin_bit_cast(half8, w), lacc[nb], 0, 0, 0);
        }
}

// O^T[.][nb] *= alpha, in place.  Written as one instruction per register with the register tied
// as input and output, so that the rarely taken rescale does not make the compiler keep a second
// copy of the accumulators (and copy them on the common path).  The leading wait covers the
// matrix-core results the multiplies read.
template <int DB, int NQB>
__device__ __forceinline__ void scale_accumulators(floatx16 (&o)[DB][NQB], int nb, float alpha) {
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

// Per-wave state for NQB blocks of 32 queries: Q^T as B operands, O^T accumulators,
// online-softmax (m, l).
template <int H, int NQB>
struct WaveState {
    using G = Geometry<H>;
    half8 q[NQB][G::KS];
    floatx16 o[G::DB][NQB];
    float m[NQB];   // reference row maximum of the raw (unscaled) scores, identical in lanes l and l^32
    float mc[NQB];  // -m * c, the additive term of the exponent; +inf while no reference exists yet
    float l[NQB];   // running sum of exp over the keys this lane has seen (half of each tile)
    floatx4 lacc[NQB];  // ping-pong kernel: row sums accumulated by the matrix core, see row_sum_mfma
};

// LDS address of this lane's K row for sub-tile `sub` of a tile: A operand of S^T = K_sub * Q^T.
template <int H>
__device__ __forceinline__ const _Float16* k_operand_ptr(const _Float16* ks, int sub, int lane) {
    return ks + (sub * 32 + (lane & 31)) * Geometry<H>::KSTR + 8 * (lane >> 5);
}

// LDS address this lane hands to the transpose reads of sub-tile `sub`.  Inside each group of 16
// lanes, lane j receives, for i = 0..3, element (j % 4) of the 8-byte row fetched by lane
// 4 i + j / 4.  With lane s of a group pointing at V[key0 + s / 4][d0 + 4 (s % 4) ...], lane j ends
// up with V[key0 + i][d0 + j], i = 0..3: four consecutive keys of one head-dim column.
template <int H>
__device__ __forceinline__ const _Float16* v_operand_ptr(const _Float16* vs, int sub, int lane) {
    const int s16 = lane & 15;
    return vs + (sub * 32 + 4 * (lane >> 5) + (s16 >> 2)) * Geometry<H>::VSTR + 16 * ((lane >> 4) & 1) +
           4 * (s16 & 3);
}

// S^T = K_sub * Q^T for 32 keys and the wave's NQB x 32 queries.
template <int H, int NQB>
__device__ __forceinline__ void qk_mfma(floatx16 (&s)[NQB], const half8 (&q)[NQB][Geometry<H>::KS],
                                        const _Float16* krow) {
#pragma unroll
    for (int nb = 0; nb < NQB; ++nb)
#pragma unroll
        for (int r = 0; r < 16; ++r) s[nb][r] = 0.f;
#pragma unroll
    for (int kk = 0; kk < Geometry<H>::KS; ++kk) {
        const half8 a = *reinterpret_cast<const half8*>(krow + kk * 16);
#pragma unroll
        for (int nb = 0; nb < NQB; ++nb)
            s[nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, q[nb][kk], s[nb], 0, 0, 0);
    }
}

// O^T += V_sub^T * P^T.  k-slot (g, i) of k-step t is key 16 t + 8 (i / 4) + 4 g + i % 4 on both
// operands: that is where the packed P^T registers (accumulator rows 8 t .. 8 t + 7) come from, and
// the two transpose reads fetch keys 16 t + 4 g + {0..3} and 16 t + 8 + 4 g + {0..3}.
template <int H, int NQB>
__device__ __forceinline__ void pv_mfma(floatx16 (&o)[Geometry<H>::DB][NQB], const _Float16* vrow,
                                        const uint32_t (&pk)[NQB][8]) {
    using G = Geometry<H>;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        half8 pb[NQB];
#pragma unroll
        for (int nb = 0; nb < NQB; ++nb) {
            const u32x4 w = {pk[nb][4 * t], pk[nb][4 * t + 1], pk[nb][4 * t + 2], pk[nb][4 * t + 3]};
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
            for (int nb = 0; nb < NQB; ++nb)
                o[db][nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, pb[nb], o[db][nb], 0, 0, 0);
        }
    }
}

// Slow path of the online softmax, first part: bring the reference up to the true running maximum
// of the rows and rescale O and l.  mcu receives the exponent term to redo this sub-tile with.
template <int H, int NQB>
__device__ __forceinline__ void softmax_rebase(WaveState<H, NQB>& st, const floatx16 (&s)[NQB], float c,
                                               float (&mcu)[NQB], float bias = 0.f) {
    using G = Geometry<H>;
#pragma unroll
    for (int nb = 0; nb < NQB; ++nb) {
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
        st.lacc[nb][0] *= alpha;
        scale_accumulators<G::DB, NQB>(st.o, nb, alpha);
        st.m[nb] = m_new;
        st.mc[nb] = empty ? __builtin_inff() : -m_new * c - bias;
        mcu[nb] = empty ? 0.f : -m_new * c - bias;
    }
}

// ... second part: redo the exponentials of this sub-tile against the new reference.
template <int H, int NQB>
__device__ __forceinline__ void softmax_fix(WaveState<H, NQB>& st, const floatx16 (&s)[NQB], float c,
                                         uint32_t (&pk)[NQB][8], float (&ts)[NQB]) {
    float mcu[NQB];
    softmax_rebase<H, NQB>(st, s, c, mcu);
    exp_pack_sum<NQB>(s, c, mcu, pk, ts);
}

// Fast path: exponentiate against the reference maximum of the rows seen so far, without looking
// at this sub-tile's maximum.  Any reference works as long as numerator and denominator share it;
// it only has to keep exp2 inside the fp16 range.  Each lane checks that with its own partial row
// sum: 16 non-negative terms whose sum is <= kTrip are each <= kTrip, and anything that overflowed
// (inf) or was computed from an undefined reference (NaN) fails the comparison.  Only then the wave
// takes the slow path.
template <int H, int NQB>
__device__ __forceinline__ void softmax_check(WaveState<H, NQB>& st, const floatx16 (&s)[NQB], float c,
                                              uint32_t (&pk)[NQB][8], float (&ts)[NQB]) {
    bool ok = ts[0] <= kTrip;
#pragma unroll
    for (int nb = 1; nb < NQB; ++nb) ok = ok & (ts[nb] <= kTrip);
    if (__builtin_expect(__builtin_amdgcn_ballot_w64(!ok) != 0, 0)) softmax_fix<H, NQB>(st, s, c, pk, ts);
#pragma unroll
    for (int nb = 0; nb < NQB; ++nb) st.l[nb] += ts[nb];
}

// Processes 32 keys (one sub-tile) for the wave's queries, one stage after the other.  Used for
// the ragged last tile and for the additive-mask and causal variants.
//   ks/vs : LDS tile base for the current buffer
//   nvalid: number of valid keys in this sub-tile (only read when MASKED)
//   qrow  : sequence position of this lane's query in block 0 (block nb adds 32 nb); causal only
template <int H, int NQB, bool MASKED, int MODE>
__device__ __forceinline__ void process_subtile(WaveState<H, NQB>& st, const _Float16* ks,
                                                const _Float16* vs, int sub, int nvalid,
                                                float c, int lane,
                                                const _Float16* const (&mask_row)[NQB],
                                                int key_base, int L, int qrow = 0, bool mask_vec = false) {
    const int g = lane >> 5;
    // Additive mask: this lane's 16 keys of the sub-tile are four runs of four consecutive keys.
    // The mask values are fetched before the first product so that their latency hides behind it:
    // as 8-byte loads when every run is 8-byte aligned and entirely inside the row (L % 4 == 0 and
    // an aligned mask pointer, which `mask_vec` says), as single fp16 loads otherwise.
    half4 mk[NQB][4];
    if constexpr (MODE == kAdditive) {
#pragma unroll
        for (int nb = 0; nb < NQB; ++nb) {
            const _Float16* mrow = mask_row[nb];
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                const int key = key_base + 8 * r4 + 4 * g;
                mk[nb][r4] = half4{(_Float16)0.f, (_Float16)0.f, (_Float16)0.f, (_Float16)0.f};
                if (mrow != nullptr) {
                    if (mask_vec) {
                        if (key < L) mk[nb][r4] = *reinterpret_cast<const half4*>(mrow + key);
                    } else {
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                            if (key + j < L) mk[nb][r4][j] = mrow[key + j];
                    }
                }
            }
        }
    }
    floatx16 s[NQB];
    qk_mfma<H, NQB>(s, st.q, k_operand_ptr<H>(ks, sub, lane));

    if constexpr (MODE == kCausal) {
#pragma unroll
        for (int nb = 0; nb < NQB; ++nb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int key = key_base + 8 * (r >> 2) + 4 * g + (r & 3);
                if (key > qrow + 32 * nb) s[nb][r] = -__builtin_inff();
            }
    }
    if constexpr (MODE == kAdditive) {
        // The mask is added to the scaled score; S holds raw scores, so the mask is brought to raw
        // units: s * scale + mask = scale * (s + mask / scale).
        const float inv_scale = 1.4426950408889634f / c;
#pragma unroll
        for (int nb = 0; nb < NQB; ++nb)
#pragma unroll
            for (int r = 0; r < 16; ++r) s[nb][r] += (float)mk[nb][r >> 2][r & 3] * inv_scale;
    }
    if constexpr (MASKED) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int key = 8 * (r >> 2) + 4 * g + (r & 3);
            if (key >= nvalid) {
#pragma unroll
                for (int nb = 0; nb < NQB; ++nb) s[nb][r] = -__builtin_inff();
            }
        }
    }

    uint32_t pk[NQB][8];
    float ts[NQB];
    exp_pack_sum<NQB>(s, c, st.mc, pk, ts);
    softmax_check<H, NQB>(st, s, c, pk, ts);
    pv_mfma<H, NQB>(st.o, v_operand_ptr<H>(vs, sub, lane), pk);
}

// One stage of the software pipeline: three independent pieces of work on three sub-tiles,
//   s_next = K_{j+1} Q^T          (matrix core)
//   p_cur  = exp2(s_cur ...)      (vector ALU)
//   O^T   += V_{j-1}^T p_prev     (matrix core)
// written out in the order the instructions should issue: the exponentials are cut into 8 NQB chunks
// of one fp16 pair (2 fma, 2 exp, 1 pack, 1 dot2: about the duration of one 32x32x16 MFMA), each
// followed by its share of the matrix instructions, with the LDS operand reads issued PF operands
// ahead of their use.  A scheduling barrier after every chunk keeps the compiler from regrouping
// them, so that one wave by itself keeps the matrix core and the vector ALU busy together.
template <int H, int NQB>
__device__ __forceinline__ void pipeline_stage(WaveState<H, NQB>& st, floatx16 (&s_next)[NQB],
                                               const floatx16 (&s_cur)[NQB], uint32_t (&p_cur)[NQB][8],
                                               const uint32_t (&p_prev)[NQB][8], const _Float16* krow,
                                               const _Float16* vrow, float c) {
    using G = Geometry<H>;
    constexpr int NQK = G::KS;            // operand slots of the first product (K rows)
    constexpr int NPV = 2 * G::DB;        // operand slots of the second product (V^T blocks)
    constexpr int NU = NQK + NPV;
    constexpr int NM = NQB * NU;          // matrix instructions of this stage
    constexpr int NC = 8 * NQB;           // chunks of vector work (one fp16 pair each)
    constexpr int D = 2;                  // chunks of vector work issued before the first MFMA
    constexpr int PF = NU < 3 ? NU : 3;   // operand slots fetched ahead
    typedef short short8v __attribute__((ext_vector_type(8)));

    half8 opnd[NU];
    auto fetch = [&](int u) {
        if (u < NQK) {
            opnd[u] = *reinterpret_cast<const half8*>(krow + u * 16);
        } else {
            const int t = (u - NQK) / G::DB, db = (u - NQK) % G::DB;
            const _Float16* p0 = vrow + (16 * t) * G::VSTR + db * 32;
            const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((FA_LDS short4v*)(p0));
            const short4v hi =
                __builtin_amdgcn_ds_read_tr16_b64_v4i16((FA_LDS short4v*)(p0 + 8 * G::VSTR));
            const short8v both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            opnd[u] = __builtin_bit_cast(half8, both);
        }
    };
    auto mma = [&](int j) {
        const int u = j / NQB, nb = j % NQB;
        if (u < NQK) {
            if (u == 0) {
                floatx16 z;
#pragma unroll
                for (int r = 0; r < 16; ++r) z[r] = 0.f;
                s_next[nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(opnd[u], st.q[nb][u], z, 0, 0, 0);
            } else {
                s_next[nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(opnd[u], st.q[nb][u], s_next[nb], 0, 0, 0);
            }
        } else {
            const int t = (u - NQK) / G::DB, db = (u - NQK) % G::DB;
            const u32x4 w = {p_prev[nb][4 * t], p_prev[nb][4 * t + 1], p_prev[nb][4 * t + 2],
                             p_prev[nb][4 * t + 3]};
            st.o[db][nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(opnd[u], __builtin_bit_cast(half8, w),
                                                                  st.o[db][nb], 0, 0, 0);
        }
    };

    const half2v ones = {(_Float16)1.0f, (_Float16)1.0f};
    float ts[NQB];
#pragma unroll
    for (int nb = 0; nb < NQB; ++nb) ts[nb] = 0.f;
    float e0 = 0.f, e1 = 0.f;   // exponentials of the previous chunk, packed one chunk later

#pragma unroll
    for (int u = 0; u < PF; ++u) fetch(u);
#pragma unroll
    for (int i = 0; i <= NC; ++i) {
        if (i < NC) {
            const int nb = i >> 3, r = (i & 7) * 2;
            const float a0 = __builtin_fmaf(s_cur[nb][r], c, st.mc[nb]);
            const float a1 = __builtin_fmaf(s_cur[nb][r + 1], c, st.mc[nb]);
            const float n0 = __builtin_amdgcn_exp2f(a0);
            const float n1 = __builtin_amdgcn_exp2f(a1);
            if (i > 0) {
                const int pnb = (i - 1) >> 3, pr2 = (i - 1) & 7;
                const uint32_t pp = pack_rtz(e0, e1);
                p_cur[pnb][pr2] = pp;
                ts[pnb] = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, pp), ones, ts[pnb], false);
            }
            e0 = n0;
            e1 = n1;
        } else {
            const uint32_t pp = pack_rtz(e0, e1);
            p_cur[NQB - 1][7] = pp;
            ts[NQB - 1] = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, pp), ones, ts[NQB - 1], false);
        }
        if (i >= D) {
            const int jlo = (i - D) * NM / NC;
            const int jhi = i == NC ? NM : (i - D + 1) * NM / NC;
#pragma unroll
            for (int j = jlo; j < jhi; ++j) {
                mma(j);
                if (j % NQB == 0 && j / NQB + PF < NU) fetch(j / NQB + PF);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    softmax_check<H, NQB>(st, s_cur, c, p_cur, ts);
}

// O = O^T / l in f32, one rounding to fp16, 8-byte stores of four consecutive head-dim elements.
// With lse given (one float per query row of this (batch, head)), also writes
// log(sum_j exp(score_j)) = m * scale + log(l), the quantity a backward pass needs.
template <int H, int NQB>
__device__ __forceinline__ void store_output(WaveState<H, NQB>& st, _Float16* obase, int64_t stride_l,
                                             int q0, int L, int lane, float* lse = nullptr, float c = 0.f,
                                             float l_bias = 0.f) {
    using G = Geometry<H>;
    const int g = lane >> 5;
    const int ln = lane & 31;
#pragma unroll
    for (int nb = 0; nb < NQB; ++nb) {
        const float lt = pair_sum(st.l[nb]);
        // A row whose every key carried a -inf mask has l = 0: emit zeros rather than NaN.
        const float inv = lt > 0.f ? 1.0f / lt : 0.f;
        const int row = q0 + nb * 32 + ln;
        if (lse != nullptr && g == 0 && row < L)
            lse[row] = lt > 0.f ? (st.m[nb] * c + __builtin_log2f(lt) + l_bias) * 0.6931471805599453f : -__builtin_inff();
        if (row < L) {
            _Float16* orow = obase + (int64_t)row * stride_l;
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

// Template parameters: head_dim H, NW wave64s per workgroup, BK keys per LDS tile, NQB blocks of 32
// query rows per wave, WPE waves per SIMD the register budget is sized for.
template <int H, int NW, int BK, int NQB, int WPE, int MODE>
__global__ __launch_bounds__(NW * 64, WPE) void fwd_kernel(const FwdParams p) {
    using G = Geometry<H>;
    constexpr int QW = 32 * NQB;            // query rows per wave
    constexpr int BQ = NW * QW;             // query rows per workgroup
    constexpr int NT = NW * 64;
    constexpr int NSUB = BK / 32;
    static_assert(BK == 64, "the pipelined loop is written for two sub-tiles per tile");

    extern __shared__ __attribute__((aligned(16))) _Float16 smem[];
    _Float16* const ks_base = smem;                                // [2][BK][KSTR]
    _Float16* const vs_base = smem + 2 * BK * G::KSTR;             // [2][BK][VSTR]
    constexpr int KTILE = BK * G::KSTR;
    constexpr int VTILE = BK * G::VSTR;

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
    // causal: longest-running query tiles of a head first
    const int qt = MODE == kCausal ? p.n_qtiles - 1 - logical % p.n_qtiles : logical % p.n_qtiles;
    const int b = bh / p.R;
    const int h = bh % p.R;
    const int L = p.L;

    const int64_t head_off = (int64_t)b * p.stride_b + (int64_t)h * p.stride_h;
    const _Float16* qbase = p.q + head_off;
    const _Float16* kbase = p.k + head_off;
    const _Float16* vbase = p.v + head_off;
    _Float16* obase = p.o + head_off;
    const int q0 = qt * BQ + wave * QW;

    // V columns beyond H (only when H = 16) stay zero for the whole kernel.
    if constexpr (G::HV != H) {
        for (int i = tid; i < 2 * VTILE; i += NT) vs_base[i] = (_Float16)0.f;
        __syncthreads();
    }

    WaveState<H, NQB> st;
#pragma unroll
    for (int nb = 0; nb < NQB; ++nb) {
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

    const int ntiles = (L + BK - 1) / BK;
    const int nfull = L / BK;
    const float c = p.scale_log2e;
    const int64_t sl = p.stride_l;
    TileLoader<H, NW, BK> loader;
    loader.init(sl, tid);

    if constexpr (MODE != kPlain) {
        // Additive-mask and causal variants: plain double-buffered loop, one sub-tile after the
        // other.  Causal: the workgroup stops at the tile that holds its last query, and a wave
        // skips the sub-tiles that lie entirely above its own last query.
        const _Float16* mask_row[NQB];
#pragma unroll
        for (int nb = 0; nb < NQB; ++nb) {
            const int row = q0 + nb * 32 + ln;
            mask_row[nb] = nullptr;
            if constexpr (MODE == kAdditive)
                if (row < L) mask_row[nb] = p.mask + (int64_t)b * L * L + (int64_t)row * L;
        }
        int nt = ntiles;
        if constexpr (MODE == kCausal) {
            const int wg_last = min(qt * BQ + BQ, L) - 1;
            nt = wg_last / BK + 1;
        }
        const int wave_last = q0 + QW - 1;
        const bool mask_vec = MODE == kAdditive && (L & 3) == 0 && (reinterpret_cast<uintptr_t>(p.mask) & 7) == 0;

        loader.load_k(kbase, sl, 0, L, tid);
        loader.load_v(vbase, sl, 0, L, tid);
        loader.store_k(ks_base, tid);
        loader.store_v(vs_base, tid);
        __syncthreads();
        for (int t = 0; t < nt; ++t) {
            const int buf = t & 1;
            const bool has_next = t + 1 < nt;
            if (has_next) {
                loader.load_k(kbase, sl, (t + 1) * BK, L, tid);
                loader.load_v(vbase, sl, (t + 1) * BK, L, tid);
            }
#pragma unroll
            for (int sub = 0; sub < NSUB; ++sub) {
                const int key_base = t * BK + sub * 32;
                const int nvalid = L - key_base;
                if (nvalid > 0 && (MODE != kCausal || key_base <= wave_last))
                    process_subtile<H, NQB, true, MODE>(st, ks_base + buf * KTILE, vs_base + buf * VTILE,
                                                        sub, nvalid, c, lane, mask_row, key_base, L, q0 + ln,
                                                        mask_vec);
            }
            if (has_next) {
                loader.store_k(ks_base + (buf ^ 1) * KTILE, tid);
                loader.store_v(vs_base + (buf ^ 1) * VTILE, tid);
            }
            __syncthreads();
        }
    } else {
        // Software pipeline over the full tiles.  With j the sub-tile index, stage j issues
        // QK^T of sub-tile j + 1, the exponentials of sub-tile j and PV of sub-tile j - 1, so K runs
        // one tile ahead of V: iteration T of the loop below reads K tile T + 1 and V tile T and
        // refills the other K buffer with tile T + 2 and the other V buffer with tile T + 1.
        loader.load_k(kbase, sl, 0, L, tid);
        loader.load_v(vbase, sl, 0, L, tid);
        loader.store_k(ks_base, tid);
        loader.store_v(vs_base, tid);
        loader.load_k(kbase, sl, BK, L, tid);
        loader.store_k(ks_base + KTILE, tid);
        __syncthreads();

        const bool ragged = nfull < ntiles;
        if (nfull > 0) {
            floatx16 sa[NQB], sb[NQB];
            uint32_t pa[NQB][8], pb[NQB][8];
            float ts[NQB];
            // stage 0 (no PV yet)
            qk_mfma<H, NQB>(sa, st.q, k_operand_ptr<H>(ks_base, 0, lane));
            qk_mfma<H, NQB>(sb, st.q, k_operand_ptr<H>(ks_base, 1, lane));
            exp_pack_sum<NQB>(sa, c, st.mc, pa, ts);
            softmax_check<H, NQB>(st, sa, c, pa, ts);
            // every wave is done with K tile 0 before anyone overwrites its buffer
            __syncthreads();

            for (int T = 0; T + 1 < nfull; ++T) {
                const _Float16* kcur = ks_base + ((T + 1) & 1) * KTILE;
                const _Float16* vcur = vs_base + (T & 1) * VTILE;
                loader.load_k(kbase, sl, (T + 2) * BK, L, tid);
                loader.load_v(vbase, sl, (T + 1) * BK, L, tid);
                pipeline_stage<H, NQB>(st, sa, sb, pb, pa, k_operand_ptr<H>(kcur, 0, lane),
                                       v_operand_ptr<H>(vcur, 0, lane), c);
                pipeline_stage<H, NQB>(st, sb, sa, pa, pb, k_operand_ptr<H>(kcur, 1, lane),
                                       v_operand_ptr<H>(vcur, 1, lane), c);
                loader.store_k(ks_base + (T & 1) * KTILE, tid);
                loader.store_v(vs_base + ((T + 1) & 1) * VTILE, tid);
                __syncthreads();
            }

            // drain: exponentials of the last full sub-tile, PV of the last two
            // (PV of sub-tile j - 1 goes first: a rescale triggered by sub-tile j must see it in O)
            const _Float16* vlast = vs_base + ((nfull - 1) & 1) * VTILE;
            if (ragged) loader.load_v(vbase, sl, nfull * BK, L, tid);
            pv_mfma<H, NQB>(st.o, v_operand_ptr<H>(vlast, 0, lane), pa);
            exp_pack_sum<NQB>(sb, c, st.mc, pb, ts);
            softmax_check<H, NQB>(st, sb, c, pb, ts);
            pv_mfma<H, NQB>(st.o, v_operand_ptr<H>(vlast, 1, lane), pb);
            if (ragged) {
                loader.store_v(vs_base + (nfull & 1) * VTILE, tid);
                __syncthreads();
            }
        }
        if (ragged) {
            const int buf = nfull & 1;
            const int key0 = nfull * BK;
            const _Float16* no_mask[NQB] = {};
#pragma unroll
            for (int sub = 0; sub < NSUB; ++sub) {
                const int nvalid = L - key0 - sub * 32;
                if (nvalid > 0)
                    process_subtile<H, NQB, true, kPlain>(st, ks_base + buf * KTILE, vs_base + buf * VTILE,
                                                          sub, nvalid, c, lane, no_mask, key0 + sub * 32, L);
            }
        }
    }

    store_output<H, NQB>(st, obase, p.stride_l, q0, L, lane,
                         p.lse != nullptr ? p.lse + ((int64_t)b * p.R + h) * L : nullptr, c);
}

// ---------------------------------------------------------------------------------------------
// Ping-pong variant: eight waves per workgroup, two per SIMD.  A SIMD picks between its waves
// oldest first, so two free-running waves do not share it evenly: the older one runs at nearly
// its single-wave speed, the younger one fills the gaps, and they drift apart (measured by
// `fa_test issue-probe`).  Here the two waves of a SIMD are kept in step instead.  The waves form
// two groups (0-3 and 4-7, one wave of each per SIMD) that alternate between a vector phase
// (exponentials of sub-tile j) and a matrix phase (PV of sub-tile j, QK^T of sub-tile j + 1), the
// second group one phase behind the first, with a workgroup barrier between phases: while one
// group keeps the matrix cores busy the other does the softmax on the vector ALUs of the same SIMDs.
//
// Causal (CAUSAL = true): a wave stops computing at the sub-tile that holds its last query and then
// only keeps up its share of the K/V streaming and of the barriers; scores above the diagonal are
// set to -inf in the (at most three) sub-tiles that straddle it.  Query tile t of a head costs
// t + 1 key blocks, so a workgroup takes the tiles t and n - 1 - t one after the other and all
// workgroups of the grid do the same amount of work.
//
// K and V stream through three-slot LDS rings.  Group 0 loads K, group 1 loads V, each during its
// own vector phases: at its first vector phase of tile T a group writes tile T + 2 (fetched into
// registers one tile earlier) to the ring and, at the start of the following matrix phase, issues
// the global loads of tile T + 3.  Slot (T + 2) % 3 last held tile T - 1, whose final reader
// finished at least one barrier earlier.
template <int H, int NQB>
constexpr int lds_bytes_pingpong() {
    using G = Geometry<H>;
    return 3 * 64 * (G::KSTR + G::VSTR) * (int)sizeof(_Float16);
}

__device__ __forceinline__ void phase_barrier() {
    // LDS traffic of this wave is complete (writes visible, reads returned) before the barrier;
    // global loads in flight are deliberately not waited for.  The scheduling barriers keep the
    // compiler from moving matrix or vector instructions of one phase into the next.
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
}

// One group's share of a 64-key tile: per-thread chunk offsets are computed once, a tile is then
// fetched with one pointer bump and NP 16-byte loads.
template <int H, int NT>
struct GroupLoader {
    static constexpr int CPR = H / 8;
    static constexpr int NCHUNK = 64 * CPR;
    static constexpr int NP = (NCHUNK + NT - 1) / NT;
    static constexpr bool EXACT = NCHUNK % NT == 0;
    u32x4 reg[NP];
    int64_t goff[NP];   // element offset of the chunk inside a tile
    int loff[NP];       // element offset of the chunk inside an LDS tile
    int row[NP];
    int col[NP];

    __device__ __forceinline__ void init(int64_t stride_l, int lds_stride, int gtid) {
#pragma unroll
        for (int i = 0; i < NP; ++i) {
            const int idx = gtid + i * NT;
            row[i] = (EXACT || idx < NCHUNK) ? idx / CPR : (1 << 30);
            col[i] = (idx % CPR) * 8;
            goff[i] = (int64_t)(idx / CPR) * stride_l + (idx % CPR) * 8;
            loff[i] = (idx / CPR) * lds_stride + (idx % CPR) * 8;
        }
    }
    // Rows at or beyond L are read from row L - 1 instead (no predicated loads, so no load ever
    // waits for another): their scores are masked to -inf, or belong to sub-tiles that are never
    // consumed, and a probability of exactly zero times a finite V row contributes nothing.
    // Tiles starting at or beyond `limit` are not fetched at all (limit <= L).
    __device__ __forceinline__ void load(const _Float16* src, int64_t stride_l, int key0, int limit, int L) {
        if (key0 >= limit) return;
        if (key0 + 64 <= L && EXACT) {
            const _Float16* tile = src + (int64_t)key0 * stride_l;
#pragma unroll
            for (int i = 0; i < NP; ++i) reg[i] = *reinterpret_cast<const u32x4*>(tile + goff[i]);
        } else {
#pragma unroll
            for (int i = 0; i < NP; ++i) {
                const int r = min(key0 + min(row[i], 63), L - 1);
                reg[i] = *reinterpret_cast<const u32x4*>(src + (int64_t)r * stride_l + col[i]);
            }
        }
    }
    __device__ __forceinline__ void store(_Float16* dst) const {
#pragma unroll
        for (int i = 0; i < NP; ++i)
            if (EXACT || row[i] < 64) *reinterpret_cast<u32x4*>(dst + loff[i]) = reg[i];
    }
};

template <int H, int NW, int NQB, int WPE, bool CAUSAL>
__global__ __launch_bounds__(NW * 64, WPE) void fwd_kernel_pingpong(const FwdParams p) {
    using G = Geometry<H>;
    constexpr int BK = 64;
    static_assert(NW == 8 || NW == 16, "two groups of four or eight waves");
    constexpr int QW = 32 * NQB;
    constexpr int BQ = NW * QW;
    constexpr int KTILE = BK * G::KSTR;
    constexpr int VTILE = BK * G::VSTR;
    constexpr int GT = NW * 32;             // threads of one group
    typedef short short8v __attribute__((ext_vector_type(8)));

    extern __shared__ __attribute__((aligned(16))) _Float16 smem[];
    _Float16* const ks_base = smem;                      // [3][BK][KSTR]
    _Float16* const vs_base = smem + 3 * KTILE;          // [3][BK][VSTR]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // waves w, w + 4, w + 8, ... share a SIMD: group = bit 2 of the wave index
    const int grp = (wave >> 2) & 1;
    const int gtid = ((wave >> 3) << 8) | (tid & 255);
    const int g = lane >> 5;
    const int ln = lane & 31;

    const int wg = blockIdx.x;
    const int logical = (wg % kNumXcd) * p.wgs_per_xcd + wg / kNumXcd;
    if (logical >= p.total_wgs) return;
    // Causal: query tile t of a head costs t + 1 key blocks, so a workgroup takes two tiles, t and
    // n_qtiles - 1 - t, one after the other: every workgroup of the grid then does the same amount
    // of work, whatever order the hardware hands them out in.  p.n_qtiles counts these pairs.
    const int tiles_per_head = (p.L + BQ - 1) / BQ;
    const int bh = logical / p.n_qtiles;
    const int slot = logical % p.n_qtiles;
    const int b = bh / p.R;
    const int h = bh % p.R;
    const int L = p.L;

    const int64_t head_off = (int64_t)b * p.stride_b + (int64_t)h * p.stride_h;
    const _Float16* qbase = p.q + head_off;
    const _Float16* kbase = p.k + head_off;
    const _Float16* vbase = p.v + head_off;
    _Float16* obase = p.o + head_off;
    const int64_t sl = p.stride_l;

    if constexpr (G::HV != H) {
        for (int i = tid; i < 3 * VTILE; i += NW * 64) vs_base[i] = (_Float16)0.f;
        __syncthreads();
    }

    for (int pass = 0; pass < (CAUSAL ? 2 : 1); ++pass) {
    const int qt = CAUSAL ? (pass == 0 ? tiles_per_head - 1 - slot : slot) : slot;
    if (CAUSAL && pass == 1 && 2 * slot == tiles_per_head - 1) break;   // middle tile of an odd count
    const int q0 = qt * BQ + wave * QW;

    WaveState<H, NQB> st;
#pragma unroll
    for (int nb = 0; nb < NQB; ++nb) {
        const int row = q0 + nb * 32 + ln;
#pragma unroll
        for (int kk = 0; kk < G::KS; ++kk) {
            u32x4 w = {0u, 0u, 0u, 0u};
            if (row < L)
                w = *reinterpret_cast<const u32x4*>(qbase + (int64_t)row * sl + kk * 16 + 8 * g);
            st.q[nb][kk] = __builtin_bit_cast(half8, w);
        }
        st.m[nb] = -__builtin_inff();
        st.mc[nb] = __builtin_inff();
        st.l[nb] = 0.f;
        st.lacc[nb] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int db = 0; db < G::DB; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) st.o[db][nb][r] = 0.f;
    }

    const float c = p.scale_log2e;
    // causal: the workgroup stops at the sub-tile that holds its last query, and each wave at the
    // sub-tile that holds its own last query (nact); after that a wave only keeps up its share of
    // the K/V streaming and the barriers
    const int Lk = CAUSAL ? min(qt * BQ + BQ, L) : L;
    const int nsub = (Lk + 31) >> 5;
    const int last_valid = Lk - (nsub - 1) * 32;    // valid keys in the last sub-tile (1..32)
    const int nact = CAUSAL ? min(nsub, (q0 + QW) >> 5) : nsub;

    // Group 0 streams K, group 1 streams V.
    GroupLoader<H, GT> gl;
    gl.init(sl, grp == 0 ? G::KSTR : G::VSTR, gtid);
    const _Float16* const gsrc = grp == 0 ? kbase : vbase;
    _Float16* const ring = grp == 0 ? ks_base : vs_base;
    const int ring_tile = grp == 0 ? KTILE : VTILE;

    // prologue: tiles 0 and 1 into the ring, tile 2 into registers
    gl.load(gsrc, sl, 0, Lk, L);
    gl.store(ring);
    gl.load(gsrc, sl, BK, Lk, L);
    gl.store(ring + ring_tile);
    gl.load(gsrc, sl, 2 * BK, Lk, L);
    __syncthreads();

    floatx16 s[NQB];
    uint32_t pk[NQB][8];
    const half8 sel = row_sum_operand(lane);
    qk_mfma<H, NQB>(s, st.q, k_operand_ptr<H>(ks_base, 0, lane));
    if (grp == 1) phase_barrier();                  // the second group runs one phase behind

    for (int j = 0; j < nact; ++j) {
        const int T = j >> 1;
        const int jn = j + 1;
        // ---- vector phase -------------------------------------------------------------------
        // First the LDS traffic of this phase: the tile fetched one tile-time ago goes into the
        // ring, and the K rows of the next sub-tile come out of it (they were written several
        // phases ago), so that the matrix phase starts with its operands in registers.
        if ((j & 1) == 0) gl.store(ring + ((T + 2) % 3) * ring_tile);
        half8 kop[G::KS];
        {
            const _Float16* krow = k_operand_ptr<H>(ks_base + ((jn >> 1) % 3) * KTILE, jn & 1, lane);
#pragma unroll
            for (int kk = 0; kk < G::KS; ++kk) kop[kk] = *reinterpret_cast<const half8*>(krow + kk * 16);
        }
        // ... and the first half of the V^T operands of this sub-tile
        const _Float16* vrow = v_operand_ptr<H>(vs_base + (T % 3) * VTILE, j & 1, lane);
        half8 vop[2][G::DB];
        auto vfetch = [&](int t) {
#pragma unroll
            for (int db = 0; db < G::DB; ++db) {
                const _Float16* p0 = vrow + (16 * t) * G::VSTR + db * 32;
                const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((FA_LDS short4v*)(p0));
                const short4v hi =
                    __builtin_amdgcn_ds_read_tr16_b64_v4i16((FA_LDS short4v*)(p0 + 8 * G::VSTR));
                const short8v both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                vop[t][db] = __builtin_bit_cast(half8, both);
            }
        };
        vfetch(0);
        __builtin_amdgcn_sched_barrier(0);
        if (j == nsub - 1 && last_valid < 32) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int key = 8 * (r >> 2) + 4 * g + (r & 3);
                if (key >= last_valid) {
#pragma unroll
                    for (int nb = 0; nb < NQB; ++nb) s[nb][r] = -__builtin_inff();
                }
            }
        }
        if constexpr (CAUSAL) {
            if (j * 32 + 31 > q0) {     // the sub-tile reaches above the diagonal for some of the wave's queries
#pragma unroll
                for (int nb = 0; nb < NQB; ++nb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int key = j * 32 + 8 * (r >> 2) + 4 * g + (r & 3);
                        if (key > q0 + 32 * nb + ln) s[nb][r] = -__builtin_inff();
                    }
            }
        }
        // Exponentials against the reference maximum of the rows seen so far; the row sums are left
        // to the matrix phase (row_sum_mfma), the overflow check works on the packed values.
        if (__builtin_expect(__builtin_amdgcn_ballot_w64(trips(exp_pack_or<NQB>(s, c, st.mc, pk))) != 0, 0)) {
            float mcu[NQB];
            softmax_rebase<H, NQB>(st, s, c, mcu, kBias);
            exp_pack_or<NQB>(s, c, mcu, pk);
        }
        phase_barrier();
        // ---- matrix phase -------------------------------------------------------------------
#pragma unroll
        for (int kk = 0; kk < G::KS; ++kk) {
#pragma unroll
            for (int nb = 0; nb < NQB; ++nb) {
                if (kk == 0) {
                    floatx16 z;
#pragma unroll
                    for (int r = 0; r < 16; ++r) z[r] = 0.f;
                    s[nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kop[kk], st.q[nb][kk], z, 0, 0, 0);
                } else {
                    s[nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kop[kk], st.q[nb][kk], s[nb], 0, 0, 0);
                }
            }
            if (kk == 0) {
                vfetch(1);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < 2; ++t) {
#pragma unroll
            for (int db = 0; db < G::DB; ++db) {
#pragma unroll
                for (int nb = 0; nb < NQB; ++nb) {
                    const u32x4 w = {pk[nb][4 * t], pk[nb][4 * t + 1], pk[nb][4 * t + 2], pk[nb][4 * t + 3]};
                    st.o[db][nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                        vop[t][db], __builtin_bit_cast(half8, w), st.o[db][nb], 0, 0, 0);
                }
            }
        }
        row_sum_mfma<NQB>(st.lacc, sel, pk);
        // the global loads of the tile three ahead go last: they cost this wave a few issue slots
        // while its matrix instructions are already queued
        if ((j & 1) == 0) gl.load(gsrc, sl, (T + 3) * BK, Lk, L);
        phase_barrier();
    }
    if constexpr (CAUSAL) {
        for (int j = nact; j < nsub; ++j) {
            const int T = j >> 1;
            if ((j & 1) == 0) gl.store(ring + ((T + 2) % 3) * ring_tile);
            phase_barrier();
            if ((j & 1) == 0) gl.load(gsrc, sl, (T + 3) * BK, Lk, L);
            phase_barrier();
        }
    }
    if (grp == 0) phase_barrier();

#pragma unroll
    for (int nb = 0; nb < NQB; ++nb) st.l[nb] = st.lacc[nb][0];
    store_output<H, NQB>(st, obase, sl, q0, L, lane,
                         p.lse != nullptr ? p.lse + ((int64_t)b * p.R + h) * L : nullptr, c, kBias);
    }   // pass
}

}  // namespace fa
