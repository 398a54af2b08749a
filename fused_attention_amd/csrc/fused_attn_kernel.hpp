// Fused multi-head attention forward for gfx950 (MI355X, CDNA4).
//
// One kernel computes O = softmax(Q K^T * scale) V per (batch, head) without ever
// writing the L x L score matrix to memory.  It replaces, as a single pass, the
// reference's attention_kernel and every threadblock_* helper it calls
// (reference include/fused_attn.cuh:48-538 and :605-858).
//
// Two kernels share the pieces in this file and in fused_attn_kernel_impl.inc:
//   fwd_kernel           four waves, software pipelined inside each wave (plain and causal); its
//                        additive-mask variant (plain loop) serves small grids and unaligned masks
//   fwd_kernel_pingpong  eight waves in two groups that alternate vector and matrix phases;
//                        plain, causal and additive mask (mask rows 16-byte aligned)
// Work decomposition
//   workgroup  = NW wave64s, each wave owns 32 NQB query rows (NQB = 1 or 2 blocks of 32)
//   K/V        = streamed in 64-key tiles through an LDS ring: global -> registers -> LDS, two slots
//                (fwd_kernel), or direct-to-LDS loads, three slots (fwd_kernel_pingpong)
//   per 32 keys: S^T = K_sub * Q^T        v_mfma_f32_32x32x16_{f16,bf16}, Q held in registers
//                online softmax on S^T     f32, state (m, l) per lane
//                O^T += V_sub^T * P^T      same MFMA, V^T fetched with ds_read_b64_tr_b16
//
// Why the transposed products: in the 32x32 accumulator layout lane l owns column
// (l % 32) -- one query -- and 16 of the 32 rows (keys); lane l^32 owns the other 16.
// A softmax row therefore lives in one lane pair, so row max / row sum need 15 in-lane
// ops and a single v_permlane32_swap.  The packed 16-bit P^T registers are, as they stand,
// a valid B operand of the second product provided the A operand (V^T) enumerates keys
// in the same order, which the transpose-read from the V tile provides.
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
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint16_t u16x4 __attribute__((ext_vector_type(4)));

#define FA_LDS __attribute__((address_space(3)))

struct FwdParams {
    const _Float16* q;
    const _Float16* k;
    const _Float16* v;
    const _Float16* mask;  // additive [B, L, L] or nullptr
    _Float16* o;
    float* lse;            // optional [B, R, L] natural-log row sums of exp(scores), or nullptr
    int64_t stride_b;      // q, k, v: elements between batches
    int64_t stride_h;      // ... between heads
    int64_t stride_l;      // ... between sequence positions
    int64_t ostride_b;     // the same three for o
    int64_t ostride_h;
    int64_t ostride_l;
    int B, R, L;
    int n_qtiles;          // workgroups per (batch, head): ceil(L / queries per workgroup), or half of
                           // that (rounded up) when a causal workgroup takes a pair of query tiles
    int total_wgs;         // B * R * n_qtiles
    int wgs_per_xcd;       // ceil(total_wgs / 8)
    int heads_per_xcd;     // causal eight-wave launches: 0 = every workgroup takes the pair of query tiles
                           // (t, n - 1 - t) of one head; > 0 = resident grid, the heads of an XCD's
                           // workgroups (B * R / 8 of them) dealt out tile by tile, see the kernel
    float scale_log2e;     // scale * log2(e)
    float bias;            // bias of the reference of the exponentials, log2 units (see kBiasMin)
};

constexpr int kNumXcd = 8;

// Kernel variants of the non-ping-pong kernel.
constexpr int kPlain = 0;    // no mask: software-pipelined loop
constexpr int kAdditive = 1; // additive [B, L, L] mask
constexpr int kCausal = 2;   // key index <= query index, key tiles above the diagonal skipped
constexpr int kCausalDealt = 3;   // eight-wave kernel only: causal with the query tiles dealt out to a resident grid

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

// Additive-mask variant: behind the K/V buffers every wave has a private slab for the mask values
// of its 32 NQB queries and the 64 keys of the current tile (row stride kMaskStr halves: 128 bytes
// of mask plus 16 of padding).
constexpr int kMaskStr = 72;
// Not at head_dim 128: there the slabs would cost the second resident workgroup of a compute unit.
template <int H>
constexpr bool mask_staging() { return H <= 64; }
template <int H, int NW, int BK, int NQB>
constexpr int lds_bytes_masked() {
    return lds_bytes<H, NW, BK>() + (mask_staging<H>() ? NW * 32 * NQB * kMaskStr * (int)sizeof(_Float16) : 0);
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

// Bias (log2 units) of the reference the exponentials are taken against, in every kernel
// (FwdParams::bias), and the largest sum of a query's 32 probabilities of one sub-tile that the
// eight-wave kernel's fast path accepts.  A key at the reference maximum gets the probability
// 2^-bias.  The probabilities are rounded to fp16 before the second product (normal numbers down
// to 2^-14, subnormals down to 2^-24), so a weight more than 24 - bias log2 units below the row
// maximum is lost: a tail of L small weights loses at most L 2^-(24 - bias) of the row.  The
// launcher picks bias = 11 - ceil(log2 L), between kBiasMin and kBiasMax, which keeps that share
// at or below 2^-13 = 1.2e-4 whatever the sequence length; what is left of the fp16 range is the
// leash of the speculative reference, which may lag the true maximum by 15 + bias log2 units (14
// in the four-wave kernels, whose check works on half rows) before the check sends the wave down
// the slow path: 14 units at L = 4096, 12 at 16384, 10 at 65536.
constexpr float kBiasMin = -8.0f;
constexpr float kBiasMax = 6.0f;
constexpr float kTripSum = 32768.f;

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

// Ring tiles of the ping-pong kernel are chunk-major: a 64-key tile of H columns is stored as H / 8
// columns of 64 rows x 16 bytes, column c at c * kColStride halves.  One direct-to-LDS load of a
// wave (64 lanes x 16 bytes, contiguous in LDS) fills one column, lane = key row.  The 64-byte pad
// between columns spreads the four columns touched by a transpose read over all banks.
constexpr int kColStride = 64 * 8 + 32;
template <int H>
constexpr int ring_tile_k() { return (H / 8) * kColStride; }
template <int H>
constexpr int ring_tile_v() { return (Geometry<H>::HV / 8) * kColStride; }
// Per-lane part of the K operand address in a ring tile: row (sub * 32 + lane % 32) of column
// lane / 32; k-step kk adds 2 kk columns.
__device__ __forceinline__ const _Float16* k_ring_ptr(const _Float16* ks, int sub, int lane) {
    return ks + (lane >> 5) * kColStride + (sub * 32 + (lane & 31)) * 8;
}

// Per-lane part of the transpose-read address in a ring tile (see v_operand_ptr for which element
// ends up where): lane s of a 16-lane group points at row key0 + s / 4, halves 4 (s % 4) ... of the
// 32-byte span that starts at column 2 * ((lane / 16) % 2); head-dim block db adds 4 db columns.
__device__ __forceinline__ const _Float16* v_ring_ptr(const _Float16* vs, int sub, int lane) {
    const int s16 = lane & 15;
    return vs + (2 * ((lane >> 4) & 1) + ((s16 & 3) >> 1)) * kColStride +
           (sub * 32 + 4 * (lane >> 5) + (s16 >> 2)) * 8 + 4 * (s16 & 1);
}

template <int H, int NQB>
constexpr int lds_bytes_pingpong() {
    return 3 * (ring_tile_k<H>() + ring_tile_v<H>()) * (int)sizeof(_Float16);
}

// Additive-mask variant of the ping-pong kernel: behind the rings every wave has a private slab
// for the mask values of its 32 NQB queries and the 32 keys of one sub-tile (row stride
// kMaskSubStr halves: 64 bytes of mask plus 16 of padding).
constexpr int kMaskSubStr = 40;
template <int H, int NW, int NQB>
constexpr int lds_bytes_pingpong_masked() {
    return lds_bytes_pingpong<H, NQB>() + NW * 32 * NQB * kMaskSubStr * (int)sizeof(_Float16);
}

// Barrier between the phases of the ping-pong kernel.  It does not wait for the wave's own LDS
// reads: nothing is handed from wave to wave through LDS stores (the rings are written by
// direct-to-LDS loads, which their issuer waits for with vmcnt), and every read of a ring slot is
// consumed by a matrix instruction at least one barrier before the loads that overwrite the slot
// are issued.  The scheduling barriers keep the compiler from moving matrix or vector
// instructions of one phase into the next.
__device__ __forceinline__ void ring_barrier() {
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
}

// One group's share of a 64-key ring tile, fetched straight into LDS.  Wave w of the group (NWG
// waves) owns the columns w * NP ... w * NP + NP - 1; lane l fetches the 16 bytes of key row l.
// Rows at or beyond L are read from row L - 1 instead: their scores are masked to -inf, or belong
// to sub-tiles that are never consumed, and a probability of exactly zero times a finite V row
// contributes nothing.  Tiles starting at or beyond `limit` are not fetched at all (limit <= L).
// The loads are asynchronous: the issuing wave waits for vmcnt before the barrier that hands the
// tile to its readers.
template <int H, int NWG>
struct RingLoader {
    static constexpr int CPR = H / 8;
    static constexpr int NP = (CPR + NWG - 1) / NWG;
    int col0;
    uint32_t lane_off;   // byte offset of this lane's row inside a full tile

    __device__ __forceinline__ void init(int wave_in_group, int64_t stride_l, int lane) {
        col0 = wave_in_group * NP;
        lane_off = (uint32_t)lane * (uint32_t)stride_l * 2u;
    }
    // The load is written in assembly so that the compiler does not see an LDS write: it would
    // otherwise wait for the load before the next LDS read of the wave.  M0 holds the LDS address
    // of lane 0's 16 bytes; lane l lands 16 l bytes further on.
    static __device__ __forceinline__ void dma16(uint32_t lds_addr, const _Float16* base, uint32_t voff) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                     :: "s"(lds_addr), "v"(voff), "s"(base) : "memory", "m0");
    }
    __device__ __forceinline__ void issue(const _Float16* src, int64_t stride_l, int key0, int limit, int L,
                                          _Float16* tile, int lane) const {
        issue_at(src + (int64_t)key0 * stride_l + col0 * 8, stride_l, key0, limit, L, tile, lane);
    }
    // `base` = src + key0 * stride_l + 8 * col0, kept by callers that walk the tiles in order
    __device__ __forceinline__ void issue_at(const _Float16* base, int64_t stride_l, int key0, int limit, int L,
                                             _Float16* tile, int lane) const {
        if (key0 >= limit) return;
        uint32_t voff = lane_off;
        if (key0 + 64 > L) voff = (uint32_t)(min(key0 + lane, L - 1) - key0) * (uint32_t)stride_l * 2u;
        const uint32_t lds0 = (uint32_t)(uintptr_t)(FA_LDS void*)tile + (uint32_t)col0 * (kColStride * 2);
#pragma unroll
        for (int i = 0; i < NP; ++i)
            if (CPR % NWG == 0 || col0 + i < CPR) dma16(lds0 + i * (kColStride * 2), base + i * 8, voff);
    }
};

__device__ __forceinline__ void wait_ring_loads() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

}  // namespace fa

// The kernels proper are written once and compiled for both element types: fp16 in namespace fa,
// bf16 in namespace fa::bf16.  All 16-bit data travel as bit patterns (half8 / u32x4 registers,
// _Float16 pointers for address arithmetic); only the few operations that interpret them differ.
#define FA_ELEM_BF16 0
#include "fused_attn_kernel_impl.inc"
#undef FA_ELEM_BF16
#define FA_ELEM_BF16 1
#include "fused_attn_kernel_impl.inc"
#undef FA_ELEM_BF16
