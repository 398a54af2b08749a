// C ABI of libfused_attn_gfx950.so: argument validation, launch geometry and the launch
// itself.  Host counterpart of launch_attention_kernel (reference
// include/fused_attn.cuh:860-894): picks the workgroup shape, sizes the dynamic LDS block,
// builds the grid and launches on the caller's stream.
#include "fused_attn_kernel.hpp"
#include "qkv_proj_kernel.hpp"

#include "../../include/fused_attn.h"

#include <mutex>
#include <utility>
#include <vector>

namespace {

constexpr int kKeyTile = 64;     // keys per LDS tile
constexpr int kNumCu = 256;      // compute units of one MI355X

// Launch shape: wave64s per workgroup and blocks of 32 query rows per wave.
struct Shape {
    int waves;
    int nqb;
    int rows() const { return waves * 32 * nqb; }
};

// Three shapes, picked by how the problem's workgroups fill the 256 compute units:
//   {8, 2}  eight 64-row waves share one K/V stream, run by the ping-pong kernel, 512 queries per
//           workgroup, one resident per compute unit (head_dim <= 64 only: with head_dim 128 a
//           64-row wave would need the whole register file of a SIMD);
//   {8, 1}  the same kernel with 32-row waves, 256 queries per workgroup: the only ping-pong
//           shape of head_dim 128 (one resident per compute unit); with head_dim <= 64 it serves
//           the grids that {8, 2} fills badly (without mask two are resident per compute unit;
//           the causal and the additive-mask variants do not fit 128 registers and run one);
//   {4, 1}  four 32-row waves, 128 queries per workgroup, three (head_dim <= 64) or two
//           (head_dim 128) resident per compute unit: more, smaller workgroups for small problems.
int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// How well a shape uses the chip, in 1/1024: the share of the (rounds x slots) grid of resident
// workgroup slots that the problem's workgroups occupy, times the share of each workgroup's query
// rows that exist (the last workgroup of a sequence may be mostly empty).
int64_t usage(int64_t heads, int64_t L, int64_t rows, int64_t slots) {
    const int64_t per_head = ceil_div(L, rows);
    const int64_t wgs = heads * per_head;
    // in floating point: the products overflow 64 bits for the largest accepted shapes
    const double filled = (double)wgs / ((double)ceil_div(wgs, slots) * (double)slots);
    const double rows_used = (double)L / ((double)per_head * (double)rows);
    return (int64_t)(1024.0 * filled * rows_used);
}

// Causal launches of the eight-wave kernel.  Query tile t of a head costs t + 1 key blocks.  The
// plain schedule gives every workgroup the pair (t, n - 1 - t), n + 1 blocks, and the grid runs
// ceil(pairs / 256) rounds of them; a last round that is mostly empty costs as much as a full one,
// and in a lone part-filled round the idle compute units could have taken the small tiles.
// The dealt schedule (kernel: p.heads_per_xcd > 0) keeps 32 workgroups resident per XCD and deals
// the tiles of the XCD's heads out in descending cost, serpentine over the workgroups; it needs
// B * R to be a multiple of 8 so that the XCDs carry equal loads.  Time in key blocks of the
// busiest workgroup under either schedule; the dealt one is taken when it saves 8 % or more
// (measured: 5 to 17 % faster then, against 11 to 28 % fewer blocks).
struct CausalPlan {
    bool dealt;
    int64_t blocks;       // key blocks the busiest workgroup walks through
};

CausalPlan plan_causal_walk(int64_t heads, int64_t n, int64_t H);

// One causal launch asks for its plan twice (shape choice, then grid), and a serving loop asks for
// the same few plans over and over: the last results are kept per host thread.
CausalPlan plan_causal(int64_t heads, int64_t n, int64_t H) {
    struct Entry {
        int64_t heads, n, H;
        CausalPlan plan;
    };
    constexpr int kEntries = 8;
    thread_local Entry cache[kEntries] = {};
    thread_local int next = 0;
    for (const Entry& e : cache)
        if (e.heads == heads && e.n == n && e.H == H) return e.plan;
    const CausalPlan plan = plan_causal_walk(heads, n, H);
    cache[next] = Entry{heads, n, H, plan};
    next = (next + 1) % kEntries;
    return plan;
}

CausalPlan plan_causal_walk(int64_t heads, int64_t n, int64_t H) {
    const int64_t pairs = heads * ceil_div(n, 2);
    const CausalPlan paired{false, ceil_div(pairs, kNumCu) * (n + 1)};
    constexpr int kPerXcd = kNumCu / fa::kNumXcd;
    // head_dim below 64: dealing the tiles out spreads an XCD's workgroups over more heads at a
    // time than its L2 holds K and V for, and measures slower than the part-filled round
    if (H < 64 || heads % fa::kNumXcd != 0) return paired;
    const int64_t hx = heads / fa::kNumXcd;
    const int64_t items = hx * n;
    if (items > (int64_t)1 << 22) return paired;     // the walk below is linear in the items
    int64_t load[kPerXcd] = {};
    for (int64_t j0 = 0, round = 0; j0 < items; j0 += kPerXcd, ++round)
        for (int w = 0; w < kPerXcd; ++w) {
            const int64_t j = j0 + ((round & 1) ? kPerXcd - 1 - w : w);
            if (j < items) load[w] += n - j / hx;
        }
    int64_t worst = 0;
    for (int w = 0; w < kPerXcd; ++w) worst = load[w] > worst ? load[w] : worst;
    return worst * 100 <= paired.blocks * 92 ? CausalPlan{true, worst} : paired;
}

// mask_rows_aligned: an additive mask whose rows are 16-byte aligned (L % 8 == 0, aligned pointer).
Shape pick_shape(int64_t B, int64_t R, int64_t L, int64_t H, bool has_mask, bool mask_rows_aligned,
                 bool causal) {
    const int64_t heads = B * R;
    // The ping-pong kernel takes an additive mask only through its coalesced, LDS-staged fetch;
    // any other mask goes to four 32-row waves (the mask staging registers and LDS slabs leave room
    // for two such workgroups per compute unit, not for 64-row waves).
    if (has_mask && !mask_rows_aligned) return {4, 1};
    // The ping-pong kernel is the fastest per compute unit, so it is taken whenever its
    // workgroups fill the chip well enough.  Thresholds measured on MI355X: a lone round may be
    // emptier than the tail of several, because idle units leave the busy ones more of the
    // power budget.  A causal ping-pong workgroup takes two query tiles (see the kernel).
    const int64_t tile8 = H > 64 ? 256 : 512;
    const int64_t rows8 = tile8 * (causal ? 2 : 1);
    const int64_t wgs8 = heads * ceil_div(L, rows8);
    int64_t usage8 = usage(heads, L, rows8, kNumCu);
    if (causal) {
        // with the dealt schedule: useful key blocks over the blocks the 256 compute units are held for
        const int64_t n = ceil_div(L, tile8);
        const CausalPlan plan = plan_causal(heads, n, H);
        if (plan.dealt) {
            const double held = (double)plan.blocks * kNumCu;
            const double useful = (double)heads * (double)n * (double)(n + 1) / 2.0;
            const double rows_used = (double)L / ((double)n * (double)tile8);
            if (1024.0 * useful / held * rows_used >= 614.0) return H > 64 ? Shape{8, 1} : Shape{8, 2};
        }
    }
    // Usage of 0.55 in a lone round, 0.7 in a part-filled second round, 0.6 from two rounds on.
    const bool pingpong = wgs8 >= 2 * kNumCu ? usage8 >= 614 : usage8 >= (wgs8 <= kNumCu ? 560 : 717);
    // 256-query workgroups with an additive mask: up to 30 % faster than the four-wave kernel,
    // whose masked loop is not pipelined, from 160 workgroups on, unless a quarter or more of the
    // query rows of a head's workgroups do not exist.
    const int64_t per_head = ceil_div(L, 256);
    const bool masked81 = has_mask && heads * per_head >= 160 && 4 * L >= 3 * per_head * 256;
    if (H > 64) return pingpong || masked81 ? Shape{8, 1} : Shape{4, 1};
    if (pingpong) return {8, 2};
    // 256-query ping-pong workgroups.  Thresholds from sweeps of mid-size shapes on MI355X.
    // Causal (a workgroup takes a pair of 256-query tiles, one resident per compute unit): 4 to
    // 21 % faster than the four-wave kernel when the pairs fill 55 % or more of a single round,
    // slower on emptier or on several rounds.
    if (causal)
        return heads * ceil_div(L, 512) <= kNumCu && usage(heads, L, 512, kNumCu) >= 560 ? Shape{8, 1} : Shape{4, 1};
    // Additive mask: one resident per compute unit.
    if (has_mask) return masked81 ? Shape{8, 1} : Shape{4, 1};
    // Plain, two per compute unit: per compute unit they run at 0.93 of the 512-query ones and
    // 1.1 to 1.25 times as fast as the four-wave kernel, but they need 160 or more workgroups to
    // beat the latter's finer grain.
    return heads * per_head >= 160 ? Shape{8, 1} : Shape{4, 1};
}

// Dynamic LDS above 64 KiB has to be opted into per kernel function and per device: done on the
// first launch of that kernel on that device.
hipError_t allow_large_lds(const void* kernel, int bytes) {
    static std::mutex lock;
    static std::vector<std::pair<const void*, int>> done;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    std::lock_guard<std::mutex> guard(lock);
    for (const auto& d : done)
        if (d.first == kernel && d.second == dev) return hipSuccess;
    e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e == hipSuccess) done.emplace_back(kernel, dev);
    return e;
}

// BF selects the bf16 instantiation (namespace fa::bf16) of the same kernel source.
template <int H, int NW, int NQB, int WPE, int MODE, bool BF>
hipError_t launch(const fa::FwdParams& p, hipStream_t stream) {
    constexpr int lds = MODE == fa::kAdditive ? fa::lds_bytes_masked<H, NW, kKeyTile, NQB>() : fa::lds_bytes<H, NW, kKeyTile>();
    auto kernel = BF ? fa::bf16::fwd_kernel<H, NW, kKeyTile, NQB, WPE, MODE> : fa::fwd_kernel<H, NW, kKeyTile, NQB, WPE, MODE>;
    if constexpr (lds > 64 * 1024) {
        const hipError_t e = allow_large_lds(reinterpret_cast<const void*>(kernel), lds);
        if (e != hipSuccess) return e;
    }
    const int grid = p.wgs_per_xcd * fa::kNumXcd;
    // the launch's own status, not the thread's sticky last error (which may stem from the caller's code)
    fa::FwdParams params = p;
    void* args[] = {&params};
    return hipLaunchKernel(reinterpret_cast<const void*>(kernel), dim3(grid), dim3(NW * 64), args, lds, stream);
}

template <int H, int NW, int NQB, int WPE, int MODE, bool BF>
hipError_t launch_pingpong(const fa::FwdParams& p, hipStream_t stream) {
    constexpr int lds = MODE == fa::kAdditive ? fa::lds_bytes_pingpong_masked<H, NW, NQB>() : fa::lds_bytes_pingpong<H, NQB>();
    auto kernel = BF ? fa::bf16::fwd_kernel_pingpong<H, NW, NQB, WPE, MODE> : fa::fwd_kernel_pingpong<H, NW, NQB, WPE, MODE>;
    if constexpr (lds > 64 * 1024) {
        const hipError_t e = allow_large_lds(reinterpret_cast<const void*>(kernel), lds);
        if (e != hipSuccess) return e;
    }
    const int grid = p.wgs_per_xcd * fa::kNumXcd;
    // the launch's own status, not the thread's sticky last error (which may stem from the caller's code)
    fa::FwdParams params = p;
    void* args[] = {&params};
    return hipLaunchKernel(reinterpret_cast<const void*>(kernel), dim3(grid), dim3(NW * 64), args, lds, stream);
}

// The eight-wave kernel with its products written as 16 x 16 tiles (fwd_kernel_pp16), head_dim 64
// (64-row waves) and 128 (32-row waves).
// Plain launches: on a full chip the clock follows the switching activity and the 16 x 16 x 32
// instruction moves half as many accumulator registers per flop; where part of the chip idles the
// clock is not held back and its 36 (34) matrix instructions per sub-tile instead of 20 (18) cost
// more than they save, and a part-filled last round takes that from the whole launch.  Measured on
// the same box, by workgroups, head_dim 64: 256 +2.9 and +3.6 %, 480 +1.1 %, 512 +3.5 %; 192 -5 to
// -9 %, 384 -3.4 and -4.6 %, 448 -0.7 %, 640 -1.0 %, 1152 -0.8 %.  head_dim 128: 224 +3.4 %, 256
// +3.1 %, 480 +2.5 %, 512 +2.1 %, 1280 +3.1 %, 2048 +5.2 %; 192 -0.3 %, 384 -2.0 %, 448 +1.3 %, 640
// -0.9 %, 800 -0.2 %, 1088 +0.1 %, 1600 -0.9 %.  Taken when the last round is at least seven
// eighths full.
// Causal launches in pairs of tiles or dealt out: there the gain is the kernel's deal of 16-query
// blocks to the waves, which does not depend on the clock, and only an emptier single round loses
// (head_dim 64: 144 pairs -4.3 %, 160 -6.2 %, 192 -1.4 and +1.3 %, 200 -0.6 %; 240 +3.6 %, 256
// +5.5 %, 400 +1.4 %, 960 +4.5 and +7.5 %, 1152 +5.4 %, dealt +3.2 to +4.7 %; head_dim 128: 1024
// pairs +5.1 and +5.4 %, dealt +4.2 %): taken from seven eighths of a round on.
bool use_tiles16(int64_t H, Shape sh, const fa::FwdParams& p, bool causal) {
    if (sh.waves != 8 || !((H == 64 && sh.nqb == 2) || H == 128)) return false;
    if (8 * (int64_t)p.total_wgs < 7 * kNumCu) return false;
    if (causal) return true;            // (a dealt launch is a whole resident grid)
    if (H == 64 && p.total_wgs < kNumCu) return false;     // (224 and 240 workgroups: +1.6 and +2.5 % at L = 4096, -1.4 % at L = 1024)
    const int last = p.total_wgs % kNumCu;
    return last == 0 || 8 * last >= 7 * kNumCu;
}

template <int H, bool BF, int MODE>
hipError_t launch_pp16(const fa::FwdParams& p, hipStream_t stream) {
    constexpr int lds = fa::lds_bytes_pingpong<H, 2>();
    auto kernel = BF ? fa::bf16::fwd_kernel_pp16<H, 8, true, MODE> : fa::fwd_kernel_pp16<H, 8, true, MODE>;
    if constexpr (lds > 64 * 1024) {
        const hipError_t e = allow_large_lds(reinterpret_cast<const void*>(kernel), lds);
        if (e != hipSuccess) return e;
    }
    fa::FwdParams params = p;
    void* args[] = {&params};
    return hipLaunchKernel(reinterpret_cast<const void*>(kernel), dim3(p.wgs_per_xcd * fa::kNumXcd), dim3(8 * 64), args,
                           lds, stream);
}

template <int H, bool BF>
hipError_t launch_pp16_mode(int mode, const fa::FwdParams& p, hipStream_t stream) {
    switch (mode) {
        case fa::kPlain: return launch_pp16<H, BF, fa::kPlain>(p, stream);
        case fa::kCausal: return launch_pp16<H, BF, fa::kCausal>(p, stream);
        case fa::kCausalDealt: return launch_pp16<H, BF, fa::kCausalDealt>(p, stream);
        default: return hipErrorInvalidValue;
    }
}

hipError_t launch_tiles16(int64_t H, int mode, bool bf16, const fa::FwdParams& p, hipStream_t stream) {
    if (H == 64) return bf16 ? launch_pp16_mode<64, true>(mode, p, stream) : launch_pp16_mode<64, false>(mode, p, stream);
    if (H == 128) return bf16 ? launch_pp16_mode<128, true>(mode, p, stream) : launch_pp16_mode<128, false>(mode, p, stream);
    return hipErrorInvalidValue;
}

template <int H, int MODE, bool BF>
hipError_t dispatch_shape(Shape sh, const fa::FwdParams& p, hipStream_t stream) {
    // the dealt causal schedule exists for the eight-wave kernel at head_dim 64 and 128 only
    // (plan_causal never asks for it elsewhere)
    constexpr int BASE = MODE == fa::kCausalDealt ? fa::kCausal : MODE;
    if (MODE == fa::kCausalDealt && (sh.waves != 8 || H < 64)) return hipErrorInvalidValue;
    // the ping-pong kernel for the eight-wave shapes
    if (sh.waves == 8) {
        if constexpr (H > 64)
            return launch_pingpong<H, 8, 1, 2, MODE, BF>(p, stream);
        else if (sh.nqb == 2)
            return launch_pingpong<H, 8, 2, 2, H < 64 ? BASE : MODE, BF>(p, stream);
        else if constexpr (MODE == fa::kPlain)
            return launch_pingpong<H, 8, 1, 4, MODE, BF>(p, stream);
        else
            return launch_pingpong<H, 8, 1, 2, H < 64 ? BASE : MODE, BF>(p, stream);
    }
    // four 32-row waves; three per SIMD where the registers allow it
    if constexpr (H > 64 || MODE == fa::kAdditive)
        return launch<H, 4, 1, 2, BASE, BF>(p, stream);
    else
        return launch<H, 4, 1, 3, BASE, BF>(p, stream);
}

template <int MODE, bool BF>
hipError_t dispatch_head_dim(int64_t H, Shape sh, const fa::FwdParams& p, hipStream_t stream) {
    switch (H) {
        case 16: return dispatch_shape<16, MODE, BF>(sh, p, stream);
        case 32: return dispatch_shape<32, MODE, BF>(sh, p, stream);
        case 64: return dispatch_shape<64, MODE, BF>(sh, p, stream);
        case 128: return dispatch_shape<128, MODE, BF>(sh, p, stream);
        default: return hipErrorInvalidValue;
    }
}

template <int MODE>
hipError_t dispatch(int64_t H, Shape sh, const fa::FwdParams& p, hipStream_t stream, bool bf16) {
    return bf16 ? dispatch_head_dim<MODE, true>(H, sh, p, stream) : dispatch_head_dim<MODE, false>(H, sh, p, stream);
}

bool aligned16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0; }

struct Strides {
    int64_t b, h, l;
};

bool strides_ok(const Strides& s, int64_t H) {
    return s.l >= H && s.h >= 0 && s.b >= 0 && (s.l % 8) == 0 && (s.h % 8) == 0 && (s.b % 8) == 0;
}

bool extent_ok(const Strides& s, int64_t B, int64_t R, int64_t L) {
    constexpr int64_t kMaxElems = (int64_t)1 << 62;
    return !(L > kMaxElems / s.l || (s.h > 0 && R > kMaxElems / s.h) || (s.b > 0 && B > kMaxElems / s.b));
}

int validate(const void* q, const void* k, const void* v, const void* mask, void* out, int64_t B,
             int64_t R, int64_t L, int64_t H, const Strides& in, const Strides& os,
             fa::FwdParams* p, float scale, Shape* shape, bool causal, void* lse) {
    const int64_t stride_b = in.b, stride_h = in.h, stride_l = in.l;
    if (q == nullptr || k == nullptr || v == nullptr || out == nullptr) return FA_ERR_NULL_POINTER;
    if (!fa_fwd_query(H)) return FA_ERR_BAD_HEAD_DIM;
    if (B < 1 || R < 1 || L < 1) return FA_ERR_BAD_SHAPE;
    // the kernels track the row maximum of the raw scores, which is the maximum of the scaled ones
    // only for a positive scale, and they divide the additive mask by the scale
    if (!(scale > 0.f) || scale > 3.0e38f) return FA_ERR_BAD_SCALE;
    if (!strides_ok(in, H) || !strides_ok(os, H)) return FA_ERR_BAD_STRIDE;
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(out)) return FA_ERR_MISALIGNED;
    if (mask != nullptr && (reinterpret_cast<uintptr_t>(mask) & 1u) != 0) return FA_ERR_MISALIGNED;
    constexpr int64_t kMaxInt = 0x7fffffff;
    if (L > kMaxInt - 4096 || B > kMaxInt || R > kMaxInt || B * R > kMaxInt) return FA_ERR_TOO_LARGE;
    // the tile loaders keep 32-bit byte offsets inside a 64-key tile
    if (stride_l > ((int64_t)1 << 24)) return FA_ERR_TOO_LARGE;
    // (the eight-wave kernel keeps 32-bit byte offsets inside the 64 mask rows of a wave)
    *shape = pick_shape(B, R, L, H, mask != nullptr,
                        (L % 8) == 0 && L <= ((int64_t)1 << 24) && (reinterpret_cast<uintptr_t>(mask) & 15u) == 0, causal);
    const int64_t bq = shape->rows();
    int64_t n_qtiles = (L + bq - 1) / bq;
    int64_t total = 0;
    p->heads_per_xcd = 0;
    if (causal && shape->waves == 8) {
        const CausalPlan plan = plan_causal(B * R, n_qtiles, H);
        n_qtiles = (n_qtiles + 1) / 2;                                // pairs of query tiles
        if (plan.dealt) {
            p->heads_per_xcd = (int)(B * R / fa::kNumXcd);
            total = kNumCu;                                           // a resident grid
        }
    }
    if (mask != nullptr && shape->waves == 8 && n_qtiles > 1) {
        // Pairs of query tiles for a masked launch of the eight-wave kernel (see the kernel) when the
        // pairs, two tiles long, need no more time on the chip than the tiles in rounds of their own
        const int64_t pairs = (n_qtiles + 1) / 2;
        if (2 * ceil_div(B * R * pairs, kNumCu) <= ceil_div(B * R * n_qtiles, kNumCu)) n_qtiles = pairs;
    }
    if (total == 0) total = B * R * n_qtiles;
    if (total > kMaxInt - 8 || B * R > kMaxInt) return FA_ERR_TOO_LARGE;
    if (!extent_ok(in, B, R, L) || !extent_ok(os, B, R, L)) return FA_ERR_TOO_LARGE;

    p->q = static_cast<const _Float16*>(q);
    p->k = static_cast<const _Float16*>(k);
    p->v = static_cast<const _Float16*>(v);
    p->mask = static_cast<const _Float16*>(mask);
    p->o = static_cast<_Float16*>(out);
    p->lse = static_cast<float*>(lse);
    p->stride_b = stride_b;
    p->stride_h = stride_h;
    p->stride_l = stride_l;
    p->ostride_b = os.b;
    p->ostride_h = os.h;
    p->ostride_l = os.l;
    p->B = (int)B;
    p->R = (int)R;
    p->L = (int)L;
    p->n_qtiles = (int)n_qtiles;
    p->total_wgs = (int)total;
    p->wgs_per_xcd = (int)((total + fa::kNumXcd - 1) / fa::kNumXcd);
    p->scale_log2e = scale * 1.4426950408889634f;
    p->bias = fa_fwd_reference_bias(L);
    return FA_OK;
}

}  // namespace

extern "C" {

int fa_fwd_query(int64_t H) { return (H == 16 || H == 32 || H == 64 || H == 128) ? 1 : 0; }

// 11 - ceil(log2 L): a tail of L small weights then loses at most 2^-13 of a row (see kBiasMin)
float fa_fwd_reference_bias(int64_t L) {
    int log2_len = 0;
    while (log2_len < 62 && ((int64_t)1 << log2_len) < L) ++log2_len;
    const float bias = 11.0f - (float)log2_len;
    return bias < fa::kBiasMin ? fa::kBiasMin : (bias > fa::kBiasMax ? fa::kBiasMax : bias);
}

const char* fa_strerror(int status) {
    switch (status) {
        case FA_OK: return "success";
        case FA_ERR_NULL_POINTER: return "fa_fwd: q, k, v and out must be non-null device pointers";
        case FA_ERR_BAD_HEAD_DIM: return "fa_fwd: head_dim must be 16, 32, 64 or 128";
        case FA_ERR_BAD_SHAPE:
            return "fa_fwd: B, R and L must be at least 1 (fa_qkv_proj: and the feature counts multiples of 64)";
        case FA_ERR_BAD_STRIDE:
            return "fa_fwd: strides must be non-negative multiples of 8 elements and stride_l >= head_dim";
        case FA_ERR_MISALIGNED: return "fa_fwd: q, k, v and out must be 16-byte aligned";
        case FA_ERR_TOO_LARGE: return "fa_fwd: problem size exceeds the supported index range";
        case FA_ERR_BAD_FLAGS: return "fa_fwd_ex: unknown flag, or FA_FLAG_CAUSAL together with a mask";
        case FA_ERR_BAD_SCALE: return "fa_fwd: scale must be finite and positive";
        default: break;
    }
    if (status > 0) return hipGetErrorString(static_cast<hipError_t>(status));
    return "fa_fwd: unknown status";
}

int fa_fwd_strided(const void* q, const void* k, const void* v, const void* mask, void* out, void* lse,
                   int64_t B, int64_t R, int64_t L, int64_t H, int64_t stride_b, int64_t stride_h,
                   int64_t stride_l, int64_t out_stride_b, int64_t out_stride_h, int64_t out_stride_l,
                   float scale, int flags, void* stream) {
    if ((flags & ~(FA_FLAG_CAUSAL | FA_FLAG_BF16)) != 0) return FA_ERR_BAD_FLAGS;
    const bool causal = (flags & FA_FLAG_CAUSAL) != 0;
    const bool bf16 = (flags & FA_FLAG_BF16) != 0;
    if (causal && mask != nullptr) return FA_ERR_BAD_FLAGS;
    if (lse != nullptr && (reinterpret_cast<uintptr_t>(lse) & 3u) != 0) return FA_ERR_MISALIGNED;
    fa::FwdParams p;
    Shape shape{4, 2};
    const int rc = validate(q, k, v, mask, out, B, R, L, H, Strides{stride_b, stride_h, stride_l},
                            Strides{out_stride_b, out_stride_h, out_stride_l}, &p, scale, &shape, causal, lse);
    if (rc != FA_OK) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipError_t e;
    if (mask == nullptr && use_tiles16(H, shape, p, causal))
        e = launch_tiles16(H, causal ? (p.heads_per_xcd > 0 ? fa::kCausalDealt : fa::kCausal) : fa::kPlain, bf16, p, s);
    else if (causal && p.heads_per_xcd > 0)
        e = dispatch<fa::kCausalDealt>(H, shape, p, s, bf16);
    else if (causal)
        e = dispatch<fa::kCausal>(H, shape, p, s, bf16);
    else if (mask != nullptr)
        e = dispatch<fa::kAdditive>(H, shape, p, s, bf16);
    else
        e = dispatch<fa::kPlain>(H, shape, p, s, bf16);
    return static_cast<int>(e);
}

int fa_fwd_plan(int64_t B, int64_t R, int64_t L, int64_t H, int flags, int has_mask, int* plan) {
    if (plan == nullptr) return FA_ERR_NULL_POINTER;
    if ((flags & ~(FA_FLAG_CAUSAL | FA_FLAG_BF16)) != 0) return FA_ERR_BAD_FLAGS;
    const bool causal = (flags & FA_FLAG_CAUSAL) != 0;
    if (causal && has_mask) return FA_ERR_BAD_FLAGS;
    // validate() only looks at the pointers' alignment
    void* const fake = reinterpret_cast<void*>(static_cast<uintptr_t>(4096));
    fa::FwdParams p;
    Shape shape{4, 1};
    const Strides dense{L * R * H, H, R * H};
    const int rc = validate(fake, fake, fake, has_mask ? fake : nullptr, fake, B, R, L, H, dense, dense, &p, 1.0f,
                            &shape, causal, nullptr);
    if (rc != FA_OK) return rc;
    plan[0] = shape.waves;
    plan[1] = 32 * shape.nqb;
    plan[2] = p.wgs_per_xcd * fa::kNumXcd;
    plan[3] = p.total_wgs;
    plan[4] = p.n_qtiles;
    plan[5] = p.heads_per_xcd;
    plan[6] = (!has_mask && use_tiles16(H, shape, p, causal)) ? 16 : 32;
    return FA_OK;
}

int fa_fwd_ex(const void* q, const void* k, const void* v, const void* mask, void* out, void* lse,
              int64_t B, int64_t R, int64_t L, int64_t H, int64_t stride_b, int64_t stride_h,
              int64_t stride_l, float scale, int flags, void* stream) {
    return fa_fwd_strided(q, k, v, mask, out, lse, B, R, L, H, stride_b, stride_h, stride_l, stride_b, stride_h,
                          stride_l, scale, flags, stream);
}

int fa_fwd(const void* q, const void* k, const void* v, const void* mask, void* out, int64_t B,
           int64_t R, int64_t L, int64_t H, int64_t stride_b, int64_t stride_h, int64_t stride_l,
           float scale, void* stream) {
    return fa_fwd_ex(q, k, v, mask, out, nullptr, B, R, L, H, stride_b, stride_h, stride_l, scale, 0,
                     stream);
}

int fa_fwd_timed_ex(const void* q, const void* k, const void* v, const void* mask, void* out, void* lse,
                    int64_t B, int64_t R, int64_t L, int64_t H, int64_t stride_b, int64_t stride_h,
                    int64_t stride_l, int64_t out_stride_b, int64_t out_stride_h, int64_t out_stride_l,
                    float scale, int flags, void* stream, int iters, float* ms_per_launch) {
    if (ms_per_launch == nullptr) return FA_ERR_NULL_POINTER;
    if (iters < 1) return FA_ERR_BAD_SHAPE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipEvent_t e0 = nullptr, e1 = nullptr;
    hipError_t e = hipEventCreate(&e0);
    if (e != hipSuccess) return static_cast<int>(e);
    e = hipEventCreate(&e1);
    if (e != hipSuccess) {
        (void)hipEventDestroy(e0);
        return static_cast<int>(e);
    }
    int rc = FA_OK;
    e = hipEventRecord(e0, s);
    if (e != hipSuccess) rc = static_cast<int>(e);
    for (int i = 0; i < iters && rc == FA_OK; ++i)
        rc = fa_fwd_strided(q, k, v, mask, out, lse, B, R, L, H, stride_b, stride_h, stride_l, out_stride_b,
                            out_stride_h, out_stride_l, scale, flags, stream);
    if (rc == FA_OK) {
        e = hipEventRecord(e1, s);
        if (e == hipSuccess) e = hipEventSynchronize(e1);
        float ms = 0.f;
        if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
        if (e == hipSuccess)
            *ms_per_launch = ms / (float)iters;
        else
            rc = static_cast<int>(e);
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    return rc;
}

int fa_fwd_timed(const void* q, const void* k, const void* v, const void* mask, void* out, int64_t B,
                 int64_t R, int64_t L, int64_t H, int64_t stride_b, int64_t stride_h,
                 int64_t stride_l, float scale, void* stream, int iters, float* ms_per_launch) {
    return fa_fwd_timed_ex(q, k, v, mask, out, nullptr, B, R, L, H, stride_b, stride_h, stride_l, stride_b,
                           stride_h, stride_l, scale, 0, stream, iters, ms_per_launch);
}

}  // extern "C"

namespace {
template <int HR, bool BF>
hipError_t launch_qkv(const fa::qkv::Params& p, hipStream_t stream) {
    auto kernel = fa::qkv::qkv_proj_kernel<HR, BF>;
    constexpr int kQkvLds = fa::qkv::kLdsBytes;
    constexpr int kQkvThreads = fa::qkv::kWaves * 64;
    const hipError_t e = allow_large_lds(reinterpret_cast<const void*>(kernel), kQkvLds);
    if (e != hipSuccess) return e;
    fa::qkv::Params params = p;
    void* args[] = {&params};
    return hipLaunchKernel(reinterpret_cast<const void*>(kernel), dim3(p.wgs_per_xcd * fa::kNumXcd),
                           dim3(kQkvThreads), args, kQkvLds, stream);
}

// Tiles and grid of the projection kernel for an M x N output.
int qkv_geometry(int64_t M, int64_t N, fa::qkv::Params* p) {
    constexpr int64_t kMaxInt = 0x7fffffff;
    const int64_t tiles_m = ceil_div(M, fa::qkv::kTileM);
    p->tiles_n = (int)ceil_div(N, fa::qkv::kTileN);
    if (tiles_m * p->tiles_n > kMaxInt - 8) return FA_ERR_TOO_LARGE;
    p->total_tiles = (int)(tiles_m * p->tiles_n);
    // a resident grid, one workgroup per compute unit, each walking through its share of the tiles
    p->total_wgs = p->total_tiles < kNumCu ? p->total_tiles : kNumCu;
    p->wgs_per_xcd = (int)ceil_div(p->total_wgs, fa::kNumXcd);
    return FA_OK;
}

template <bool BF>
hipError_t dispatch_qkv(int64_t rope_head_dim, const fa::qkv::Params& p, hipStream_t stream) {
    switch (rope_head_dim) {
        case 0: return launch_qkv<0, BF>(p, stream);
        case 16: return launch_qkv<16, BF>(p, stream);
        case 32: return launch_qkv<32, BF>(p, stream);
        case 64: return launch_qkv<64, BF>(p, stream);
        case 128: return launch_qkv<128, BF>(p, stream);
        default: return hipErrorInvalidValue;
    }
}
}  // namespace

extern "C" {

int fa_qkv_proj(const void* x, const void* w, const void* bias, void* qkv, int64_t B, int64_t L, int64_t F_in,
                int64_t R, int64_t H, const float* rope_cos, const float* rope_sin, int flags, void* stream) {
    if ((flags & ~FA_FLAG_BF16) != 0) return FA_ERR_BAD_FLAGS;
    if (x == nullptr || w == nullptr || qkv == nullptr) return FA_ERR_NULL_POINTER;
    if ((rope_cos == nullptr) != (rope_sin == nullptr)) return FA_ERR_NULL_POINTER;
    if (!fa_fwd_query(H)) return FA_ERR_BAD_HEAD_DIM;
    if (B < 1 || L < 1 || R < 1 || F_in < 1) return FA_ERR_BAD_SHAPE;
    constexpr int64_t kMaxInt = 0x7fffffff;
    if (B > kMaxInt || L > kMaxInt || R > kMaxInt || B * L > kMaxInt - 2 * fa::qkv::kTileM) return FA_ERR_TOO_LARGE;
    const int64_t F = R * H;
    // the contraction is walked in whole steps of 64, and the three slices start on 64-feature boundaries
    if (F_in % fa::qkv::kTileK != 0 || F % 64 != 0) return FA_ERR_BAD_SHAPE;
    // the loaders keep 32-bit byte offsets inside a tile: 256 rows of x, 64 rows of w
    if (F_in > ((int64_t)1 << 22) || F > ((int64_t)1 << 22)) return FA_ERR_TOO_LARGE;
    if (!aligned16(x) || !aligned16(w) || !aligned16(qkv) || !aligned16(rope_cos) || !aligned16(rope_sin) ||
        (reinterpret_cast<uintptr_t>(bias) & 7u) != 0)
        return FA_ERR_MISALIGNED;
    fa::qkv::Params p;
    p.x = static_cast<const _Float16*>(x);
    p.w = static_cast<const _Float16*>(w);
    p.bias = static_cast<const _Float16*>(bias);
    p.out = static_cast<_Float16*>(qkv);
    p.rope_cos = rope_cos;
    p.rope_sin = rope_sin;
    p.M = (int)(B * L);
    p.K = (int)F_in;
    p.N = (int)(3 * F);
    p.F = (int)F;
    p.L = (int)L;
    const int rc = qkv_geometry(B * L, 3 * F, &p);
    if (rc != FA_OK) return rc;
    const int64_t hr = rope_cos != nullptr ? H : 0;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const hipError_t e = (flags & FA_FLAG_BF16) != 0 ? dispatch_qkv<true>(hr, p, s) : dispatch_qkv<false>(hr, p, s);
    return static_cast<int>(e);
}

int fa_qkv_proj_plan(int64_t B, int64_t L, int64_t F_in, int64_t R, int64_t H, int* plan) {
    if (plan == nullptr) return FA_ERR_NULL_POINTER;
    if (!fa_fwd_query(H)) return FA_ERR_BAD_HEAD_DIM;
    if (B < 1 || L < 1 || R < 1 || F_in < 1) return FA_ERR_BAD_SHAPE;
    constexpr int64_t kMaxInt = 0x7fffffff;
    if (B > kMaxInt || L > kMaxInt || R > kMaxInt || B * L > kMaxInt - 2 * fa::qkv::kTileM) return FA_ERR_TOO_LARGE;
    const int64_t F = R * H;
    if (F_in % fa::qkv::kTileK != 0 || F % 64 != 0) return FA_ERR_BAD_SHAPE;
    if (F_in > ((int64_t)1 << 22) || F > ((int64_t)1 << 22)) return FA_ERR_TOO_LARGE;
    fa::qkv::Params p;
    const int rc = qkv_geometry(B * L, 3 * F, &p);
    if (rc != FA_OK) return rc;
    plan[0] = p.wgs_per_xcd * fa::kNumXcd;
    plan[1] = p.total_wgs;
    plan[2] = p.total_tiles;
    plan[3] = p.tiles_n;
    return FA_OK;
}

}  // extern "C"
