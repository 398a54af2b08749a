// Instruction-issue probes for gfx950, run as `fa_test issue-probe`: how matrix (MFMA) and vector
// (VALU) instructions of one or two waves on the same SIMD overlap.  The attention kernels are
// scheduled around these numbers.  A 512-thread workgroup places waves w and w + 4 on the same
// SIMD; all figures are shader clocks (s_memtime) per instruction or per group of instructions.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdio>

namespace probe {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f16v __attribute__((ext_vector_type(16)));

#define PROBE_OK(expr)                                                                        \
    do {                                                                                      \
        hipError_t e_ = (expr);                                                               \
        if (e_ != hipSuccess) {                                                               \
            std::fprintf(stderr, "%s failed: %s\n", #expr, hipGetErrorString(e_));            \
            return 2;                                                                         \
        }                                                                                     \
    } while (0)

#define P_FMA(d, s) asm volatile("v_fma_f32 %0, %1, %2, %3" : "=v"(d) : "v"(s), "v"(a), "v"(b))
#define P_EXP(d) asm volatile("v_exp_f32 %0, %0" : "+v"(d))
#define P_CVT(d, x, y) asm volatile("v_cvt_pkrtz_f16_f32 %0, %1, %2" : "=v"(d) : "v"(x), "v"(y))
#define P_DOT(acc, x) asm volatile("v_dot2c_f32_f16 %0, %1, %2" : "+v"(acc) : "v"(0x3c003c00u), "v"(x))
#define P_MFMA(c) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(c) : "v"(x), "v"(y))

// Probe 1: waves 0-3 issue MFMAs only, waves 4-7 (same SIMDs) one kind of vector instruction only.
// mode bit 0: matrix waves run, bit 1: vector waves run.  VK: 0 fma, 1 exp, 2 cvt_pkrtz, 3 dot2c.
template <int VK>
__global__ __launch_bounds__(512) void split_kernel(long long* out, const h8* data, int iters, int mode,
                                                    float a, float b) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    long long t0 = 0, t1 = 0;
    float sink = 0.f;
    if (wave < 4) {
        if (!(mode & 1)) return;
        const h8 x = data[threadIdx.x], y = data[threadIdx.x + 512];
        f16v c[4];
        for (int n = 0; n < 4; n++)
            for (int r = 0; r < 16; r++) c[n][r] = 0.f;
        t0 = clock64();
        for (int it = 0; it < iters; it++) {
#pragma unroll
            for (int j = 0; j < 16; j++) P_MFMA(c[j & 3]);
        }
        t1 = clock64();
        for (int n = 0; n < 4; n++)
            for (int r = 0; r < 16; r++) sink += c[n][r];
    } else {
        if (!(mode & 2)) return;
        float v[8];
        for (int i = 0; i < 8; i++) v[i] = a * (lane + i);
        unsigned pk[4] = {0, 0, 0, 0};
        t0 = clock64();
        for (int it = 0; it < iters; it++) {
#pragma unroll
            for (int i = 0; i < 16; i++) {
                if (VK == 0) asm volatile("v_fma_f32 %0, %1, %0, %2" : "+v"(v[i & 7]) : "v"(a), "v"(b));
                if (VK == 1) P_EXP(v[i & 7]);
                if (VK == 2) P_CVT(pk[i & 3], v[i & 7], v[(i + 1) & 7]);
                if (VK == 3) P_DOT(v[i & 7], pk[i & 3]);
            }
        }
        t1 = clock64();
        for (int i = 0; i < 8; i++) sink += v[i];
        for (int i = 0; i < 4; i++) sink += (float)pk[i];
    }
    if (lane == 0) out[wave] = t1 - t0;
    if (sink == 1.2345f) out[8] = 1;
}

// Probe 2: every wave loops over {1 MFMA, N independent vector instructions}.
template <int N, int VK>
__global__ __launch_bounds__(512) void mixed_kernel(long long* out, const h8* data, int iters, float a, float b) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const h8 x = data[threadIdx.x], y = data[threadIdx.x + 512];
    f16v c[4];
    for (int n = 0; n < 4; n++)
        for (int r = 0; r < 16; r++) c[n][r] = 0.f;
    float v[8];
    for (int i = 0; i < 8; i++) v[i] = a * (lane + i);
    const long long t0 = clock64();
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int j = 0; j < 8; j++) {
            P_MFMA(c[j & 3]);
#pragma unroll
            for (int i = 0; i < N; i++) {
                if (VK == 0) asm volatile("v_fma_f32 %0, %1, %0, %2" : "+v"(v[(j * N + i) & 7]) : "v"(a), "v"(b));
                else P_EXP(v[(j * N + i) & 7]);
            }
        }
    }
    const long long t1 = clock64();
    float sink = 0.f;
    for (int n = 0; n < 4; n++)
        for (int r = 0; r < 16; r++) sink += c[n][r];
    for (int i = 0; i < 8; i++) sink += v[i];
    if (lane == 0) out[wave] = t1 - t0;
    if (sink == 1.2345f) out[8] = 1;
}

// Probe 3: the softmax chunk of the attention kernels (2 fma, 2 exp, 1 pack, 1 dot2 for one fp16
// pair of probabilities) with or without one MFMA per chunk.
// PAT 0: chunk + MFMA, 1: chunk without the dot2 + MFMA, 2: chunks only, 3: MFMAs only.
template <int PAT>
__global__ __launch_bounds__(512) void chunk_kernel(long long* out, const h8* data, int iters, float a, float b) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const h8 x = data[threadIdx.x], y = data[threadIdx.x + 512];
    f16v c[4];
    for (int n = 0; n < 4; n++)
        for (int r = 0; r < 16; r++) c[n][r] = 0.f;
    float s[16];
    for (int i = 0; i < 16; i++) s[i] = -0.01f * (lane + i);
    unsigned pk[8] = {};
    float acc = 0.f, e0 = 0.f, e1 = 0.f;
    const long long t0 = clock64();
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            if (PAT != 3) {
                float n0, n1;
                P_FMA(n0, s[2 * i]);
                P_FMA(n1, s[2 * i + 1]);
                P_EXP(n0);
                P_EXP(n1);
                P_CVT(pk[i], e0, e1);      // the pair exponentiated one chunk earlier
                if (PAT != 1) P_DOT(acc, pk[i]);
                e0 = n0;
                e1 = n1;
            }
            if (PAT != 2) P_MFMA(c[i & 3]);
        }
    }
    const long long t1 = clock64();
    float sink = acc + e0 + e1;
    for (int n = 0; n < 4; n++)
        for (int r = 0; r < 16; r++) sink += c[n][r];
    for (int i = 0; i < 8; i++) sink += (float)pk[i];
    if (lane == 0) out[wave] = t1 - t0;
    if (sink == 1.2345f) out[8] = 1;
}

template <int VK>
int run_split(const char* name, long long* d, const h8* data) {
    const int iters = 2000;
    long long h[8];
    double res[4][2] = {};
    for (int mode = 1; mode <= 3; mode++) {
        PROBE_OK(hipMemset(d, 0, 128));
        for (int rep = 0; rep < 2; rep++)
            hipLaunchKernelGGL(split_kernel<VK>, dim3(1), dim3(512), 0, 0, d, data, iters, mode, 0.999f, 0.001f);
        PROBE_OK(hipDeviceSynchronize());
        PROBE_OK(hipMemcpy(h, d, sizeof(h), hipMemcpyDeviceToHost));
        res[mode][0] = (double)h[0] / (iters * 16.0);
        res[mode][1] = (double)h[4] / (iters * 16.0);
    }
    std::printf("  %-10s alone: %5.1f clk/mfma, %5.1f clk/%s | together: %5.1f clk/mfma, %5.1f clk/%s\n", name,
                res[1][0], res[2][1], name, res[3][0], res[3][1], name);
    return 0;
}

template <int N, int VK>
int run_mixed(long long* d, const h8* data) {
    const int iters = 2000;
    long long h[8];
    for (int rep = 0; rep < 2; rep++)
        hipLaunchKernelGGL((mixed_kernel<N, VK>), dim3(1), dim3(256), 0, 0, d, data, iters, 0.999f, 0.001f);
    PROBE_OK(hipDeviceSynchronize());
    PROBE_OK(hipMemcpy(h, d, sizeof(h), hipMemcpyDeviceToHost));
    std::printf("  {1 mfma + %d %s}: %5.1f clk\n", N, VK ? "exp" : "fma", (double)h[0] / (iters * 8.0));
    return 0;
}

template <int PAT>
int run_chunk(const char* name, long long* d, const h8* data) {
    const int iters = 2000;
    for (int threads : {256, 512}) {
        long long h[8];
        for (int rep = 0; rep < 2; rep++)
            hipLaunchKernelGGL(chunk_kernel<PAT>, dim3(1), dim3(threads), 0, 0, d, data, iters, 0.999f, 0.001f);
        PROBE_OK(hipDeviceSynchronize());
        PROBE_OK(hipMemcpy(h, d, sizeof(h), hipMemcpyDeviceToHost));
        std::printf("  %-28s %d wave(s) per SIMD: oldest wave %5.1f, youngest wave %5.1f clk per chunk\n", name,
                    threads / 256, (double)h[0] / (iters * 8.0), (double)h[threads / 64 - 1] / (iters * 8.0));
    }
    return 0;
}

inline int issue_probe() {
    long long* d;
    h8* data;
    PROBE_OK(hipMalloc(&d, 4096));
    PROBE_OK(hipMalloc(&data, 16 * 1024));
    PROBE_OK(hipMemset(data, 0, 16 * 1024));
    std::printf("issue-probe 1: a matrix wave and a vector wave on the same SIMD (v_mfma_f32_32x32x16_f16)\n");
    run_split<0>("fma", d, data);
    run_split<1>("exp", d, data);
    run_split<2>("cvt_pkrtz", d, data);
    run_split<3>("dot2c", d, data);
    std::printf("issue-probe 2: one wave per SIMD issuing both kinds\n");
    run_mixed<0, 0>(d, data);
    run_mixed<2, 0>(d, data);
    run_mixed<4, 0>(d, data);
    run_mixed<6, 0>(d, data);
    run_mixed<8, 0>(d, data);
    run_mixed<2, 1>(d, data);
    run_mixed<4, 1>(d, data);
    std::printf("issue-probe 3: softmax chunk {2 fma, 2 exp, 1 pack, 1 dot2} with one MFMA per chunk\n");
    run_chunk<0>("chunk + mfma", d, data);
    run_chunk<1>("chunk without dot2 + mfma", d, data);
    run_chunk<2>("chunks only", d, data);
    run_chunk<3>("mfma only", d, data);
    (void)hipFree(d);
    (void)hipFree(data);
    return 0;
}
// Phase probe, run as `fa_test phase-probe`: the compute of the eight-wave attention kernel at
// head_dim 64 with everything else taken away (no LDS, no global memory in the loop).  On every
// compute unit two groups of four waves alternate, with a workgroup barrier between phases, between
// the 20 matrix instructions of a 32-key x 64-query sub-tile (4 row-sum MFMAs, 8 for QK^T, 8 for PV,
// with the kernel's dependency pattern) and its 32 fma + 32 exp + 16 pack.  Reported per phase:
// wall time, the clocks each kind of phase takes from barrier to barrier, and the shader clock.
// VWORK selects the work: 0 matrix phases only, 1 the kernel's split, and three splits the kernel
// does not use, timed for comparison: 2 the reference folded into QK^T as a fifth k-step (no fma
// in the vector phase), 3 row sums by v_add_f32 (no row-sum MFMAs), 4 pairs of packed
// probabilities added in fp16 first (half the row-sum MFMAs), 5 the kernel's split with the products
// computed as 16x16 tiles (v_mfma_f32_16x16x32_f16, twice as many instructions of half the size).
// STAMPS selects the clock readings: 0 none, 1 around every barrier (work per kind of phase; the
// readings themselves add about 250 clocks to a phase), 2 two readings around the last 1024
// phases (clocks per phase and shader clock of the undisturbed loop).
typedef _Float16 h2v __attribute__((ext_vector_type(2)));
typedef float f4v __attribute__((ext_vector_type(4)));
typedef unsigned u4v __attribute__((ext_vector_type(4)));

template <int VWORK, int STAMPS>
__global__ __launch_bounds__(512) void phase_kernel(float* out, long long* clk, const h8* data, int iters, float c,
                                                    float mc) {
    const int wave = threadIdx.x / 64;
    const int grp = (wave >> 2) & 1;
    h8 a[8], q[8];
    for (int i = 0; i < 8; i++) {
        a[i] = data[threadIdx.x + i * 512];
        q[i] = data[threadIdx.x + (i + 8) * 512];
    }
    f16v s[2], o[4];
    f4v l[2];
    unsigned pk[2][8], ps[2][4];
    for (int n = 0; n < 2; n++) {
        for (int r = 0; r < 16; r++) s[n][r] = 0.01f * r;
        for (int i = 0; i < 8; i++) pk[n][i] = 0x2c002c00u;
        for (int i = 0; i < 4; i++) ps[n][i] = 0x2c002c00u;
        l[n] = f4v{0.f, 0.f, 0.f, 0.f};
    }
    for (int n = 0; n < 4; n++)
        for (int r = 0; r < 16; r++) o[n][r] = 0.f;
    unsigned long long t0 = 0, t1 = 0, t2 = 0, r0 = 0, first = 0, mwork = 0, vwork = 0;
    for (int it = 0; it < iters; it++) {
        if (STAMPS == 2) {      // two stamps for the whole run: the last 1024 phases
            if (it == iters - 1024)
                asm volatile("s_memtime %0\n\ts_memrealtime %1\n\ts_waitcnt lgkmcnt(0)" : "=s"(first), "=s"(r0)::"memory");
        }
        if (STAMPS == 1) {
            asm volatile("s_memtime %0" : "=s"(t0));
            if (it == iters - 64) asm volatile("s_memrealtime %0\n\ts_waitcnt lgkmcnt(0)" : "=s"(r0)::"memory");
        }
        if (grp == (it & 1)) {
            __builtin_amdgcn_s_setprio(3);
#pragma unroll
            for (int t = 0; t < (VWORK == 3 ? 0 : VWORK == 4 ? 1 : 2); t++)
#pragma unroll
                for (int n = 0; n < 2; n++) {
                    const u4v w = VWORK == 4 ? u4v{ps[n][0], ps[n][1], ps[n][2], ps[n][3]}
                                             : u4v{pk[n][4 * t], pk[n][4 * t + 1], pk[n][4 * t + 2], pk[n][4 * t + 3]};
                    l[n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[7], __builtin_bit_cast(h8, w), l[n], 0, 0, 0);
                }
            if (VWORK == 5) {
                // the same products as 16x16 tiles: 16 instructions of 32 k for QK^T (8 tiles of S^T,
                // two k-steps over head_dim 64), 16 for PV (16 tiles of O^T, one k-step over the 32 keys)
#pragma unroll
                for (int kk = 0; kk < 2; kk++)
#pragma unroll
                    for (int n = 0; n < 2; n++)
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            const f4v z = {0.f, 0.f, 0.f, 0.f};
                            const f4v acc = {s[n][4 * i], s[n][4 * i + 1], s[n][4 * i + 2], s[n][4 * i + 3]};
                            const f4v r = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[kk * 2 + (i & 1)], q[(kk * 2 + n) * 2 + (i >> 1)],
                                                                                 kk == 0 ? z : acc, 0, 0, 0);
#pragma unroll
                            for (int e = 0; e < 4; e++) s[n][4 * i + e] = r[e];
                        }
#pragma unroll
                for (int t = 0; t < 16; t++) {
                    const int n = t & 1, db = (t >> 1) & 1, i = t >> 2;
                    const u4v w = {pk[n][4 * (i & 1)], pk[n][4 * (i & 1) + 1], pk[n][4 * (i & 1) + 2], pk[n][4 * (i & 1) + 3]};
                    f16v& oo = o[db * 2 + n];
                    const f4v acc = {oo[4 * i], oo[4 * i + 1], oo[4 * i + 2], oo[4 * i + 3]};
                    const f4v r = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[4 + db * 2 + (i >> 1)], __builtin_bit_cast(h8, w), acc, 0, 0, 0);
#pragma unroll
                    for (int e = 0; e < 4; e++) oo[4 * i + e] = r[e];
                }
            }
#pragma unroll
            for (int kk = 0; kk < (VWORK == 5 ? 0 : VWORK == 2 ? 5 : 4); kk++)
#pragma unroll
                for (int n = 0; n < 2; n++) {
                    f16v z;
                    for (int r = 0; r < 16; r++) z[r] = 0.f;
                    s[n] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kk == 4 ? a[6] : a[kk], kk == 4 ? q[n] : q[kk * 2 + n],
                                                                  kk == 0 ? z : s[n], 0, 0, 0);
                }
#pragma unroll
            for (int t = 0; t < (VWORK == 5 ? 0 : 2); t++)
#pragma unroll
                for (int db = 0; db < 2; db++)
#pragma unroll
                    for (int n = 0; n < 2; n++) {
                        const u4v w = {pk[n][4 * t], pk[n][4 * t + 1], pk[n][4 * t + 2], pk[n][4 * t + 3]};
                        o[db * 2 + n] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[4 + t * 2 + db], __builtin_bit_cast(h8, w),
                                                                               o[db * 2 + n], 0, 0, 0);
                    }
            __builtin_amdgcn_s_setprio(0);
        } else if (VWORK) {
#pragma unroll
            for (int n = 0; n < 2; n++) {
#pragma unroll
                for (int r = 0; r < 16; r += 2) {
                    const float p0 = __builtin_amdgcn_exp2f(VWORK == 2 ? s[n][r] : __builtin_fmaf(s[n][r], c, mc));
                    const float p1 = __builtin_amdgcn_exp2f(VWORK == 2 ? s[n][r + 1] : __builtin_fmaf(s[n][r + 1], c, mc));
                    pk[n][r >> 1] = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_pkrtz(p0, p1));
                    if (VWORK == 3) {
                        l[n][r & 3] += p0;
                        l[n][(r + 1) & 3] += p1;
                    }
                }
                if (VWORK == 4) {
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        ps[n][i] = __builtin_bit_cast(unsigned, __builtin_bit_cast(h2v, pk[n][i]) +
                                                                    __builtin_bit_cast(h2v, pk[n][i + 4]));
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        if (STAMPS == 1)
            asm volatile("s_memtime %0\n\ts_barrier\n\ts_memtime %1\n\ts_waitcnt lgkmcnt(0)" : "=s"(t1), "=s"(t2)::"memory");
        else
            __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        // the last 64 phases, kept in scalar registers: work of this wave per kind of phase, and the
        // release of the barrier that ends the phase
        if (STAMPS == 1 && it == iters - 65) first = t2;
        if (STAMPS == 1 && it >= iters - 64) {
            if (grp == (it & 1)) mwork += t1 - t0; else vwork += t1 - t0;
        }
    }
    if (STAMPS && blockIdx.x == 0 && threadIdx.x % 64 == 0) {
        unsigned long long r1;
        if (STAMPS == 2) asm volatile("s_memtime %0\n\ts_waitcnt lgkmcnt(0)" : "=s"(t2)::"memory");
        asm volatile("s_memrealtime %0\n\ts_waitcnt lgkmcnt(0)" : "=s"(r1)::"memory");
        long long* p = clk + wave * 4;
        p[0] = (long long)mwork;
        p[1] = (long long)vwork;
        p[2] = (long long)(t2 - first);
        p[3] = (long long)(r1 - r0);
    }
    float acc = 0.f;
    for (int n = 0; n < 2; n++) {
        for (int r = 0; r < 16; r++) acc += s[n][r];
        acc += l[n][0];
    }
    for (int n = 0; n < 4; n++)
        for (int r = 0; r < 16; r++) acc += o[n][r];
    out[blockIdx.x * blockDim.x + threadIdx.x] = acc;
}

template <int VWORK, int STAMPS>
int run_phase(const char* name, int blocks, float* out, long long* clk, const h8* data) {
    const int iters = 20000;
    hipEvent_t e0, e1;
    PROBE_OK(hipEventCreate(&e0));
    PROBE_OK(hipEventCreate(&e1));
    hipLaunchKernelGGL((phase_kernel<VWORK, STAMPS>), dim3(blocks), dim3(512), 0, nullptr, out, clk, data, 2000, 0.18f, -1.0f);
    PROBE_OK(hipEventRecord(e0, nullptr));
    hipLaunchKernelGGL((phase_kernel<VWORK, STAMPS>), dim3(blocks), dim3(512), 0, nullptr, out, clk, data, iters, 0.18f, -1.0f);
    PROBE_OK(hipEventRecord(e1, nullptr));
    PROBE_OK(hipEventSynchronize(e1));
    float ms = 0.f;
    PROBE_OK(hipEventElapsedTime(&ms, e0, e1));
    long long h[32];
    PROBE_OK(hipMemcpy(h, clk, sizeof(h), hipMemcpyDeviceToHost));
    // wave 0 of workgroup 0: 32 matrix and 32 vector phases among its last 64
    const double phase_clk = (double)h[2] / (STAMPS == 2 ? 1024.0 : 64.0);
    const double ghz = (double)h[2] / ((double)h[3] * 10.0);
    if (STAMPS == 2)
        std::printf("  %-34s %6.1f ns per phase | %5.0f clocks per phase at %.2f GHz\n", name, ms * 1e6 / iters, phase_clk, ghz);
    else if (STAMPS)
        std::printf("  %-34s %6.1f ns per phase | with stamps: %5.0f clocks per phase, matrix work %4.0f, vector work %4.0f, %.2f GHz\n",
                    name, ms * 1e6 / iters, phase_clk, (double)h[0] / 32.0, (double)h[1] / 32.0, ghz);
    else
        std::printf("  %-34s %6.1f ns per phase\n", name, ms * 1e6 / iters);
    return 0;
}

inline int phase_probe() {
    hipDeviceProp_t prop;
    PROBE_OK(hipGetDeviceProperties(&prop, 0));
    const int blocks = prop.multiProcessorCount;
    float* out;
    long long* clk;
    h8* data;
    PROBE_OK(hipMalloc(&out, (size_t)blocks * 512 * 4));
    PROBE_OK(hipMalloc(&clk, 32 * sizeof(long long)));
    PROBE_OK(hipMalloc(&data, 16 * 512 * sizeof(h8)));
    _Float16* host = new _Float16[16 * 512 * 8];
    unsigned st = 1u;
    for (int i = 0; i < 16 * 512 * 8; i++) {     // sum of 12 uniforms - 6: close to N(0,1)
        float u = 0.f;
        for (int k = 0; k < 12; k++) {
            st = st * 1664525u + 1013904223u;
            u += (float)(st >> 8) / 16777216.0f;
        }
        host[i] = (_Float16)(u - 6.0f);
    }
    PROBE_OK(hipMemcpy(data, host, 16 * 512 * sizeof(h8), hipMemcpyHostToDevice));
    delete[] host;
    std::printf("phase-probe: two groups of four waves per compute unit alternate between the matrix and the vector work of one\n"
                "32-key x 64-query sub-tile at head_dim 64 (N(0,1) operands, no memory traffic), %d compute units\n", blocks);
    for (int rep = 0; rep < 2; rep++) {
        if (run_phase<0, 2>("matrix phases only", blocks, out, clk, data)) return 2;
        if (run_phase<1, 2>("matrix and vector phases", blocks, out, clk, data)) return 2;
        if (run_phase<0, 1>("matrix phases only", blocks, out, clk, data)) return 2;
        if (run_phase<1, 1>("matrix and vector phases", blocks, out, clk, data)) return 2;
        if (run_phase<2, 2>("reference as a fifth k-step, no fma", blocks, out, clk, data)) return 2;
        if (run_phase<3, 2>("row sums by v_add_f32", blocks, out, clk, data)) return 2;
        if (run_phase<4, 2>("half the row-sum mfma, pk_add_f16", blocks, out, clk, data)) return 2;
        if (run_phase<5, 2>("products as 16x16x32 tiles", blocks, out, clk, data)) return 2;
        if (run_phase<5, 1>("products as 16x16x32 tiles", blocks, out, clk, data)) return 2;
    }
    (void)hipFree(out);
    (void)hipFree(clk);
    (void)hipFree(data);
    return 0;
}

}  // namespace probe
