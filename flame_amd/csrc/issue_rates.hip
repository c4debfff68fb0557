// Issue-rate microbenchmark for gfx950: how long one SIMD needs for a bf16 MFMA (32x32x16), a
// plain fp32 vector instruction (v_fma_f32) and a transcendental one (v_exp_f32 / v_rcp_f32),
// alone and mixed in one instruction stream, with 1, 2 or 4 waves per SIMD, and with the two
// kinds of work in DIFFERENT waves of one SIMD.  The stick-breaking kernels are priced with
// these numbers (the vector-issue floor that bench.py prints next to the MFMA roofline).
//   build: make -C flame_amd/csrc issue_rates        run: flame_amd/csrc/issue_rates
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("err %s line %d\n", hipGetErrorString(e), __LINE__); exit(1); } } while (0)
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

// role: 0 = per-wave interleaved {NM mfma, NV fma, NT trans} groups; 1 = heterogeneous: waves 0..3 of an 8-wave
// block run MFMA only, waves 4..7 vector only.
template <int NM, int NV, int NT, bool HET>
__global__ __launch_bounds__(512) void k(float* out, int iters) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    bf16x8 a, b;
    for (int j = 0; j < 8; ++j) { a[j] = (__bf16)(0.001f * (lane + j)); b[j] = (__bf16)(0.002f * (lane - j)); }
    f32x16 acc[4];
    for (int i = 0; i < 4; ++i) acc[i] = f32x16{0};
    float w[8], e = 1.0f + 1e-6f * lane, t[4];
    for (int i = 0; i < 8; ++i) w[i] = 1.0f + 0.1f * i;
    for (int i = 0; i < 4; ++i) t[i] = 0.5f + 0.01f * lane + i;
    auto body = [&](bool do_m, bool do_v) {
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int g = 0; g < 8; ++g) {
                if (do_m) {
#pragma unroll
                    for (int i = 0; i < NM; ++i) acc[(g * NM + i) & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[(g * NM + i) & 3], 0, 0, 0);
                }
                if (do_v) {
#pragma unroll
                    for (int i = 0; i < NV; ++i) w[i & 7] = __builtin_fmaf(w[i & 7], e, 0.5f);
#pragma unroll
                    for (int i = 0; i < NT; ++i) t[i & 3] = (i & 1) ? __builtin_amdgcn_rcpf(t[i & 3]) : __builtin_amdgcn_exp2f(t[i & 3]);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };
    if (!HET) body(true, true);
    else if (wave < 4) body(true, false);
    else body(false, true);
    float r = 0;
    for (int i = 0; i < 8; ++i) r += w[i];
    for (int i = 0; i < 4; ++i) r += t[i];
    for (int i = 0; i < 4; ++i) for (int j = 0; j < 16; ++j) r += acc[i][j];
    out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = r;
}

template <int NM, int NV, int NT, bool HET> void run(const char* name, float* d, int wps, int n_cu) {
    // wps = waves per SIMD; block = 4*wps waves (HET: wps must be even: half of each kind per SIMD)
    const int iters = 2000;
    int blocks = n_cu * wps, tpb = 256;
    if (HET) { blocks = n_cu * wps / 2; tpb = 512; }
    hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
    float ms = 0, best = 1e9;
    for (int rep = 0; rep < 4; ++rep) {
        CK(hipEventRecord(e0));
        hipLaunchKernelGGL((k<NM, NV, NT, HET>), dim3(blocks), dim3(tpb), 0, 0, d, iters);
        CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
        CK(hipEventElapsedTime(&ms, e0, e1));
        if (rep > 0 && ms < best) best = ms;
    }
    const double groups = (double)iters * 8;          // groups per wave
    const double ns_group_wave = best * 1e6 / groups; // wall time of one group of one wave
    // SIMD time per group summed over its waves' groups: wall / (groups per SIMD)
    const double per_simd = ns_group_wave / wps * (HET ? 2 : 1);
    printf("%-34s wps %d  %8.3f ms  wall/group %7.2f ns  SIMD-time per group %7.2f ns\n", name, wps, best, ns_group_wave, per_simd);
    fflush(stdout);
}

int main() {
    int dev = 0, n_cu = 0; CK(hipGetDevice(&dev));
    CK(hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev));
    int clk = 0; CK(hipDeviceGetAttribute(&clk, hipDeviceAttributeClockRate, dev));
    printf("CUs %d, clock attr %d kHz\n", n_cu, clk);
    float* d; CK(hipMalloc(&d, (size_t)n_cu * 8 * 512 * 4));
    // warm the clocks
    for (int i = 0; i < 20; ++i) hipLaunchKernelGGL((k<1, 0, 0, false>), dim3(n_cu), dim3(256), 0, 0, d, 2000);
    CK(hipDeviceSynchronize());
    for (int wps : {1, 2, 4}) {
        run<1, 0, 0, false>("1 MFMA", d, wps, n_cu);
        run<0, 8, 0, false>("8 fma", d, wps, n_cu);
        run<0, 0, 4, false>("4 trans", d, wps, n_cu);
        run<1, 4, 0, false>("1 MFMA + 4 fma", d, wps, n_cu);
        run<1, 8, 0, false>("1 MFMA + 8 fma", d, wps, n_cu);
        run<1, 12, 0, false>("1 MFMA + 12 fma", d, wps, n_cu);
        run<1, 16, 0, false>("1 MFMA + 16 fma", d, wps, n_cu);
        run<1, 0, 4, false>("1 MFMA + 4 trans", d, wps, n_cu);
        run<1, 8, 2, false>("1 MFMA + 8 fma + 2 trans", d, wps, n_cu);
        run<2, 16, 0, false>("2 MFMA + 16 fma", d, wps, n_cu);
        run<0, 16, 0, false>("16 fma", d, wps, n_cu);
        run<0, 8, 2, false>("8 fma + 2 trans", d, wps, n_cu);
        run<0, 8, 4, false>("8 fma + 4 trans", d, wps, n_cu);
        run<0, 16, 4, false>("16 fma + 4 trans", d, wps, n_cu);
        run<2, 16, 4, false>("2 MFMA + 16 fma + 4 trans", d, wps, n_cu);
    }
    for (int wps : {2, 4}) {
        run<1, 8, 0, true>("HET: MFMA waves | 8-fma waves", d, wps, n_cu);
        run<1, 16, 0, true>("HET: MFMA waves | 16-fma waves", d, wps, n_cu);
        run<1, 0, 4, true>("HET: MFMA waves | 4-trans waves", d, wps, n_cu);
    }
    printf("done\n");
    return 0;
}
