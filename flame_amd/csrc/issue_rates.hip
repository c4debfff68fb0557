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


// ---- second table: one vector (or scalar) instruction kind per loop, written in assembly so that the compiler
// cannot change it; 8 independent registers unless the label says otherwise.  time per instruction per SIMD.
#define REP8(I) I(a0) I(a1) I(a2) I(a3) I(a4) I(a5) I(a6) I(a7)
#define BODY32(I) REP8(I) REP8(I) REP8(I) REP8(I)
template <int V>
__global__ __launch_bounds__(256) void vk(float* out, int iters) {
    const int lane = threadIdx.x & 63;
    float a0 = 1.0f + lane * 1e-3f, a1 = a0 + 1, a2 = a0 + 2, a3 = a0 + 3, a4 = a0 + 4, a5 = a0 + 5, a6 = a0 + 6, a7 = a0 + 7;
    float x = 0.999f + lane * 1e-6f, y = 1e-3f * lane;
    int m = lane & 1;
    unsigned long long p0 = lane, p1 = lane * 3;
    for (int it = 0; it < iters; ++it) {
#define ONE(N, TEXT) if (V == N) { BODY32(TEXT) }
#define I0(a) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(a) : "v"(x), "v"(y));
        ONE(0, I0)
#define I1(a) asm volatile("v_fmac_f32 %0, %1, %2" : "+v"(a) : "v"(x), "v"(y));
        ONE(1, I1)
#define I2(a) asm volatile("v_mul_f32 %0, %0, %1" : "+v"(a) : "v"(x));
        ONE(2, I2)
#define I3(a) asm volatile("v_add_f32 %0, %0, %1" : "+v"(a) : "v"(y));
        ONE(3, I3)
#define I4(a) asm volatile("v_sub_f32 %0, %1, %0" : "+v"(a) : "v"(x));
        ONE(4, I4)
#define I5(a) asm volatile("v_mov_b32 %0, %1" : "+v"(a) : "v"(x));
        ONE(5, I5)
#define I6(a) asm volatile("v_add_u32 %0, %0, %1" : "+v"(a) : "v"(m));
        ONE(6, I6)
#define I7(a) asm volatile("v_fma_f32 %0, %0, %1, %2 clamp" : "+v"(a) : "v"(x), "v"(y));
        ONE(7, I7)
#define I8(a) asm volatile("v_fma_f32 %0, %0, %1, 1.0" : "+v"(a) : "v"(x));
        ONE(8, I8)
#define I9(a) asm volatile("v_mul_f32_e64 %0, %0, %1 clamp" : "+v"(a) : "v"(x));
        ONE(9, I9)
#define I10(a) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(a0) : "v"(x), "v"(y));
        ONE(10, I10)
#define I11(a) asm volatile("v_max_f32 %0, %0, %1" : "+v"(a) : "v"(x));
        ONE(11, I11)
#define I12(a) asm volatile("v_cmp_lt_f32_e64 s[20:21], %0, %1" :: "v"(a), "v"(x) : "s20", "s21");
        ONE(12, I12)
#define I13(a) asm volatile("v_cndmask_b32_e64 %0, %0, %1, s[20:21]" : "+v"(a) : "v"(x) : "s20", "s21");
        ONE(13, I13)
#define I14(a) asm volatile("v_cvt_pk_bf16_f32 %0, %0, %1" : "+v"(a) : "v"(x));
        ONE(14, I14)
#define I15(a) asm volatile("v_med3_f32 %0, %0, %1, %2" : "+v"(a) : "v"(x), "v"(y));
        ONE(15, I15)
#define I16(a) asm volatile("v_lshlrev_b32 %0, 1, %0" : "+v"(a));
        ONE(16, I16)
#define I17(a) asm volatile("v_lshl_add_u32 %0, %0, 1, %1" : "+v"(a) : "v"(m));
        ONE(17, I17)
#define I18(a) asm volatile("v_mul_lo_u32 %0, %0, %1" : "+v"(a) : "v"(m));
        ONE(18, I18)
#define I19(a) asm volatile("v_lshl_add_u64 %0, %0, 0, %1" : "+v"(p0) : "v"(p1));
        ONE(19, I19)
#define I20(a) asm volatile("v_mov_b64 %0, %1" : "=v"(p0) : "v"(p1));
        ONE(20, I20)
#define I21(a) asm volatile("v_readlane_b32 s20, %0, 3" :: "v"(a) : "s20");
        ONE(21, I21)
#define I22(a) asm volatile("v_writelane_b32 %0, s3, 3" : "+v"(a));
        ONE(22, I22)
#define I23(a) asm volatile("v_fma_f32 %0, %0, s4, %1" : "+v"(a) : "v"(y));
        ONE(23, I23)
#define I24(a) asm volatile("v_mov_b32_dpp %0, %0 row_shr:1 row_mask:0xf bank_mask:0xf" : "+v"(a));
        ONE(24, I24)
#define I25(a) asm volatile("v_exp_f32 %0, %0" : "+v"(a));
        ONE(25, I25)
#define I26(a) asm volatile("v_rcp_f32 %0, %0" : "+v"(a));
        ONE(26, I26)
#define I27(a) asm volatile("v_fma_f32 %0, %0, %1, %2\n s_mov_b32 s20, 7" : "+v"(a) : "v"(x), "v"(y) : "s20");
        ONE(27, I27)
#define I28(a) asm volatile("v_fma_f32 %0, %0, %1, %2\n s_waitcnt lgkmcnt(0)" : "+v"(a) : "v"(x), "v"(y));
        ONE(28, I28)
    }
    out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = (float)(p0 & 1) + a0 + a1 + a2 + a3 + a4 + a5 + a6 + a7;
}

template <int V> void vrun(const char* name, float* d, int n_cu) {
    const int iters = 4000;
    printf("%-44s", name);
    for (int wps : {1, 2, 4}) {
        hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
        float ms = 0, best = 1e9;
        for (int rep = 0; rep < 4; ++rep) {
            CK(hipEventRecord(e0));
            hipLaunchKernelGGL((vk<V>), dim3(n_cu * wps), dim3(256), 0, 0, d, iters);
            CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
            CK(hipEventElapsedTime(&ms, e0, e1));
            if (rep > 0 && ms < best) best = ms;
        }
        printf("  wps %d %6.2f ns", wps, best * 1e6 / ((double)iters * 32) / wps);
    }
    printf("\n");
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
    printf("\nper instruction kind: SIMD time per instruction (ns) with 1, 2, 4 waves per SIMD\n");
    vrun<0>("v_fma_f32 (three vector registers)", d, n_cu);
    vrun<1>("v_fmac_f32", d, n_cu);
    vrun<2>("v_mul_f32", d, n_cu);
    vrun<3>("v_add_f32", d, n_cu);
    vrun<4>("v_sub_f32", d, n_cu);
    vrun<5>("v_mov_b32", d, n_cu);
    vrun<6>("v_add_u32", d, n_cu);
    vrun<7>("v_fma_f32 clamp", d, n_cu);
    vrun<8>("v_fma_f32 with inline constant", d, n_cu);
    vrun<9>("v_mul_f32 clamp (VOP3)", d, n_cu);
    vrun<10>("v_fma_f32, ONE dependent chain", d, n_cu);
    vrun<11>("v_max_f32", d, n_cu);
    vrun<12>("v_cmp_lt_f32 -> scalar pair", d, n_cu);
    vrun<13>("v_cndmask_b32 (mask in a scalar pair)", d, n_cu);
    vrun<14>("v_cvt_pk_bf16_f32", d, n_cu);
    vrun<15>("v_med3_f32", d, n_cu);
    vrun<16>("v_lshlrev_b32", d, n_cu);
    vrun<17>("v_lshl_add_u32", d, n_cu);
    vrun<18>("v_mul_lo_u32", d, n_cu);
    vrun<19>("v_lshl_add_u64", d, n_cu);
    vrun<20>("v_mov_b64", d, n_cu);
    vrun<21>("v_readlane_b32", d, n_cu);
    vrun<22>("v_writelane_b32", d, n_cu);
    vrun<23>("v_fma_f32 with a scalar-register operand", d, n_cu);
    vrun<24>("v_mov_b32 dpp row_shr", d, n_cu);
    vrun<25>("v_exp_f32", d, n_cu);
    vrun<26>("v_rcp_f32", d, n_cu);
    vrun<27>("v_fma_f32 + s_mov_b32 (per PAIR)", d, n_cu);
    vrun<28>("v_fma_f32 + s_waitcnt, nothing pending (per PAIR)", d, n_cu);
    printf("done\n");
    return 0;
}
