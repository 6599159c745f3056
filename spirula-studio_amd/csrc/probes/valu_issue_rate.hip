// valu_issue_rate.hip -- how many cycles of a SIMD one wavefront instruction of a given class takes on gfx950.
//
// The compositing kernels are bound by vector-instruction issue, so their cost model needs the issue rate of each
// instruction class, and the classes differ. Measured on an MI355X (2.37 GHz under this load, measured here too),
// with two and more wavefronts per SIMD, in cycles of a SIMD per wavefront instruction:
//   fp32 add / mul / fma, v_mov                                   2.4 - 3.1
//   a stream of nothing but compares, v_cndmask, min / max, rndne,
//   conversions, 32-bit integer operations or DPP forms           4.1 - 4.5
//   the same compares and selects with fp32 operations between    2.6 - 2.8 on average (the stream's limit is not the
//                                                                 instruction's own cost)
//   transcendentals (v_exp_f32, v_rcp_f32), v_permlane16/32_swap  8.2
//   a scalar instruction between two vector ones                  about 1.8 more for the pair
//   a run of three and more v_cndmask_b32 in the 32-bit encoding (mask in vcc): 16 each -- pairs between other
//   instructions cost nothing extra, nor does the 64-bit encoding; the compiled kernels hold no such run.
// "Four cycles per wavefront instruction" holds for the unmixed second group only.
//
// Method: every workgroup is one wavefront that runs `iters` times through 64 instructions of one class over eight
// independent registers; blocks = 256 CUs x 4 SIMDs x (wavefronts per SIMD). Time from events around the launch;
// cycles = time x clock x 1024 SIMDs / wavefront instructions. The clock is whatever the card runs at under this load:
// measured first (s_memtime against the constant 100 MHz counter), or passed as the first argument in GHz.
//
//     make -C spirula-studio_amd/csrc probes && spirula-studio_amd/csrc/probes/valu_issue_rate [clock GHz]
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

#define SSR_REP8(x) x x x x x x x x
#define SSR_OPS8(op, tail)                                                                                              \
    SSR_REP8(op " %0, %0, " tail "\n " op " %1, %1, " tail "\n " op " %2, %2, " tail "\n " op " %3, %3, " tail "\n " op \
                " %4, %4, " tail "\n " op " %5, %5, " tail "\n " op " %6, %6, " tail "\n " op " %7, %7, " tail "\n")
#define SSR_REGS : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3), "+v"(a4), "+v"(a5), "+v"(a6), "+v"(a7) : "v"(c), "v"(d)

template <int kKind>
__global__ void issue_kernel(float* out, int iters) {
    float a0 = threadIdx.x, a1 = a0 + 1, a2 = a0 + 2, a3 = a0 + 3, a4 = a0 + 4, a5 = a0 + 5, a6 = a0 + 6, a7 = a0 + 7;
    const float c = 1.0001f, d = 0.5f;
    for (int i = 0; i < iters; i++) {
        if (kKind == 0) asm volatile(SSR_OPS8("v_fma_f32", "%8, %9") SSR_REGS);
        if (kKind == 1) asm volatile(SSR_OPS8("v_mul_f32", "%8") SSR_REGS);
        if (kKind == 2) asm volatile(SSR_OPS8("v_add_f32", "%8") SSR_REGS);
        if (kKind == 3) asm volatile(SSR_REP8("v_mov_b32 %0, %1\n v_mov_b32 %1, %2\n v_mov_b32 %2, %3\n v_mov_b32 %3, %4\n v_mov_b32 %4, %5\n v_mov_b32 %5, %6\n v_mov_b32 %6, %7\n v_mov_b32 %7, %0\n") SSR_REGS);
        if (kKind == 4) asm volatile(SSR_REP8("v_cmp_gt_f32 vcc, %0, %8\n v_cndmask_b32 %1, %1, %9, vcc\n v_cmp_gt_f32 vcc, %2, %8\n v_cndmask_b32 %3, %3, %9, vcc\n v_cmp_gt_f32 vcc, %4, %8\n v_cndmask_b32 %5, %5, %9, vcc\n v_cmp_gt_f32 vcc, %6, %8\n v_cndmask_b32 %7, %7, %9, vcc\n") SSR_REGS : "vcc");
        if (kKind == 5) asm volatile(SSR_OPS8("v_mul_f32_dpp", "%8 row_shr:1 row_mask:0xf bank_mask:0xf") SSR_REGS);
        if (kKind == 6) asm volatile(SSR_REP8("v_add_u32 %0, %0, %8\n v_lshl_add_u32 %1, %1, 3, %8\n v_add_u32 %2, %2, %8\n v_lshl_add_u32 %3, %3, 3, %8\n v_add_u32 %4, %4, %8\n v_lshl_add_u32 %5, %5, 3, %8\n v_add_u32 %6, %6, %8\n v_lshl_add_u32 %7, %7, 3, %8\n") SSR_REGS);
        if (kKind == 7) asm volatile(SSR_REP8("v_exp_f32 %0, %0\n v_rcp_f32 %1, %1\n v_exp_f32 %2, %2\n v_rcp_f32 %3, %3\n v_exp_f32 %4, %4\n v_rcp_f32 %5, %5\n v_exp_f32 %6, %6\n v_rcp_f32 %7, %7\n") SSR_REGS);
        if (kKind == 8) asm volatile(SSR_REP8("v_permlane16_swap_b32 %0, %1\n v_permlane32_swap_b32 %2, %3\n v_permlane16_swap_b32 %4, %5\n v_permlane32_swap_b32 %6, %7\n v_permlane16_swap_b32 %1, %2\n v_permlane32_swap_b32 %3, %4\n v_permlane16_swap_b32 %5, %6\n v_permlane32_swap_b32 %7, %0\n") SSR_REGS);
        // 32 vector + 32 scalar instructions, interleaved: what a scalar instruction between two vector ones costs
        if (kKind == 9) asm volatile(SSR_REP8("v_fma_f32 %0, %0, %8, %9\n s_and_b64 s[20:21], s[20:21], exec\n v_fma_f32 %2, %2, %8, %9\n s_or_b64 s[22:23], s[22:23], exec\n v_fma_f32 %4, %4, %8, %9\n s_and_b64 s[20:21], s[20:21], exec\n v_fma_f32 %6, %6, %8, %9\n s_or_b64 s[22:23], s[22:23], exec\n") SSR_REGS : "s20", "s21", "s22", "s23", "scc");
        if (kKind == 10) asm volatile(SSR_REP8("v_cmp_gt_f32 vcc, %0, %8\n v_cmp_gt_f32 vcc, %1, %8\n v_cmp_gt_f32 vcc, %2, %8\n v_cmp_gt_f32 vcc, %3, %8\n v_cmp_gt_f32 vcc, %4, %8\n v_cmp_gt_f32 vcc, %5, %8\n v_cmp_gt_f32 vcc, %6, %8\n v_cmp_gt_f32 vcc, %7, %8\n") SSR_REGS : "vcc");
        if (kKind == 11) asm volatile("v_cmp_gt_f32 vcc, %0, %8\n" SSR_OPS8("v_cndmask_b32", "%9, vcc") SSR_REGS : "vcc");
        if (kKind == 12) asm volatile(SSR_REP8("v_min_f32 %0, %0, %8\n v_max_f32 %1, %1, %9\n v_min_f32 %2, %2, %8\n v_max_f32 %3, %3, %9\n v_min_f32 %4, %4, %8\n v_max_f32 %5, %5, %9\n v_min_f32 %6, %6, %8\n v_max_f32 %7, %7, %9\n") SSR_REGS);
        if (kKind == 13) asm volatile(SSR_REP8("v_rndne_f32 %0, %0\n v_rndne_f32 %1, %1\n v_rndne_f32 %2, %2\n v_rndne_f32 %3, %3\n v_rndne_f32 %4, %4\n v_rndne_f32 %5, %5\n v_rndne_f32 %6, %6\n v_rndne_f32 %7, %7\n") SSR_REGS);
        if (kKind == 14) asm volatile(SSR_REP8("v_cvt_i32_f32 %0, %0\n v_cvt_f32_i32 %0, %0\n v_cvt_i32_f32 %2, %2\n v_cvt_f32_i32 %2, %2\n v_cvt_i32_f32 %4, %4\n v_cvt_f32_i32 %4, %4\n v_cvt_i32_f32 %6, %6\n v_cvt_f32_i32 %6, %6\n") SSR_REGS);
        if (kKind == 15) asm volatile(SSR_REP8("v_cmp_gt_f32 s[20:21], %0, %8\n v_cndmask_b32 %1, %1, %9, s[20:21]\n v_cmp_gt_f32 s[22:23], %2, %8\n v_cndmask_b32 %3, %3, %9, s[22:23]\n v_cmp_gt_f32 s[20:21], %4, %8\n v_cndmask_b32 %5, %5, %9, s[20:21]\n v_cmp_gt_f32 s[22:23], %6, %8\n v_cndmask_b32 %7, %7, %9, s[22:23]\n") SSR_REGS : "s20", "s21", "s22", "s23");
        if (kKind == 16) asm volatile("s_mov_b64 s[20:21], 0x5555\n" SSR_OPS8("v_cndmask_b32", "%9, s[20:21]") SSR_REGS : "s20", "s21");
        if (kKind == 17) asm volatile(SSR_REP8("v_cmp_gt_f32 vcc, %0, %8\n v_cndmask_b32 %1, %1, %9, vcc\n v_cndmask_b32 %2, %2, %9, vcc\n v_cndmask_b32 %3, %3, %9, vcc\n v_cmp_gt_f32 vcc, %4, %8\n v_cndmask_b32 %5, %5, %9, vcc\n v_cndmask_b32 %6, %6, %9, vcc\n v_cndmask_b32 %7, %7, %9, vcc\n") SSR_REGS : "vcc");
        if (kKind == 18) asm volatile("v_cmp_gt_f32 vcc, %0, %8\n" SSR_REP8("v_cndmask_b32 %0, %1, %9, vcc\n v_cndmask_b32 %1, %2, %9, vcc\n v_cndmask_b32 %2, %3, %9, vcc\n v_cndmask_b32 %3, %4, %9, vcc\n v_cndmask_b32 %4, %5, %9, vcc\n v_cndmask_b32 %5, %6, %9, vcc\n v_cndmask_b32 %6, %7, %9, vcc\n v_cndmask_b32 %7, %0, %9, vcc\n") SSR_REGS : "vcc");
        if (kKind == 19) asm volatile(SSR_REP8("v_cmp_gt_f32 vcc, %0, %8\n v_fma_f32 %1, %1, %8, %9\n v_cndmask_b32 %2, %2, %9, vcc\n v_fma_f32 %3, %3, %8, %9\n v_cmp_gt_f32 vcc, %4, %8\n v_fma_f32 %5, %5, %8, %9\n v_cndmask_b32 %6, %6, %9, vcc\n v_fma_f32 %7, %7, %8, %9\n") SSR_REGS : "vcc");
        if (kKind == 20) asm volatile(SSR_REP8("v_cmp_gt_f32 vcc, %0, %8\n v_fma_f32 %1, %1, %8, %9\n v_fma_f32 %2, %2, %8, %9\n v_fma_f32 %3, %3, %8, %9\n v_fma_f32 %4, %4, %8, %9\n v_fma_f32 %5, %5, %8, %9\n v_fma_f32 %6, %6, %8, %9\n v_cndmask_b32 %7, %7, %9, vcc\n") SSR_REGS : "vcc");
        if (kKind == 21) asm volatile("v_cmp_gt_f32 vcc, %0, %8\n" SSR_OPS8("v_cndmask_b32_e64", "%9, vcc") SSR_REGS : "vcc");
        if (kKind == 22) asm volatile(SSR_REP8("v_cmp_gt_f32 vcc, %0, %8\n v_cndmask_b32 %1, %1, %9, vcc\n v_fma_f32 %2, %2, %8, %9\n v_cndmask_b32 %3, %3, %9, vcc\n v_cmp_gt_f32 vcc, %4, %8\n v_cndmask_b32 %5, %5, %9, vcc\n v_fma_f32 %6, %6, %8, %9\n v_cndmask_b32 %7, %7, %9, vcc\n") SSR_REGS : "vcc");
        if (kKind == 23) asm volatile("v_cmp_gt_f32 vcc, %0, %8\n s_mov_b64 s[20:21], 0x5555\n" SSR_REP8("v_cndmask_b32 %0, %0, %9, s[20:21]\n v_cndmask_b32 %1, %1, %9, vcc\n v_cndmask_b32 %2, %2, %9, s[20:21]\n v_cndmask_b32 %3, %3, %9, vcc\n v_cndmask_b32 %4, %4, %9, s[20:21]\n v_cndmask_b32 %5, %5, %9, vcc\n v_cndmask_b32 %6, %6, %9, s[20:21]\n v_cndmask_b32 %7, %7, %9, vcc\n") SSR_REGS : "vcc", "s20", "s21");
        if (kKind == 24) asm volatile("v_cmp_gt_f32 vcc, %0, %8\n" SSR_REP8("v_fma_f32 %0, %0, %8, %9\n v_cndmask_b32 %1, %1, %9, vcc\n v_cndmask_b32 %2, %2, %9, vcc\n v_fma_f32 %3, %3, %8, %9\n v_fma_f32 %4, %4, %8, %9\n v_cndmask_b32 %5, %5, %9, vcc\n v_cndmask_b32 %6, %6, %9, vcc\n v_fma_f32 %7, %7, %8, %9\n") SSR_REGS : "vcc");
    }
    out[blockIdx.x * blockDim.x + threadIdx.x] = a0 + a1 + a2 + a3 + a4 + a5 + a6 + a7;
}

// The shader clock: s_memtime counts it, the constant-rate counter runs at 100 MHz; a wavefront that spins for a while
// reads both at either end.
__global__ void clock_kernel(unsigned long long* out, int iters) {
    const unsigned long long c0 = clock64(), w0 = wall_clock64();
    float a = threadIdx.x;
    for (int i = 0; i < iters; i++) asm volatile("v_fma_f32 %0, %0, %0, %0" : "+v"(a));
    const unsigned long long c1 = clock64(), w1 = wall_clock64();
    if (threadIdx.x == 0) { out[0] = c1 - c0; out[1] = w1 - w0; out[2] = (unsigned long long)a; }
}

template <int kKind>
static int measure(const char* name, float* d, int vector_per_iter, double ghz) {
    const int iters = 2000;
    printf("%-34s", name);
    for (int wps : {1, 2, 4, 8}) {
        const int blocks = 256 * 4 * wps;   // one wavefront a workgroup: wps wavefronts per SIMD when spread evenly
        hipEvent_t a, b;
        if (hipEventCreate(&a) != hipSuccess || hipEventCreate(&b) != hipSuccess) return 1;
        hipLaunchKernelGGL(issue_kernel<kKind>, dim3(blocks), dim3(64), 0, 0, d, 10);
        if (hipEventRecord(a, 0) != hipSuccess) return 1;
        hipLaunchKernelGGL(issue_kernel<kKind>, dim3(blocks), dim3(64), 0, 0, d, iters);
        if (hipEventRecord(b, 0) != hipSuccess || hipEventSynchronize(b) != hipSuccess) return 1;
        float ms = 0;
        if (hipEventElapsedTime(&ms, a, b) != hipSuccess) return 1;
        const double insts = (double)blocks * iters * vector_per_iter;
        printf("  %d/SIMD: %5.2f", wps, ms * 1e6 * ghz * 1024 / insts);
        if (hipEventDestroy(a) != hipSuccess || hipEventDestroy(b) != hipSuccess) return 1;
    }
    printf("   cycles per vector instruction\n");
    return 0;
}

int main(int argc, char** argv) {
    double ghz = argc > 1 ? atof(argv[1]) : 0.0;
    float* d = nullptr;
    if (hipMalloc(&d, (size_t)256 * 4 * 8 * 64 * sizeof(float)) != hipSuccess) { printf("hipMalloc failed\n"); return 1; }
    if (ghz <= 0.0) {   // measured under load: every SIMD busy with the spinning kernel
        unsigned long long* t = nullptr;
        unsigned long long h[3] = {0, 0, 0};
        if (hipMalloc(&t, sizeof(h)) != hipSuccess) return 1;
        hipLaunchKernelGGL(clock_kernel, dim3(256 * 4 * 2), dim3(64), 0, 0, t, 2000000);
        if (hipMemcpy(h, t, sizeof(h), hipMemcpyDeviceToHost) != hipSuccess || hipFree(t) != hipSuccess) return 1;
        ghz = h[1] ? 0.1 * (double)h[0] / (double)h[1] : 2.3;
        printf("shader clock under load: %.3f GHz (s_memtime against the 100 MHz counter)\n", ghz);
    }
    printf("cycles of a SIMD per wavefront (64-lane) vector instruction at %.2f GHz, by wavefronts per SIMD\n", ghz);
    int rc = 0;
    rc |= measure<0>("v_fma_f32", d, 64, ghz);
    rc |= measure<1>("v_mul_f32", d, 64, ghz);
    rc |= measure<2>("v_add_f32", d, 64, ghz);
    rc |= measure<3>("v_mov_b32", d, 64, ghz);
    rc |= measure<4>("v_cmp_gt_f32 + v_cndmask_b32", d, 64, ghz);
    rc |= measure<5>("v_mul_f32_dpp row_shr:1", d, 64, ghz);
    rc |= measure<6>("v_add_u32 / v_lshl_add_u32", d, 64, ghz);
    rc |= measure<7>("v_exp_f32 / v_rcp_f32", d, 64, ghz);
    rc |= measure<8>("v_permlane16/32_swap_b32", d, 64, ghz);
    rc |= measure<9>("v_fma_f32 with s_and/s_or between", d, 32, ghz);
    rc |= measure<10>("v_cmp_gt_f32 (to vcc)", d, 64, ghz);
    rc |= measure<11>("v_cndmask_b32 (vcc)", d, 64, ghz);
    rc |= measure<12>("v_min_f32 / v_max_f32", d, 64, ghz);
    rc |= measure<13>("v_rndne_f32", d, 64, ghz);
    rc |= measure<14>("v_cvt_i32_f32 / v_cvt_f32_i32", d, 64, ghz);
    rc |= measure<15>("v_cmp (to sgprs) + v_cndmask (sgprs)", d, 64, ghz);
    rc |= measure<16>("v_cndmask_b32 (sgprs set once)", d, 64, ghz);
    rc |= measure<17>("v_cmp (vcc) + 3 v_cndmask (vcc)", d, 64, ghz);
    rc |= measure<18>("v_cndmask_b32 (vcc), dst != src", d, 64, ghz);
    rc |= measure<19>("cmp vcc, fma, cndmask vcc, fma", d, 64, ghz);
    rc |= measure<20>("cmp vcc, 6 fma, cndmask vcc", d, 64, ghz);
    rc |= measure<21>("v_cndmask_b32_e64 (vcc set once)", d, 64, ghz);
    rc |= measure<22>("cmp vcc, cndmask, fma, cndmask", d, 64, ghz);
    rc |= measure<23>("cndmask (sgprs), cndmask (vcc), ...", d, 64, ghz);
    rc |= measure<24>("fma, 2 cndmask (vcc), fma", d, 64, ghz);
    if (hipFree(d) != hipSuccess) rc = 1;
    return rc;
}
