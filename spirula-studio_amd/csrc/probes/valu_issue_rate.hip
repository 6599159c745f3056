// valu_issue_rate.hip -- how many cycles of a SIMD one wavefront instruction of a given class takes on gfx950.
//
// The compositing kernels are bound by vector-instruction issue, so their cost model needs the issue rate of each
// instruction class, and the classes differ: measured on an MI355X (2.3 GHz under this load), with two and more
// wavefronts per SIMD, fp32 add / mul / fma and v_mov take 2.3 - 2.8 cycles per wavefront instruction, compares,
// v_cndmask, DPP forms and 32-bit integer operations 4.1, transcendentals (v_exp_f32, v_rcp_f32) 7.8; a scalar
// instruction between two vector ones costs the pair about 1.8 cycles more. "Four cycles per wavefront instruction"
// holds for the second group only.
//
// Method: every workgroup is one wavefront that runs `iters` times through 64 instructions of one class over eight
// independent registers; blocks = 256 CUs x 4 SIMDs x (wavefronts per SIMD). Time from events around the launch;
// cycles = time x clock x 1024 SIMDs / wavefront instructions. The clock is whatever the card runs at: pass it as the
// first argument in GHz (default 2.3; rocprofv3's GRBM_GUI_ACTIVE / 8 over a kernel's duration gives it).
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
    }
    out[blockIdx.x * blockDim.x + threadIdx.x] = a0 + a1 + a2 + a3 + a4 + a5 + a6 + a7;
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
    const double ghz = argc > 1 ? atof(argv[1]) : 2.3;
    float* d = nullptr;
    if (hipMalloc(&d, (size_t)256 * 4 * 8 * 64 * sizeof(float)) != hipSuccess) { printf("hipMalloc failed\n"); return 1; }
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
    if (hipFree(d) != hipSuccess) rc = 1;
    return rc;
}
