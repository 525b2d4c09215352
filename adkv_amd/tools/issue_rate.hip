// Vector-instruction issue rates on gfx950, the numbers the decode kernels' instruction budget is
// priced with.  Each kernel runs ITER iterations of 16 independent instances of ONE instruction per
// wave (256-thread workgroups, 256 * waves-per-SIMD of them so that every SIMD of the 256 CUs holds
// that many waves); the table gives nanoseconds per instruction per SIMD and, from wave 0's
// cycle counter, shader-clock ticks per instruction.
//
//     python -m adkv_amd.tools.issue_rate        (builds this file with hipcc and runs it)
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#define ITER 4096
#define REP16(X) X(0) X(1) X(2) X(3) X(4) X(5) X(6) X(7) X(8) X(9) X(10) X(11) X(12) X(13) X(14) X(15)

#define KERNEL(NAME, ASM) \
__global__ __launch_bounds__(256) void NAME(uint32_t* out, uint32_t seed) { \
    uint32_t r[16]; uint32_t a = seed + threadIdx.x, b = seed * 3 + 1, c = seed ^ 0x3c003c00; \
    for (int i = 0; i < 16; i++) r[i] = seed + i; \
    unsigned long long t0 = clock64(); \
    for (int it = 0; it < ITER; it++) { \
        _Pragma("unroll") for (int i = 0; i < 16; i++) asm volatile(ASM : "+v"(r[i]) : "v"(a), "v"(b), "v"(c)); \
    } \
    unsigned long long t1 = clock64(); \
    uint32_t s = 0; for (int i = 0; i < 16; i++) s ^= r[i]; \
    if (s == 0x12345) out[threadIdx.x] = s; \
    if (blockIdx.x == 0 && threadIdx.x == 0) out[1000] = (uint32_t)(t1 - t0); \
}
KERNEL(k_mov,      "v_mov_b32 %0, %1")
KERNEL(k_add_f32,  "v_add_f32 %0, %1, %2")
KERNEL(k_fma_f32,  "v_fma_f32 %0, %1, %2, %3")
KERNEL(k_pk_mul,   "v_pk_mul_f16 %0, %1, %2")
KERNEL(k_pk_add,   "v_pk_add_f16 %0, %1, %2")
KERNEL(k_pk_fma,   "v_pk_fma_f16 %0, %1, %2, %3")
KERNEL(k_dot2,     "v_dot2_f32_f16 %0, %1, %2, %3")
KERNEL(k_dot2c,    "v_dot2c_f32_f16 %0, %1, %2")
KERNEL(k_perm,     "v_perm_b32 %0, %1, %2, %3")
KERNEL(k_bfi,      "v_bfi_b32 %0, %1, %2, %3")
KERNEL(k_and_or,   "v_and_or_b32 %0, %1, %2, %3")
KERNEL(k_fma_mix,  "v_fma_mix_f32 %0, %1, %2, %3 op_sel_hi:[1,1,0]")
KERNEL(k_lshl,     "v_lshlrev_b32 %0, 4, %1")
KERNEL(k_add_dpp,  "v_add_f32_dpp %0, %1, %2 row_ror:8 row_mask:0xf bank_mask:0x3")
// dependent chains
KERNEL(k_pk_mul_dep, "v_pk_mul_f16 %0, %0, %2")
KERNEL(k_pk_fma_dep, "v_pk_fma_f16 %0, %0, %2, %3")
KERNEL(k_fma_f32_dep,"v_fma_f32 %0, %0, %2, %3")

__global__ __launch_bounds__(256) void k_lds64(uint32_t* out, uint32_t seed) {
    __shared__ uint2 lut[8192];
    for (int i = threadIdx.x; i < 8192; i += 256) lut[i] = make_uint2(i, i);
    __syncthreads();
    uint32_t addr = ((threadIdx.x * 2654435761u + seed) & 0xFF00u) | ((threadIdx.x & 31) << 3);
    uint2 r[16];
    for (int it = 0; it < ITER; it++) {
        _Pragma("unroll") for (int i = 0; i < 16; i++) asm volatile("ds_read_b64 %0, %1" : "=v"(r[i]) : "v"(addr));
        asm volatile("s_waitcnt lgkmcnt(0)");
    }
    uint32_t s = 0; for (int i = 0; i < 16; i++) s ^= r[i].x ^ r[i].y;
    if (s == 0x12345) out[threadIdx.x] = s;
}
__global__ __launch_bounds__(256) void k_lds64_rand(uint32_t* out, uint32_t seed) {
    __shared__ uint2 lut[8192];
    for (int i = threadIdx.x; i < 8192; i += 256) lut[i] = make_uint2(i, i);
    __syncthreads();
    uint32_t addr = ((threadIdx.x * 2654435761u + seed) & 0xFFF8u);
    uint2 r[16];
    for (int it = 0; it < ITER; it++) {
        _Pragma("unroll") for (int i = 0; i < 16; i++) asm volatile("ds_read_b64 %0, %1" : "=v"(r[i]) : "v"(addr));
        asm volatile("s_waitcnt lgkmcnt(0)");
    }
    uint32_t s = 0; for (int i = 0; i < 16; i++) s ^= r[i].x ^ r[i].y;
    if (s == 0x12345) out[threadIdx.x] = s;
}


__global__ void k_clock(unsigned long long* out) {
    unsigned long long c0 = clock64(), w0 = wall_clock64();
    float x = threadIdx.x;
    for (int i = 0; i < 2000000; i++) x = __builtin_fmaf(x, 1.000001f, 0.5f);
    unsigned long long c1 = clock64(), w1 = wall_clock64();
    if (threadIdx.x == 0) { out[0] = c1 - c0; out[1] = w1 - w0; out[2] = (unsigned long long)x; }
}

typedef void (*kfn)(uint32_t*, uint32_t);
struct E { const char* n; kfn f; };
int main() {
    uint32_t* d; (void)hipMalloc(&d, 8192);
    unsigned long long* dc; (void)hipMalloc(&dc, 64); unsigned long long hc[3];
    E ks[] = {{"v_mov_b32", k_mov}, {"v_fma_f32", k_fma_f32}, {"v_pk_mul_f16", k_pk_mul},
              {"v_pk_fma_f16", k_pk_fma}, {"v_dot2c_f32_f16", k_dot2c},
              {"v_perm_b32", k_perm}, {"v_fma_mix_f32", k_fma_mix},
              {"v_lshlrev_b32", k_lshl}, {"v_add_f32_dpp (bank-masked)", k_add_dpp},
              {"v_dot2_f32_f16 (3-operand)", k_dot2}, {"pk_fma dep-chain", k_pk_fma_dep},
              {"ds_read_b64 lut-pattern", k_lds64}};
    hipEvent_t e0, e1; (void)hipEventCreate(&e0); (void)hipEventCreate(&e1);
    // warm the clocks
    for (int w = 0; w < 200; w++) hipLaunchKernelGGL(k_pk_fma, dim3(1024), dim3(256), 0, 0, d, 1u);
    (void)hipDeviceSynchronize();
    hipLaunchKernelGGL(k_clock, dim3(1), dim3(64), 0, 0, dc); (void)hipDeviceSynchronize();
    (void)hipMemcpy(hc, dc, 24, hipMemcpyDeviceToHost);
    printf("clock64 ticks %llu, wall_clock64 ticks %llu (100 MHz) -> clock64 rate %.1f MHz; 2M dependent fma => %.2f clock64 ticks per fma\n",
           hc[0], hc[1], hc[0] * 100.0 / hc[1], hc[0] / 2e6);
    int wlist[] = {1, 2, 3, 4, 8};
    for (int wi = 0; wi < 5; wi++) {
        int wps = wlist[wi];
        int blocks = 256 * wps;
        printf("--- %d wave(s) per SIMD\n", wps);
        for (auto& k : ks) {
            for (int w = 0; w < 20; w++) hipLaunchKernelGGL(k.f, dim3(blocks), dim3(256), 0, 0, d, 1u);
            (void)hipDeviceSynchronize();
            (void)hipEventRecord(e0);
            for (int w = 0; w < 20; w++) hipLaunchKernelGGL(k.f, dim3(blocks), dim3(256), 0, 0, d, 1u);
            (void)hipEventRecord(e1); (void)hipEventSynchronize(e1);
            float ms; (void)hipEventElapsedTime(&ms, e0, e1); ms /= 20;
            double ns_per_inst = ms * 1e6 / ((double)ITER * 16 * wps);
            uint32_t ticks = 0; (void)hipMemcpy(&ticks, d + 1000, 4, hipMemcpyDeviceToHost);
            printf("%-26s %8.3f ms  %6.3f ns/inst/SIMD   wave0: %.2f clock64 ticks/inst, implied clock %.0f MHz\n", k.n, ms, ns_per_inst,
                   ticks / (double)(ITER * 16), ticks / (ms * 1e3));
        }
    }
    return 0;
}
