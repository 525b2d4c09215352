// Vector-instruction issue rates on gfx950, the numbers the decode kernels' instruction budget is
// priced with.  Each kernel runs ITER rounds of 16 independent instances of ONE instruction per
// wave (256-thread workgroups, 256 * waves-per-SIMD of them so that every SIMD of the 256 CUs holds
// that many waves); the table gives nanoseconds per instruction per SIMD and, from wave 0's
// cycle counter, shader-clock ticks per instruction.
//
//     python -m adkv_amd.tools.issue_rate        (builds this file with hipcc and runs it)
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#define ITER 4096
// The timed loops are unrolled UNR times: a taken branch costs the wave that takes it some 20 cycles
// of issue, which with 16 instructions per trip and four waves per SIMD reads as 2.28 ns per packed
// instruction where the pipe itself takes 1.77 ns (4 cycles at 2.26 GHz).  -DUNR=1 shows that.
#ifndef UNR
#define UNR 8
#endif
#define REP16(X) X(0) X(1) X(2) X(3) X(4) X(5) X(6) X(7) X(8) X(9) X(10) X(11) X(12) X(13) X(14) X(15)

#define KERNEL(NAME, ASM) \
__global__ __launch_bounds__(1024) void NAME(uint32_t* out, uint32_t seed) { \
    uint32_t r[16]; uint32_t a = seed + threadIdx.x, b = seed * 3 + 1, c = seed ^ 0x3c003c00; \
    for (int i = 0; i < 16; i++) r[i] = seed + i; \
    unsigned long long t0 = clock64(); \
    for (int it = 0; it < ITER / UNR; it++) { \
        _Pragma("unroll") for (int u = 0; u < UNR; u++) { \
            _Pragma("unroll") for (int i = 0; i < 16; i++) asm volatile(ASM : "+v"(r[i]) : "v"(a), "v"(b), "v"(c)); \
        } \
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
// the wider survey (run with --all): which plain 32-bit and scalar-f16 forms issue at the fast rate
KERNEL(k_mul_f32,  "v_mul_f32 %0, %1, %2")
KERNEL(k_max_f32,  "v_max_f32 %0, %1, %2")
KERNEL(k_and,      "v_and_b32 %0, %1, %2")
KERNEL(k_or,       "v_or_b32 %0, %1, %2")
KERNEL(k_xor,      "v_xor_b32 %0, %1, %2")
KERNEL(k_add_u32,  "v_add_u32 %0, %1, %2")
KERNEL(k_bfe,      "v_bfe_u32 %0, %1, 8, 8")
KERNEL(k_lshl_or,  "v_lshl_or_b32 %0, %1, 4, %2")
KERNEL(k_lshl_add, "v_lshl_add_u32 %0, %1, 4, %2")
KERNEL(k_add3,     "v_add3_u32 %0, %1, %2, %3")
KERNEL(k_or3,      "v_or3_b32 %0, %1, %2, %3")
KERNEL(k_alignbit, "v_alignbit_b32 %0, %1, %2, 8")
KERNEL(k_lshr,     "v_lshrrev_b32 %0, 4, %1")
KERNEL(k_mul_u24,  "v_mul_u32_u24 %0, %1, %2")
KERNEL(k_mad_u24,  "v_mad_u32_u24 %0, %1, %2, %3")
KERNEL(k_cndmask,  "v_cndmask_b32 %0, %1, %2, vcc")
KERNEL(k_mul_f16,  "v_mul_f16 %0, %1, %2")
KERNEL(k_add_f16,  "v_add_f16 %0, %1, %2")
KERNEL(k_fma_f16,  "v_fma_f16 %0, %1, %2, %3")
KERNEL(k_cvt_f32_f16, "v_cvt_f32_f16 %0, %1")
KERNEL(k_cvt_f16_f32, "v_cvt_f16_f32 %0, %1")
KERNEL(k_sdwa_or,  "v_or_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_1 src1_sel:DWORD")
KERNEL(k_mov_dpp,  "v_mov_b32_dpp %0, %1 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf")
KERNEL(k_add_dpp_full, "v_add_f32_dpp %0, %1, %2 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf")
KERNEL(k_rcp,      "v_rcp_f32 %0, %1")
KERNEL(k_exp,      "v_exp_f32 %0, %1")
// dependent chains
KERNEL(k_pk_mul_dep, "v_pk_mul_f16 %0, %0, %2")
KERNEL(k_pk_fma_dep, "v_pk_fma_f16 %0, %0, %2, %3")
KERNEL(k_fma_f32_dep,"v_fma_f32 %0, %0, %2, %3")

__global__ __launch_bounds__(1024) void k_lds64(uint32_t* out, uint32_t seed) {
    __shared__ uint2 lut[8192];
    for (int i = threadIdx.x; i < 8192; i += blockDim.x) lut[i] = make_uint2(i, i);
    __syncthreads();
    uint32_t addr = ((threadIdx.x * 2654435761u + seed) & 0xFF00u) | ((threadIdx.x & 31) << 3);
    uint2 r[16];
    for (int it = 0; it < ITER / UNR; it++) {
        _Pragma("unroll") for (int u = 0; u < UNR; u++) {
            _Pragma("unroll") for (int i = 0; i < 16; i++) asm volatile("ds_read_b64 %0, %1" : "=v"(r[i]) : "v"(addr));
            asm volatile("s_waitcnt lgkmcnt(0)");
        }
    }
    uint32_t s = 0; for (int i = 0; i < 16; i++) s ^= r[i].x ^ r[i].y;
    if (s == 0x12345) out[threadIdx.x] = s;
}

// Matrix-core instructions beside packed vector arithmetic: NV independent v_pk_fma_f16 and NM
// v_mfma per iteration, evenly interleaved.  If the time follows NV alone, a matrix instruction
// rides free of the vector pipe's issue slots; if it follows NV + NM, it costs a slot like any other.
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
template <int NV, int NM, int KIND>
__global__ __launch_bounds__(1024) void k_mix(uint32_t* out, uint32_t seed) {
    uint32_t r[16]; uint32_t a = seed + threadIdx.x, b = seed * 3 + 1, c = seed ^ 0x3c003c00;
    for (int i = 0; i < 16; i++) r[i] = seed + i;
    f32x4 acc[8];
    for (int i = 0; i < 8; i++) acc[i] = f32x4{(float)i, 1.f, 2.f, 3.f};
    f16x4 ma = {(_Float16)1, (_Float16)2, (_Float16)(int)(seed & 3), (_Float16)0.5f}, mb = ma;
    constexpr int N = NV > NM ? NV : NM;
    unsigned long long t0 = clock64();
    for (int it = 0; it < ITER / UNR; it++) {
        _Pragma("unroll") for (int u = 0; u < UNR; u++)
        _Pragma("unroll") for (int i = 0; i < N; i++) {
            if (i * NV / N != (i + 1) * NV / N)
                asm volatile("v_pk_fma_f16 %0, %1, %2, %3" : "+v"(r[i & 15]) : "v"(a), "v"(b), "v"(c));
            if (i * NM / N != (i + 1) * NM / N) {
                if (KIND == 0) asm volatile("v_mfma_f32_4x4x4_16b_f16 %0, %1, %2, %0" : "+v"(acc[i & 7]) : "v"(ma), "v"(mb));
                else           asm volatile("v_mfma_f32_16x16x16_f16 %0, %1, %2, %0" : "+v"(acc[i & 7]) : "v"(ma), "v"(mb));
            }
        }
    }
    unsigned long long t1 = clock64();
    uint32_t s = 0; for (int i = 0; i < 16; i++) s ^= r[i];
    float fs = 0; for (int i = 0; i < 8; i++) fs += acc[i].x + acc[i].y + acc[i].z + acc[i].w;
    if (s == 0x12345 || fs == 1.2345f) out[threadIdx.x] = s;
    if (blockIdx.x == 0 && threadIdx.x == 0) out[1000] = (uint32_t)(t1 - t0);
}

__global__ void k_clock(unsigned long long* out) {
    unsigned long long c0 = clock64(), w0 = wall_clock64();
    float x = threadIdx.x;
    for (int i = 0; i < 2000000; i++) x = __builtin_fmaf(x, 1.000001f, 0.5f);
    unsigned long long c1 = clock64(), w1 = wall_clock64();
    if (threadIdx.x == 0) { out[0] = c1 - c0; out[1] = w1 - w0; out[2] = (unsigned long long)x; }
}

typedef void (*kfn)(uint32_t*, uint32_t);
struct E { const char* n; kfn f; int static_lds = 0; };
int main(int argc, char** argv) {
    const bool all = argc > 1 && argv[1][0] == '-' && argv[1][1] == '-' && argv[1][2] == 'a';
    uint32_t* d; (void)hipMalloc(&d, 8192);
    unsigned long long* dc; (void)hipMalloc(&dc, 64); unsigned long long hc[3];
    E ks[] = {{"v_mov_b32", k_mov}, {"v_fma_f32", k_fma_f32}, {"v_pk_mul_f16", k_pk_mul},
              {"v_pk_fma_f16", k_pk_fma}, {"v_dot2c_f32_f16", k_dot2c},
              {"v_perm_b32", k_perm}, {"v_fma_mix_f32", k_fma_mix},
              {"v_lshlrev_b32", k_lshl}, {"v_add_f32_dpp (bank-masked)", k_add_dpp},
              {"v_dot2_f32_f16 (3-operand)", k_dot2}, {"pk_fma dep-chain", k_pk_fma_dep},
              {"ds_read_b64 lut-pattern", k_lds64, 65536}};
    E survey[] = {{"v_mov_b32", k_mov}, {"v_fma_f32", k_fma_f32}, {"v_add_f32", k_add_f32}, {"v_mul_f32", k_mul_f32},
                  {"v_max_f32", k_max_f32}, {"v_and_b32", k_and}, {"v_or_b32", k_or}, {"v_xor_b32", k_xor},
                  {"v_add_u32", k_add_u32}, {"v_bfe_u32", k_bfe}, {"v_bfi_b32", k_bfi}, {"v_and_or_b32", k_and_or},
                  {"v_lshl_or_b32", k_lshl_or}, {"v_lshl_add_u32", k_lshl_add}, {"v_add3_u32", k_add3},
                  {"v_or3_b32", k_or3}, {"v_alignbit_b32", k_alignbit}, {"v_lshrrev_b32", k_lshr},
                  {"v_mul_u32_u24", k_mul_u24}, {"v_mad_u32_u24", k_mad_u24}, {"v_cndmask_b32", k_cndmask},
                  {"v_mul_f16", k_mul_f16}, {"v_add_f16", k_add_f16}, {"v_fma_f16", k_fma_f16},
                  {"v_pk_add_f16", k_pk_add}, {"v_cvt_f32_f16", k_cvt_f32_f16}, {"v_cvt_f16_f32", k_cvt_f16_f32},
                  {"v_or_b32_sdwa (byte sel)", k_sdwa_or}, {"v_mov_b32_dpp quad_perm", k_mov_dpp},
                  {"v_add_f32_dpp quad_perm", k_add_dpp_full}, {"v_rcp_f32", k_rcp}, {"v_exp_f32", k_exp},
                  {"fma_f32 dep-chain", k_fma_f32_dep}, {"pk_mul dep-chain", k_pk_mul_dep}};
    hipEvent_t e0, e1; (void)hipEventCreate(&e0); (void)hipEventCreate(&e1);
    // warm the clocks
    for (int w = 0; w < 200; w++) hipLaunchKernelGGL(k_pk_fma, dim3(1024), dim3(256), 0, 0, d, 1u);
    (void)hipDeviceSynchronize();
    hipLaunchKernelGGL(k_clock, dim3(1), dim3(64), 0, 0, dc); (void)hipDeviceSynchronize();
    (void)hipMemcpy(hc, dc, 24, hipMemcpyDeviceToHost);
    printf("clock64 ticks %llu, wall_clock64 ticks %llu (100 MHz) -> clock64 rate %.1f MHz; 2M dependent fma => %.2f clock64 ticks per fma\n",
           hc[0], hc[1], hc[0] * 100.0 / hc[1], hc[0] / 2e6);
    // Placement is forced through the LDS request: one workgroup of 4 * wps waves per CU asks for
    // 96 KB (a second one cannot join it), eight waves per SIMD are two 16-wave workgroups of 72 KB.
    // Left to itself the dispatcher does not spread small workgroups evenly over the CUs.
    auto time_one = [&](const E& k, int wps) {
        const int blocks = wps == 8 ? 512 : 256, threads = wps == 8 ? 1024 : 256 * wps;
        const size_t lds = (wps == 8 ? 72 * 1024 : 96 * 1024) - k.static_lds;
        (void)hipFuncSetAttribute((const void*)k.f, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        for (int w = 0; w < 20; w++) hipLaunchKernelGGL(k.f, dim3(blocks), dim3(threads), lds, 0, d, 1u);
        (void)hipDeviceSynchronize();
        (void)hipEventRecord(e0);
        for (int w = 0; w < 20; w++) hipLaunchKernelGGL(k.f, dim3(blocks), dim3(threads), lds, 0, d, 1u);
        (void)hipEventRecord(e1); (void)hipEventSynchronize(e1);
        float ms; (void)hipEventElapsedTime(&ms, e0, e1); ms /= 20;
        double ns_per_inst = ms * 1e6 / ((double)ITER * 16 * wps);
        uint32_t ticks = 0; (void)hipMemcpy(&ticks, d + 1000, 4, hipMemcpyDeviceToHost);
        printf("%-26s %8.3f ms  %6.3f ns/inst/SIMD   wave0: %.2f clock64 ticks/inst, implied clock %.0f MHz\n", k.n, ms, ns_per_inst,
               ticks / (double)(ITER * 16), ticks / (ms * 1e3));
    };
    if (argc > 1 && argv[1][0] == '-' && argv[1][1] == '-' && argv[1][2] == 'm') {
        // nanoseconds per ITERATION per wave-slot (ms / ITER / waves per SIMD): compare rows
        E mix[] = {{"16 pk_fma", k_mix<16, 0, 0>}, {"16 pk_fma + 4 mfma 4x4x4", k_mix<16, 4, 0>},
                   {"16 pk_fma + 8 mfma 4x4x4", k_mix<16, 8, 0>}, {"16 pk_fma + 16 mfma 4x4x4", k_mix<16, 16, 0>},
                   {"16 mfma 4x4x4", k_mix<0, 16, 0>}, {"8 pk_fma + 16 mfma 4x4x4", k_mix<8, 16, 0>},
                   {"16 pk_fma + 4 mfma 16x16x16", k_mix<16, 4, 1>}, {"16 pk_fma + 8 mfma 16x16x16", k_mix<16, 8, 1>},
                   {"16 mfma 16x16x16", k_mix<0, 16, 1>}};
        for (int wps : {2, 4, 8}) {
            printf("--- %d wave(s) per SIMD: ns/inst/SIMD below is the time of one iteration / 16\n", wps);
            for (auto& k : mix) time_one(k, wps);
        }
        return 0;
    }
    int wlist[] = {1, 2, 3, 4, 8};
    for (int wi = 0; wi < 5; wi++) {
        int wps = wlist[wi];
        printf("--- %d wave(s) per SIMD\n", wps);
        for (auto& k : ks) time_one(k, wps);
        if (all && (wps == 4 || wps == 8)) {
            printf("--- survey, %d wave(s) per SIMD\n", wps);
            for (auto& k : survey) time_one(k, wps);
        }
    }
    return 0;
}
