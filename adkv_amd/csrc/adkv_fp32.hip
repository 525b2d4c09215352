// fp32 ("train/eval") form of the ADKV recurrence for gfx950.
//
// Restates, per (batch, channel), the step of src/adkv/train/train_model.py:8-22,61-81 and of its
// Triton twin src/adkv/hf/llama_adkv_eval.py:86-97: every operation is a separately rounded fp32
// operation (this file is compiled with contraction off and IEEE division), so results are
// bit-identical to an unfused CPU evaluation.
//
//   s  = max(sc, 1e-8);  q = clamp(rint((x - zp) / s), QL, QU);  r = q*s;  xhat = r + zp
//   zp = zp + alpha*r;   sc = clamp(sc + (sc*beta)*(|q| - tgt), sc_min, sc_max)
//
// One lane owns one channel and walks the tokens in order; loads run LOOKAHEAD tokens ahead of the
// dependent chain.  The path is latency-bound (one IEEE divide per token on the critical path).
#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <stdint.h>

#include "../../include/adkv_hip.h"

#pragma clang fp contract(off)

namespace adkv_fp32 {

constexpr int BLK = 64;
constexpr int LOOKAHEAD = 8;

template <typename T> struct IO;
template <> struct IO<float> {
    static __device__ __forceinline__ float ld(const float *p) { return *p; }
    static __device__ __forceinline__ void st(float *p, float v) { *p = v; }
};
template <> struct IO<_Float16> {
    static __device__ __forceinline__ float ld(const _Float16 *p) { return (float)*p; }
    static __device__ __forceinline__ void st(_Float16 *p, float v) { *p = (_Float16)v; }
};
template <> struct IO<__hip_bfloat16> {
    static __device__ __forceinline__ float ld(const __hip_bfloat16 *p)
    {
        return __uint_as_float((uint32_t)*reinterpret_cast<const uint16_t *>(p) << 16);
    }
    static __device__ __forceinline__ void st(__hip_bfloat16 *p, float v)
    {
        // round to nearest even; NaN stays NaN
        uint32_t u = __float_as_uint(v);
        uint16_t h = (v != v) ? (uint16_t)((u >> 16) | 0x40) : (uint16_t)((u + 0x7FFF + ((u >> 16) & 1)) >> 16);
        *reinterpret_cast<uint16_t *>(p) = h;
    }
};

// torch.clamp semantics: NaN passes through
__device__ __forceinline__ float clamp_keep_nan(float x, float lo, float hi)
{
    if (x != x)
        return x;
    return x < lo ? lo : (x > hi ? hi : x);
}

template <typename T>
__global__ __launch_bounds__(BLK) void quant_kernel(
    const T *__restrict__ x, T *xhat, int8_t *__restrict__ codes, float *__restrict__ zp_io,
    float *__restrict__ sc_io, const float *__restrict__ zp0, const float *__restrict__ sc0,
    const float *__restrict__ alpha, const float *__restrict__ beta, const float *__restrict__ tgt,
    float *__restrict__ zp_seq, float *__restrict__ sc_seq,
    int Tn, int C, long stride_b, long stride_t, float ql, float qu, float sc_min, float sc_max)
{
    const int c = blockIdx.x * BLK + threadIdx.x;
    const int b = blockIdx.y;
    if (c >= C)
        return;
    const long bc = (long)b * C + c;
    float zp = zp0 ? zp0[c] : zp_io[bc];
    float sc = sc0 ? sc0[c] : sc_io[bc];
    const float al = alpha[c], be = beta[c], tg = tgt[c];
    const T *xp = x + b * stride_b + c;
    T *op = xhat ? xhat + b * stride_b + c : nullptr;
    const long dense = (long)b * Tn * C + c; // codes / zp_seq / sc_seq are contiguous [B, T, C]

    float buf[LOOKAHEAD];
#pragma unroll
    for (int i = 0; i < LOOKAHEAD; i++)
        buf[i] = i < Tn ? IO<T>::ld(xp + i * stride_t) : 0.0f;

    for (int t0 = 0; t0 < Tn; t0 += LOOKAHEAD) {
#pragma unroll
        for (int i = 0; i < LOOKAHEAD; i++) {
            const int t = t0 + i;
            if (t >= Tn)
                break;
            const float xv = buf[i];
            if (t + LOOKAHEAD < Tn)
                buf[i] = IO<T>::ld(xp + (long)(t + LOOKAHEAD) * stride_t);
            if (zp_seq)
                zp_seq[dense + (long)t * C] = zp;
            if (sc_seq)
                sc_seq[dense + (long)t * C] = sc;
            const float s = (sc != sc) ? sc : (sc < 1e-8f ? 1e-8f : sc);
            const float r = xv - zp;
            const float u = r / s;
            const float q = clamp_keep_nan(__builtin_rintf(u), ql, qu);
            const float xr = q * s;
            if (op)
                IO<T>::st(op + (long)t * stride_t, xr + zp);
            if (codes)
                codes[dense + (long)t * C] = (q != q) ? (int8_t)0 : (int8_t)q;
            const float ax = al * xr;
            const float e = __builtin_fabsf(q) - tg;
            const float sb = sc * be;
            const float sbe = sb * e;
            zp = zp + ax;
            sc = clamp_keep_nan(sc + sbe, sc_min, sc_max);
        }
    }
    if (zp_io) {
        zp_io[bc] = zp;
        sc_io[bc] = sc;
    }
}

} // namespace adkv_fp32

extern "C" int adkv_quant_f32(const void *x, void *xhat, void *codes, void *zp_state, void *sc_state,
                              const void *zp_init, const void *sc_init, const void *alpha,
                              const void *beta, const void *tgt, void *zp_seq, void *sc_seq,
                              int B, int T, int C, int64_t stride_b, int64_t stride_t, int x_dtype,
                              int lower_limit, int upper_limit, float sc_min, float sc_max,
                              void *stream)
{
    using namespace adkv_fp32;
    if (!x || !alpha || !beta || !tgt)
        return ADKV_E_NULL;
    if ((zp_state == nullptr) != (sc_state == nullptr) || (zp_init == nullptr) != (sc_init == nullptr))
        return ADKV_E_NULL;
    if (!zp_state && !zp_init)
        return ADKV_E_NULL; // no starting state at all
    if (B <= 0 || C <= 0 || T < 0 || B > 65535 || stride_t < C || stride_b < 0)
        return ADKV_E_SHAPE;
    if (lower_limit > 0 || upper_limit < 0 || lower_limit < -128 || upper_limit > 127)
        return ADKV_E_UNSUPPORTED;
    if (T == 0 && !(zp_init && zp_state))
        return ADKV_OK;
    const dim3 grid((unsigned)((C + BLK - 1) / BLK), (unsigned)B), block(BLK);
    hipStream_t st = (hipStream_t)stream;
#define ADKV_Q32(TYPE)                                                                              \
    hipLaunchKernelGGL(quant_kernel<TYPE>, grid, block, 0, st, (const TYPE *)x, (TYPE *)xhat,       \
                       (int8_t *)codes, (float *)zp_state, (float *)sc_state, (const float *)zp_init, \
                       (const float *)sc_init, (const float *)alpha, (const float *)beta,           \
                       (const float *)tgt, (float *)zp_seq, (float *)sc_seq, T, C, (long)stride_b,  \
                       (long)stride_t, (float)lower_limit, (float)upper_limit, sc_min, sc_max)
    switch (x_dtype) {
    case ADKV_DT_F32: ADKV_Q32(float); break;
    case ADKV_DT_F16: ADKV_Q32(_Float16); break;
    case ADKV_DT_BF16: ADKV_Q32(__hip_bfloat16); break;
    default: return ADKV_E_UNSUPPORTED;
    }
#undef ADKV_Q32
    return hipGetLastError() == hipSuccess ? ADKV_OK : ADKV_E_LAUNCH;
}
