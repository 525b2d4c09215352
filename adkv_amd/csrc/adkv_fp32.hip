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
// One lane owns one channel and walks the tokens in order; loads run three groups of 8 tokens
// ahead of the dependent chain.  The path is bound by the length of that chain per token, not by
// memory.
#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <stdint.h>

#include "../../include/adkv_hip.h"
#include "adkv_device.h"

#pragma clang fp contract(off)

namespace adkv_fp32 {

constexpr int BLK = 64;

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

// One token of one channel.  The quotient is first taken with the hardware reciprocal of s (kept
// from the previous token, off the dependent chain): r = d*rs is within 2^-22 relative of the
// exact u = d/s, so rint(r) == rint(u) unless r lies closer than 2^-16 + |r|*2^-20 (four times the
// error bound) to a rounding boundary k + 1/2, or is NaN; in that band the IEEE divide decides.
// Everything after the rounding is the reference's separately rounded fp32 sequence.
struct Chan {
    float zp, sc, s, rs; // s = max(sc, 1e-8) (NaN kept), rs ~ 1/s
    float al, be, tg;
    __device__ __forceinline__ void set_scale(float v)
    {
        sc = v;
        s = (v != v) ? v : (v < 1e-8f ? 1e-8f : v);
        rs = __builtin_amdgcn_rcpf(s);
    }
    __device__ __forceinline__ float step(float xv, float ql, float qu, float sc_min, float sc_max, float &q)
    {
        const float d = xv - zp;
        const float r = d * rs;
        float n = __builtin_rintf(r);
        const float margin = __builtin_fmaf(__builtin_fabsf(r), 0x1p-20f, 0x1p-16f);
        if (__builtin_expect(!(__builtin_fabsf(r - n) < 0.5f - margin), 0))
            n = __builtin_rintf(d / s);
        q = clamp_keep_nan(n, ql, qu);
        const float xr = q * s;
        const float xh = xr + zp;
        const float ax = al * xr;
        const float e = __builtin_fabsf(q) - tg;
        const float sb = sc * be;
        const float sbe = sb * e;
        zp = zp + ax;
        set_scale(clamp_keep_nan(sc + sbe, sc_min, sc_max));
        return xh;
    }
    // The same token without a branch or a NaN test, for lanes that pay every dependent
    // instruction in full (few channels: each wave has a SIMD to itself).  The result is only
    // valid if `worst` stays below SPEC_LIMIT: it takes the unsigned maximum of the bit patterns
    // of  |r - n| + |r|*2^-20  (at or above 0.5 - 2^-15 whenever step() would have divided; a NaN
    // or infinite r gives a NaN, whose pattern is above every number's) and of  raw - raw  for the
    // unclamped new scale (0, or a NaN when raw is not finite: the clamps here drop NaNs, the
    // reference's keep them).  A caller that finds worst >= SPEC_LIMIT restores the state it
    // saved and redoes the tokens with step().
    __device__ __forceinline__ float step_spec(float xv, float ql, float qu, float sc_min, float sc_max,
                                               float &q, uint32_t &worst)
    {
        const float d = xv - zp;
        const float r = d * rs;
        const float n = __builtin_rintf(r);
        q = __builtin_amdgcn_fmed3f(n, ql, qu);
        const float t = __builtin_fmaf(__builtin_fabsf(r), 0x1p-20f, __builtin_fabsf(r - n));
        const float xr = q * s;
        const float xh = xr + zp;
        const float ax = al * xr;
        const float e = __builtin_fabsf(q) - tg;
        const float sb = sc * be;
        const float sbe = sb * e;
        zp = zp + ax;
        const float raw = sc + sbe;
        const float u = raw - raw;
        const uint32_t tb = __float_as_uint(t), ub = __float_as_uint(u);
        worst = max(worst, max(tb, ub));
        sc = __builtin_amdgcn_fmed3f(raw, sc_min, sc_max);
        s = __builtin_amdgcn_fmed3f(sc, 1e-8f, __builtin_inff()); // max(sc, 1e-8) without a NaN pass
        rs = __builtin_amdgcn_rcpf(s);
        return xh;
    }
};
constexpr float SPEC_LIMIT = 0.5f - 0x1p-15f;

constexpr int GRP = 8;  // tokens per group: the unit of speculation and of the input rotation
constexpr int NBUF = 4; // groups of input in rotation (loads run NBUF-1 groups ahead)

// x and xhat are declared non-aliasing although the caller may pass the same buffer (in-place
// use): every element is loaded before the token that stores to it is computed and is never read
// again, so no ordering between a store and a later load matters; without the promise the
// compiler serialises every prefetched load behind the stores.
//
// WIDE (16-bit inputs only): a lane loads the aligned 32-bit word its channel lies in and picks
// its half at use, so the values in flight are plain 32-bit registers with no arithmetic on
// them; 16-bit loads would be zero-extended or packed in pairs at the loop edge, which makes
// every group wait out the memory latency.  The launcher uses it when the layout allows (even C
// and strides, 4-byte aligned base).
template <typename T, bool WIDE, bool SEQ, bool OUT, bool CODES>
__global__ __launch_bounds__(BLK) void quant_kernel(
    const T *__restrict__ x, T *__restrict__ xhat, int8_t *__restrict__ codes, float *__restrict__ zp_io,
    float *__restrict__ sc_io, const float *__restrict__ zp0, const float *__restrict__ sc0,
    const float *__restrict__ alpha, const float *__restrict__ beta, const float *__restrict__ tgt,
    float *__restrict__ zp_seq, float *__restrict__ sc_seq,
    int Tn, int C, long stride_b, long stride_t, float ql, float qu, float sc_min, float sc_max)
{
    static_assert(!WIDE || sizeof(T) == 2, "wide loads are for 16-bit inputs");
    using Raw = typename std::conditional<sizeof(T) == 4, float, typename std::conditional<WIDE, uint32_t, T>::type>::type;
    const int c = blockIdx.x * BLK + threadIdx.x;
    const int b = blockIdx.y;
    if (c >= C)
        return;
    const long bc = (long)b * C + c;
    Chan ch;
    ch.zp = zp0 ? zp0[c] : zp_io[bc];
    ch.set_scale(sc0 ? sc0[c] : sc_io[bc]);
    ch.al = alpha[c];
    ch.be = beta[c];
    ch.tg = tgt[c];
    const T *xp = x + b * stride_b + c;
    T *op = OUT ? xhat + b * stride_b + c : nullptr;
    const long dense = (long)b * Tn * C + c; // codes / zp_seq / sc_seq are contiguous [B, T, C]
    const uint32_t half_shift = WIDE ? (uint32_t)(c & 1) * 16u : 0u;

    auto load_raw = [&](long t) __attribute__((always_inline)) -> Raw {
        if constexpr (WIDE)
            return *reinterpret_cast<const uint32_t *>(xp - (c & 1) + t * stride_t);
        else if constexpr (sizeof(T) == 4)
            return *reinterpret_cast<const float *>(xp + t * stride_t);
        else
            return xp[t * stride_t];
    };
    auto value = [&](Raw r) __attribute__((always_inline)) -> float {
        if constexpr (WIDE) {
            const uint16_t hb = (uint16_t)(r >> half_shift);
            return IO<T>::ld(reinterpret_cast<const T *>(&hb));
        } else if constexpr (sizeof(T) == 4) {
            return r;
        } else {
            return IO<T>::ld(&r);
        }
    };
    auto emit = [&](int t, float xh, float q) __attribute__((always_inline)) {
        if (OUT)
            IO<T>::st(op + (long)t * stride_t, xh);
        if (CODES)
            codes[dense + (long)t * C] = (q != q) ? (int8_t)0 : (int8_t)q;
    };
    // exact path, token by token (also records the state sequence)
    auto one = [&](float xv, int t) __attribute__((always_inline)) {
        if (SEQ) {
            zp_seq[dense + (long)t * C] = ch.zp;
            sc_seq[dense + (long)t * C] = ch.sc;
        }
        float q;
        const float xh = ch.step(xv, ql, qu, sc_min, sc_max, q);
        emit(t, xh, q);
    };

    // Full groups of GRP tokens.  Inputs are loaded NBUF-1 groups ahead, unconditionally (past
    // the last group the same rows are loaded again).  A group is first run speculatively with
    // its results held in registers; if any lane of the wave came near a rounding boundary or met
    // a non-finite value (about one group in thirty) the state is restored and the group is
    // redone exactly.  Recording the state sequence needs the state before every token, so that
    // variant runs the exact path only.
    const int ng = Tn / GRP;
    Raw buf[NBUF][GRP];
    long tnext = 0; // first token of the next group to load
    auto load_next = [&](Raw *dst) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < GRP; i++)
            dst[i] = load_raw(tnext + i);
        if (tnext + GRP < (long)ng * GRP)
            tnext += GRP;
    };
    auto do_group = [&](int g, const Raw *xg) __attribute__((always_inline)) {
        if (SEQ) {
#pragma unroll
            for (int i = 0; i < GRP; i++)
                one(value(xg[i]), g * GRP + i);
            return;
        }
        const Chan saved = ch;
        uint32_t worst = 0u;
        float xh[GRP], q[GRP];
#pragma unroll
        for (int i = 0; i < GRP; i++)
            xh[i] = ch.step_spec(value(xg[i]), ql, qu, sc_min, sc_max, q[i], worst);
        if (__any(worst >= __float_as_uint(SPEC_LIMIT))) {
            ch = saved;
#pragma unroll
            for (int i = 0; i < GRP; i++)
                xh[i] = ch.step(value(xg[i]), ql, qu, sc_min, sc_max, q[i]);
        }
#pragma unroll
        for (int i = 0; i < GRP; i++)
            emit(g * GRP + i, xh[i], q[i]);
    };
    if (ng > 0) {
        adkv::static_for<NBUF - 1>([&](auto ic) { load_next(buf[decltype(ic)::value]); });
        adkv::rotate_over<NBUF>(ng, [&](int g, auto ic) __attribute__((always_inline)) {
            constexpr int i = decltype(ic)::value;
            load_next(buf[(i + NBUF - 1) % NBUF]);
            do_group(g, buf[i]);
        });
    }
    for (int t = ng * GRP; t < Tn; t++)
        one(value(load_raw(t)), t);
    if (zp_io) {
        zp_io[bc] = ch.zp;
        sc_io[bc] = ch.sc;
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
    if ((zp_seq == nullptr) != (sc_seq == nullptr))
        return ADKV_E_NULL;
    if (B <= 0 || C <= 0 || T < 0 || B > 65535 || stride_t < C || stride_b < 0)
        return ADKV_E_SHAPE;
    if (lower_limit > 0 || upper_limit < 0 || lower_limit < -128 || upper_limit > 127)
        return ADKV_E_UNSUPPORTED;
    if (T == 0 && !(zp_init && zp_state))
        return ADKV_OK;
    const dim3 grid((unsigned)((C + BLK - 1) / BLK), (unsigned)B), block(BLK);
    hipStream_t st = (hipStream_t)stream;
#define ADKV_Q32_(TYPE, WIDE, SEQ, OUT, CODES)                                                      \
    hipLaunchKernelGGL((quant_kernel<TYPE, WIDE, SEQ, OUT, CODES>), grid, block, 0, st,             \
                       (const TYPE *)x, (TYPE *)xhat,                                               \
                       (int8_t *)codes, (float *)zp_state, (float *)sc_state, (const float *)zp_init, \
                       (const float *)sc_init, (const float *)alpha, (const float *)beta,           \
                       (const float *)tgt, (float *)zp_seq, (float *)sc_seq, T, C, (long)stride_b,  \
                       (long)stride_t, (float)lower_limit, (float)upper_limit, sc_min, sc_max)
#define ADKV_Q32_O(TYPE, WIDE, SEQ)                                                                 \
    do {                                                                                            \
        if (xhat && codes)                                                                          \
            ADKV_Q32_(TYPE, WIDE, SEQ, true, true);                                                 \
        else if (xhat)                                                                              \
            ADKV_Q32_(TYPE, WIDE, SEQ, true, false);                                                \
        else if (codes)                                                                             \
            ADKV_Q32_(TYPE, WIDE, SEQ, false, true);                                                \
        else                                                                                        \
            ADKV_Q32_(TYPE, WIDE, SEQ, false, false);                                               \
    } while (0)
#define ADKV_Q32(TYPE, WIDE)                                                                        \
    do {                                                                                            \
        if (zp_seq)                                                                                 \
            ADKV_Q32_O(TYPE, WIDE, true);                                                           \
        else                                                                                        \
            ADKV_Q32_O(TYPE, WIDE, false);                                                          \
    } while (0)
#define ADKV_Q32_16(TYPE)                                                                           \
    do {                                                                                            \
        if (wide)                                                                                   \
            ADKV_Q32(TYPE, true);                                                                   \
        else                                                                                        \
            ADKV_Q32(TYPE, false);                                                                  \
    } while (0)
    // 16-bit inputs: aligned 32-bit loads when every row starts on a 4-byte boundary and no
    // channel's word reaches past its row
    const bool wide = (C % 2 == 0) && (stride_t % 2 == 0) && (stride_b % 2 == 0) &&
                      (((uintptr_t)x & 3) == 0);
    switch (x_dtype) {
    case ADKV_DT_F32: ADKV_Q32(float, false); break;
    case ADKV_DT_F16: ADKV_Q32_16(_Float16); break;
    case ADKV_DT_BF16: ADKV_Q32_16(__hip_bfloat16); break;
    default: return ADKV_E_UNSUPPORTED;
    }
#undef ADKV_Q32_16
#undef ADKV_Q32
#undef ADKV_Q32_O
#undef ADKV_Q32_
    return hipGetLastError() == hipSuccess ? ADKV_OK : ADKV_E_LAUNCH;
}
