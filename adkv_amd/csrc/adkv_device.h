// Device-side building blocks of the ADKV kernels (gfx950, wave64).
//
// Arithmetic contract (reference: src/adkv/kernel/gemv.cu:79-88,150-164,220-221): the per-channel
// state (zp, sc) is fp16 and every step below is ONE IEEE round-to-nearest-even fp16 operation, so
// the state trajectory is bit-identical to the reference's half2 code.  This file must be compiled
// with -ffp-contract=off: "q*sc + zp" has to stay two roundings where the reference has two.
#pragma once

#include <hip/hip_runtime.h>
#include <type_traits>
#include <utility>
#include <stdint.h>

#pragma clang fp contract(off)

namespace adkv {

typedef _Float16 h1;
typedef _Float16 h2 __attribute__((ext_vector_type(2)));

// operand types of v_mfma_f32_4x4x4_16B_f16: four fp16 (two registers), four fp32
typedef float f4v __attribute__((ext_vector_type(4)));
typedef _Float16 h4v __attribute__((ext_vector_type(4)));
__device__ __forceinline__ h4v as_h4(uint32_t lo, uint32_t hi)
{
    return __builtin_bit_cast(h4v, make_uint2(lo, hi));
}
__device__ __forceinline__ h2 as_h2(uint32_t u) { return __builtin_bit_cast(h2, u); }
__device__ __forceinline__ uint32_t as_u32(h2 h) { return __builtin_bit_cast(uint32_t, h); }
__device__ __forceinline__ h2 pk_fma(h2 a, h2 b, h2 c) { return __builtin_elementwise_fma(a, b, c); }
__device__ __forceinline__ h2 pk_abs(h2 a) { return as_h2(as_u32(a) & 0x7FFF7FFFu); }
__device__ __forceinline__ h2 splat(h1 x) { return (h2){x, x}; }

// f(integral_constant<int, 0>), ..., f(integral_constant<int, N-1>): a loop whose index is a
// compile-time constant inside the body (register arrays indexed by it stay in registers).
template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F &&f, std::integer_sequence<int, I...>)
{
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f)
{
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// A decode loop over n items whose buffers rotate with period P: whole rotations without a
// single condition in them (conditions around loads or stores make the compiler wait for every
// load in flight), then the up to P-1 items left.  body(item, integral_constant slot).
template <int P, typename F>
__device__ __forceinline__ void rotate_over(int n, F &&body)
{
    int i0 = 0;
    for (; i0 + P <= n; i0 += P)
        static_for<P>([&](auto ic) { body(i0 + decltype(ic)::value, ic); });
    static_for<P - 1>([&](auto ic) {
        if (i0 + decltype(ic)::value < n)
            body(i0 + decltype(ic)::value, ic);
    });
}

// Activations (q, the new K / V token, the attention output) may be stored as bfloat16 instead of
// fp16: they are rounded to fp16 as they are read (bf16 -> fp32 is exact, fp32 -> fp16 rounds to
// nearest even: torch's .to(float16)) and the fp16 result is rounded to bf16 as it is written
// (torch's .to(bfloat16)), so values are those of the reference's conversions around its kernels
// (src/adkv/hf/llama_adkv.py:248-250, 274).  `bf16` is uniform over the launch.
__device__ __forceinline__ h2 load_act2(const h1 *p, int bf16)
{
    const uint32_t w = *reinterpret_cast<const uint32_t *>(p);
    if (bf16)
        return (h2){(h1)__uint_as_float(w << 16), (h1)__uint_as_float(w & 0xFFFF0000u)};
    return as_h2(w);
}

__device__ __forceinline__ uint32_t bf16_bits(h1 v)
{
    const uint32_t u = __float_as_uint((float)v);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u)
        return (u >> 16) | 0x40u; // NaN stays NaN
    return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}

__device__ __forceinline__ void store_act2(h1 *p, float a, float b, int bf16)
{
    const h2 v = {(h1)a, (h1)b};
    if (bf16)
        *reinterpret_cast<uint32_t *>(p) = bf16_bits(v.x) | (bf16_bits(v.y) << 16);
    else
        *reinterpret_cast<h2 *>(p) = v;
}

// One channel pair's filter state and fixed parameters (two channels packed per register).
struct Pair {
    h2 zp, sc, al, be, omt;
};

// Loads the pair starting at parameter index pi (even).  omt = 1 - beta*target with both steps
// rounded to fp16 (gemv.cu:220-221).
__device__ __forceinline__ void load_pair(Pair &p, const h1 *zp, const h1 *sc, const h1 *al,
                                          const h1 *be, const h1 *tg, int pi)
{
    p.zp = *reinterpret_cast<const h2 *>(zp + pi);
    p.sc = *reinterpret_cast<const h2 *>(sc + pi);
    p.al = *reinterpret_cast<const h2 *>(al + pi);
    p.be = *reinterpret_cast<const h2 *>(be + pi);
    const h2 t = *reinterpret_cast<const h2 *>(tg + pi);
    const h2 bt = p.be * t;
    p.omt = splat((h1)1.0f) - bt;
}

// EMA update with an already computed qs = r16(q*sc) (gemv.cu:158-164):
//   zp <- r16(alpha*qs + zp)   sc <- r16(sc * r16(beta*|q| + omt))
__device__ __forceinline__ void update_pair(Pair &p, h2 q, h2 qs)
{
    p.zp = pk_fma(p.al, qs, p.zp);
    const h2 f = pk_fma(p.be, pk_abs(q), p.omt);
    p.sc = p.sc * f;
}

// ---------------------------------------------------------------------------------------------
// Code-pair lookup table in LDS.
//
// Decoding a nibble pair in registers costs ~4.5 VALU ops per channel-pair-token (byte permute,
// mask, or, bias subtract, abs) and the scan is VALU-issue-bound, so the conversion is moved to
// the otherwise idle LDS pipe: the byte b = code_A | code_B << 4 of one token indexes a table whose
// entry holds the fp16 pair (q_A, q_B) and its absolute value.  Entry stride is 256 B = 32 copies of
// the 8-byte entry; lane l reads copy l % 32, so the 16 lanes a ds_read_b64 serves per clock always
// hit 16 distinct bank pairs, whatever their codes are.  Address = (b << 8) | (copy << 3) is built
// by ONE v_perm_b32 from the packed code word and a per-lane constant.
// ---------------------------------------------------------------------------------------------
constexpr int LUT_ENTRIES = 256;
constexpr int LUT_COPIES = 32;
constexpr int LUT_WORDS64 = LUT_ENTRIES * LUT_COPIES; // uint2 elements = 64 KB

__device__ __forceinline__ void lut_fill(uint2 *lut, int tid, int nthreads)
{
    for (int i = tid; i < LUT_WORDS64; i += nthreads) {
        const int b = i / LUT_COPIES;
        const h2 q = (h2){(h1)((b & 15) - 8), (h1)((b >> 4) - 8)};
        lut[i] = make_uint2(as_u32(q), as_u32(q) & 0x7FFF7FFFu);
    }
}

// Channel words A, B (8 codes each, token i at bits 4i..4i+3) -> per-token code bytes:
// even.byte[k] = token 2k, odd.byte[k] = token 2k+1, each byte = code_A | code_B << 4.
__device__ __forceinline__ void pair_bytes(uint32_t wa, uint32_t wb, uint32_t &even, uint32_t &odd)
{
    constexpr uint32_t m = 0x0F0F0F0Fu;
    even = (wa & m) | ((wb << 4) & ~m);
    odd = ((wa >> 4) & m) | (wb & ~m);
}

// lane_copy = (lane % 32) * 8.  Returns (q pair, |q| pair) of byte k (0..3) of `bytes`.  k must be
// a compile-time constant after unrolling (the selector becomes a literal).
__device__ __forceinline__ uint2 lut_get(const uint2 *lut, uint32_t bytes, uint32_t lane_copy, int k)
{
    const uint32_t sel = 0x0C0C0000u | ((4u + (uint32_t)k) << 8); // [0, 0, bytes.byte[k], lane_copy.byte[0]]
    const uint32_t addr = __builtin_amdgcn_perm(bytes, lane_copy, sel);
    return *reinterpret_cast<const uint2 *>(reinterpret_cast<const char *>(lut) + addr);
}

// EMA update given qs = r16(q*sc) and |q| (gemv.cu:158-164).
__device__ __forceinline__ void update_pair_abs(Pair &p, h2 qabs, h2 qs)
{
    p.zp = pk_fma(p.al, qs, p.zp);
    const h2 f = pk_fma(p.be, qabs, p.omt);
    p.sc = p.sc * f;
}

// Code width.  4 bits is the reference's format (8 tokens per 32-bit channel word, codes in
// [-8, 7], stored as q + 8).  2 bits is the same recurrence over codes in [-2, 1] (the range the
// reference's train model uses for bits = 2, train_model.py:96-97), stored as q + 2, 16 tokens per
// word; the reference has no kernel for it.
template <int BITS>
struct Code {
    static_assert(BITS == 2 || BITS == 4, "code width");
    static constexpr int TPW = 32 / BITS;                 // tokens per channel word = per supergroup
    static constexpr int QLO = -(1 << (BITS - 1));
    static constexpr int QHI = (1 << (BITS - 1)) - 1;
    static constexpr uint32_t FIELD = (1u << BITS) - 1u;
    static constexpr uint32_t BIAS = BITS == 4 ? 0x88888888u : 0xAAAAAAAAu; // -QLO in every field
};

// gemv.cu:150-154: fp32 subtract, IEEE fp32 divide, round-half-even, NaN -> 0, clamp to [-8,7].
template <int BITS = 4>
__device__ __forceinline__ int quantize(h1 x, h1 zp, h1 sc)
{
    const float d = (float)x - (float)zp;
    const float u = d / (float)sc;
    float r = __builtin_rintf(u);
    r = (u != u) ? 0.0f : r;
    r = __builtin_fminf(__builtin_fmaxf(r, (float)Code<BITS>::QLO), (float)Code<BITS>::QHI);
    return (int)r;
}

// The encoder's form of quantize(): the same value with as few dependent instructions between
// one token's state and the next as the arithmetic allows.
//  * x - zp is one mixed-precision fma on the fp16 halves in place (f32(x)*1 - f32(zp), rounded
//    once: exactly the reference's fp32 difference) instead of two conversions and a subtract.
//  * rsc is the hardware reciprocal of sc (1 ulp), taken as soon as sc is known.  r = d*rsc is
//    within 2^-22 relative of the exact quotient u, so for |r| < 16 it is within 2^-18 absolute:
//    unless r lies closer than 2^-16 to a rounding boundary k + 1/2, rint(r) == rint(u) (exact
//    ties always land in that band).  For |r| >= 16 both u and r are beyond the clamp on the same
//    side, whatever rint gives.  Inside the band, and for NaN (which ends as code 0, like CUDA's
//    __float2int_rn), the exact divide decides; that branch is taken by about one element in
//    30 000.
//  * The result is the clamped code as a float (an integer in [QLO, QHI]): the fp16 operands of
//    the state update are converted from it directly, the integer for the code word off the
//    critical path.
// xw / zpw hold the fp16 operands in their low (HI = false) or high (HI = true) halves.
template <int BITS, bool HI>
__device__ __forceinline__ float quantize_enc_fast(uint32_t xw, uint32_t zpw, h1 sc, float rsc)
{
    float d;
    if (HI)
        asm("v_fma_mix_f32 %0, %1, 1.0, -%2 op_sel:[1,0,1] op_sel_hi:[1,0,1]" : "=v"(d) : "v"(xw), "v"(zpw));
    else
        asm("v_fma_mix_f32 %0, %1, 1.0, -%2 op_sel_hi:[1,0,1]" : "=v"(d) : "v"(xw), "v"(zpw));
    const float r = d * rsc;
    float n = __builtin_rintf(r);
    if (__builtin_expect(!(__builtin_fabsf(r - n) < 0.5f - 0x1p-16f), 0)) {
        n = __builtin_rintf(d / (float)sc);
        n = (n != n) ? 0.0f : n;
    }
    return __builtin_amdgcn_fmed3f(n, (float)Code<BITS>::QLO, (float)Code<BITS>::QHI);
}

// quantize_enc_fast without its branch, for lanes whose wave is alone on its SIMD and pays every
// dependent instruction in full: the code is taken from the reciprocal product unconditionally and
// the squared distance of r from its integer is folded into `worst` as an unsigned maximum (a NaN
// has the largest bit pattern of all).  A caller that finds worst >= ENC_SPEC_LIMIT afterwards
// must discard the codes and the state derived from them and redo the tokens with
// quantize_enc_fast.  Squaring is monotonic, so every |r - n| >= 0.5 - 2^-16 is caught.
constexpr float ENC_SPEC_EDGE = 0.5f - 0x1p-16f;
constexpr float ENC_SPEC_LIMIT = ENC_SPEC_EDGE * ENC_SPEC_EDGE;
template <int BITS, bool HI>
__device__ __forceinline__ float quantize_enc_spec(uint32_t xw, uint32_t zpw, float rsc, uint32_t &worst)
{
    float d;
    if (HI)
        asm("v_fma_mix_f32 %0, %1, 1.0, -%2 op_sel:[1,0,1] op_sel_hi:[1,0,1]" : "=v"(d) : "v"(xw), "v"(zpw));
    else
        asm("v_fma_mix_f32 %0, %1, 1.0, -%2 op_sel_hi:[1,0,1]" : "=v"(d) : "v"(xw), "v"(zpw));
    const float r = d * rsc;
    const float n = __builtin_rintf(r);
    const float e = r - n;
    const uint32_t e2 = __float_as_uint(e * e);
    worst = worst > e2 ? worst : e2;
    return __builtin_amdgcn_fmed3f(n, (float)Code<BITS>::QLO, (float)Code<BITS>::QHI);
}

// Two small integers held as floats -> fp16 pair (exact, so the rounding mode is irrelevant).
__device__ __forceinline__ h2 pack_codes(float a, float b)
{
    return __builtin_bit_cast(h2, __builtin_amdgcn_cvt_pkrtz(a, b));
}

__device__ __forceinline__ h2 codes_to_h2(int q0, int q1) { return (h2){(h1)q0, (h1)q1}; }

// Quantise one new token's channel pair with the current state and patch its two codes into the
// channel words at token slot tt of the supergroup (gemv.cu:91-146).  Returns the code pair.
template <int BITS = 4>
__device__ __forceinline__ h2 append_pair(uint32_t &wa, uint32_t &wb, int tt, h2 x, const Pair &p)
{
    const int q0 = quantize<BITS>(x.x, p.zp.x, p.sc.x);
    const int q1 = quantize<BITS>(x.y, p.zp.y, p.sc.y);
    const uint32_t sh = (uint32_t)BITS * (uint32_t)tt;
    const uint32_t m = ~(Code<BITS>::FIELD << sh);
    wa = (wa & m) | (((uint32_t)(q0 - Code<BITS>::QLO) & Code<BITS>::FIELD) << sh);
    wb = (wb & m) | (((uint32_t)(q1 - Code<BITS>::QLO) & Code<BITS>::FIELD) << sh);
    return codes_to_h2(q0, q1);
}

// Code pair of token slot tt straight from the channel words (ragged tails only).
template <int BITS>
__device__ __forceinline__ h2 extract_pair(uint32_t wa, uint32_t wb, int tt)
{
    const uint32_t sh = (uint32_t)BITS * (uint32_t)tt;
    return codes_to_h2((int)((wa >> sh) & Code<BITS>::FIELD) + Code<BITS>::QLO,
                       (int)((wb >> sh) & Code<BITS>::FIELD) + Code<BITS>::QLO);
}

// ---------------------------------------------------------------------------------------------
// 2-bit codes: the table is indexed by a byte that holds TWO tokens of a channel pair and returns
// 16 bytes, (q, |q|) for the low nibble's token then for the high nibble's.  16 copies per entry
// (256-byte stride again, same 64 KB): a ds_read_b128 serves 16 lanes per clock.
//   even.byte[j] = tokens 4j (low nibble) and 4j+2;  odd.byte[j] = tokens 4j+1 and 4j+3;
//   nibble = code_A | code_B << 2.
// ---------------------------------------------------------------------------------------------
constexpr int LUT2_COPIES = 16;

__device__ __forceinline__ void lut2_fill(uint2 *lut, int tid, int nthreads)
{
    uint4 *l4 = reinterpret_cast<uint4 *>(lut);
    for (int i = tid; i < LUT_ENTRIES * LUT2_COPIES; i += nthreads) {
        const int b = i / LUT2_COPIES;
        const h2 lo = (h2){(h1)((b & 3) - 2), (h1)(((b >> 2) & 3) - 2)};
        const h2 hi = (h2){(h1)(((b >> 4) & 3) - 2), (h1)((b >> 6) - 2)};
        l4[i] = make_uint4(as_u32(lo), as_u32(lo) & 0x7FFF7FFFu, as_u32(hi), as_u32(hi) & 0x7FFF7FFFu);
    }
}

__device__ __forceinline__ void pair_bytes2(uint32_t wa, uint32_t wb, uint32_t &even, uint32_t &odd)
{
    constexpr uint32_t m = 0x33333333u;
    even = (wa & m) | ((wb & m) << 2);
    odd = ((wa >> 2) & m) | (wb & ~m);
}

// lane_copy = (lane % 16) * 16.  k: byte of `bytes`, a compile-time constant after unrolling.
__device__ __forceinline__ uint4 lut2_get(const uint2 *lut, uint32_t bytes, uint32_t lane_copy, int k)
{
    const uint32_t sel = 0x0C0C0000u | ((4u + (uint32_t)k) << 8);
    const uint32_t addr = __builtin_amdgcn_perm(bytes, lane_copy, sel);
    return *reinterpret_cast<const uint4 *>(reinterpret_cast<const char *>(lut) + addr);
}

} // namespace adkv
