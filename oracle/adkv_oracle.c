/*
 * ADKV CPU oracle — TEST INFRASTRUCTURE ONLY (see adkv_oracle.h).
 *
 * Scalar restatement of the reference recurrences, written from the reference's source text.
 * fp16 arithmetic is emulated exactly: every operation forms its exact result as a 128-bit
 * fixed-point integer and rounds ONCE to binary16 (round-to-nearest-even, subnormals kept).
 *
 * Build: gcc -O2 -ffp-contract=off -fno-fast-math (see Makefile).  -ffp-contract=off matters for
 * the fp32 path: the reference's fp32 recurrence is unfused.
 *
 * Parity status: the reference ships no tests, fixtures or golden vectors for this path, so no
 * function here is pinned by the reference's own data.  Each function is instead pinned by
 * independent checks in tests/ (exact rational arithmetic, closed forms, byte-level layout brute
 * force, replay invariants).  What those cannot pin is flagged "parity unpinned" at the function.
 */
#include "adkv_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

typedef __int128 i128;
typedef unsigned __int128 u128;
#define P2(k) (((i128)1) << (k)) /* 2^k as a signed 128-bit integer, 0 <= k < 126 */

/* ------------------------------------------------------------------------------------------ */
/* binary16 soft-float                                                                          */
/* ------------------------------------------------------------------------------------------ */

#define H_SIGN 0x8000u
#define H_INF 0x7C00u
#define H_QNAN 0x7E00u

static inline int h_is_nan(uint16_t h) { return (h & 0x7FFFu) > H_INF; }
static inline int h_is_inf(uint16_t h) { return (h & 0x7FFFu) == H_INF; }
static inline int h_is_zero(uint16_t h) { return (h & 0x7FFFu) == 0; }

/* value(h) = sig * 2^lsb_exp, sig signed integer |sig| < 2^11, lsb_exp in [-24, 5] */
static inline void h_unpack(uint16_t h, int *sig, int *lsb_exp)
{
    int e = (h >> 10) & 0x1F;
    int m = h & 0x3FF;
    int s = (h & H_SIGN) ? -1 : 1;
    if (e == 0) {
        *sig = s * m;
        *lsb_exp = -24;
    } else {
        *sig = s * (1024 + m);
        *lsb_exp = e - 25;
    }
}

/* Round mag * 2^unit_exp (mag > 0) to binary16 magnitude bits, RNE.  unit_exp <= -25 so that at
 * least one bit sits below the smallest subnormal step. */
static uint16_t round_mag_to_h(u128 mag, int unit_exp)
{
    int p = 0; /* index of the most significant set bit */
    {
        u128 t = mag;
        while (t >>= 1)
            p++;
    }
    int E = p + unit_exp;            /* value in [2^E, 2^(E+1)) */
    int lsb = (E >= -14) ? (E - 10) : -24; /* exponent of the result's last place */
    int shift = lsb - unit_exp;      /* bits to drop; >= 1 by the precondition on unit_exp */
    u128 q, rem, half;
    if (shift <= 0) {
        q = mag << (-shift);
        rem = 0;
        half = 1;
    } else if (shift >= 127) {
        q = 0;
        rem = 1; /* strictly below half of the smallest step */
        half = 2;
    } else {
        q = mag >> shift;
        rem = mag & ((((u128)1) << shift) - 1);
        half = ((u128)1) << (shift - 1);
    }
    if (rem > half || (rem == half && (q & 1)))
        q++;
    if (lsb == -24) {
        /* subnormal range; q == 1024 carries naturally into the smallest normal */
        return (uint16_t)q;
    }
    int e = lsb + 25;
    if (q == 2048) {
        q = 1024;
        e++;
    }
    if (e >= 31)
        return H_INF;
    return (uint16_t)((e << 10) | ((int)q - 1024));
}

/* exact signed fixed-point value v * 2^unit_exp -> binary16; zero_sign used when v == 0 */
static uint16_t fix_to_h(i128 v, int unit_exp, uint16_t zero_sign)
{
    if (v == 0)
        return zero_sign;
    uint16_t s = 0;
    u128 mag;
    if (v < 0) {
        s = H_SIGN;
        mag = (u128)(-v);
    } else {
        mag = (u128)v;
    }
    return s | round_mag_to_h(mag, unit_exp);
}

float adkv_o_h2f(uint16_t h)
{
    if (h_is_nan(h))
        return NAN;
    if (h_is_inf(h))
        return (h & H_SIGN) ? -INFINITY : INFINITY;
    int sig, le;
    h_unpack(h, &sig, &le);
    if (sig == 0)
        return (h & H_SIGN) ? -0.0f : 0.0f;
    return ldexpf((float)sig, le); /* exact: 11-bit integer scaled by a power of two */
}

uint16_t adkv_o_d2h(double d)
{
    if (d != d)
        return H_QNAN;
    uint16_t s = signbit(d) ? H_SIGN : 0;
    double a = fabs(d);
    if (a == 0.0)
        return s;
    if (isinf(a) || a >= 131072.0)
        return s | H_INF;
    if (a < 0x1p-40)
        return s; /* far below half of the smallest subnormal (2^-25) */
    /* units of 2^-49: integer part exact in u128, plus a sticky bit for anything below */
    double scaled = ldexp(a, 48); /* exact (power-of-two scaling, no overflow/underflow here) */
    double fl = floor(scaled);
    u128 mag = (u128)fl;
    mag = (mag << 1) | (scaled != fl ? 1u : 0u);
    return s | round_mag_to_h(mag, -49);
}

uint16_t adkv_o_f2h(float f) { return adkv_o_d2h((double)f); }

uint16_t adkv_o_hmul(uint16_t a, uint16_t b)
{
    if (h_is_nan(a) || h_is_nan(b))
        return H_QNAN;
    uint16_t s = (a ^ b) & H_SIGN;
    if (h_is_inf(a) || h_is_inf(b)) {
        if (h_is_zero(a) || h_is_zero(b))
            return H_QNAN;
        return s | H_INF;
    }
    int sa, ea, sb, eb;
    h_unpack(a, &sa, &ea);
    h_unpack(b, &sb, &eb);
    i128 p = (i128)sa * (i128)sb * P2(ea + eb + 48); /* units of 2^-48 */
    return fix_to_h(p, -48, s);
}

static uint16_t h_addsub(uint16_t a, uint16_t b)
{
    if (h_is_nan(a) || h_is_nan(b))
        return H_QNAN;
    if (h_is_inf(a) || h_is_inf(b)) {
        if (h_is_inf(a) && h_is_inf(b))
            return ((a ^ b) & H_SIGN) ? H_QNAN : a;
        return h_is_inf(a) ? a : b;
    }
    int sa, ea, sb, eb;
    h_unpack(a, &sa, &ea);
    h_unpack(b, &sb, &eb);
    i128 v = (i128)sa * P2(ea + 48) + (i128)sb * P2(eb + 48);
    uint16_t zs = ((a & H_SIGN) && (b & H_SIGN)) ? H_SIGN : 0; /* RNE: -0 only for (-0)+(-0) */
    return fix_to_h(v, -48, zs);
}

uint16_t adkv_o_hadd(uint16_t a, uint16_t b) { return h_addsub(a, b); }
uint16_t adkv_o_hsub(uint16_t a, uint16_t b) { return h_addsub(a, b ^ H_SIGN); }

uint16_t adkv_o_hfma(uint16_t a, uint16_t b, uint16_t c)
{
    if (h_is_nan(a) || h_is_nan(b) || h_is_nan(c))
        return H_QNAN;
    uint16_t ps = (a ^ b) & H_SIGN;
    if (h_is_inf(a) || h_is_inf(b)) {
        if (h_is_zero(a) || h_is_zero(b))
            return H_QNAN;
        if (h_is_inf(c) && ((c & H_SIGN) != ps))
            return H_QNAN;
        return ps | H_INF;
    }
    if (h_is_inf(c))
        return c;
    int sa, ea, sb, eb, sc, ec;
    h_unpack(a, &sa, &ea);
    h_unpack(b, &sb, &eb);
    h_unpack(c, &sc, &ec);
    i128 v = (i128)sa * (i128)sb * P2(ea + eb + 48);
    v += (i128)sc * P2(ec + 48);
    uint16_t zs = (ps && (c & H_SIGN)) ? H_SIGN : 0;
    return fix_to_h(v, -48, zs);
}

static inline uint16_t int_to_h(int q) { return adkv_o_d2h((double)q); }

/* ------------------------------------------------------------------------------------------ */
/* semantics B scalar steps                                                                     */
/* ------------------------------------------------------------------------------------------ */

/* Code width of the semantics-B functions below.  4 is the reference's deployment format
 * (gemv.cu throughout).  2 is this build's extension of the same recurrence to the code range
 * [-2, 1] (QL/QU as train_model.py:96-97 define them for bits=2) with 16 tokens per 32-bit word;
 * the reference has no fp16 kernel for it, so nothing there pins it. */
static int g_bits = 4;

int adkv_o_set_bits(int bits)
{
    if (bits != 2 && bits != 4)
        return -1;
    g_bits = bits;
    return 0;
}

int adkv_o_get_bits(void) { return g_bits; }

static inline int q_lo(void) { return -(1 << (g_bits - 1)); }
static inline int q_hi(void) { return (1 << (g_bits - 1)) - 1; }
static inline int tokens_per_word(void) { return 32 / g_bits; }

/* gemv.cu:150-154: fp32 subtract, IEEE fp32 divide, round-half-even to int (NaN -> 0,
 * out-of-range saturates, as __float2int_rn), clamp to [-8, 7] ([-2, 1] for 2-bit codes). */
int adkv_o_quantize_f16(uint16_t x, uint16_t zp, uint16_t sc)
{
    volatile float d = adkv_o_h2f(x) - adkv_o_h2f(zp);
    volatile float u = d / adkv_o_h2f(sc);
    if (u != u)
        return 0;
    float r = nearbyintf(u); /* default rounding mode: to nearest even */
    if (r < (float)q_lo())
        return q_lo();
    if (r > (float)q_hi())
        return q_hi();
    return (int)r;
}

/* gemv.cu:220-221: omt = 1 - beta*target, both steps rounded to fp16 */
uint16_t adkv_o_omt_f16(uint16_t beta, uint16_t tgt)
{
    return adkv_o_hsub(0x3C00u, adkv_o_hmul(beta, tgt));
}

/* gemv.cu:158-164 */
void adkv_o_update_f16(int q, uint16_t *zp, uint16_t *sc,
                       uint16_t alpha, uint16_t beta, uint16_t omt)
{
    uint16_t qf = int_to_h(q);
    uint16_t qa = qf & 0x7FFFu;
    uint16_t p = adkv_o_hmul(qf, *sc);          /* __hmul2(q_f, sc)            */
    uint16_t nzp = adkv_o_hfma(alpha, p, *zp);  /* __hfma2(alpha, ., zp)       */
    uint16_t f = adkv_o_hfma(beta, qa, omt);    /* __hfma2(beta, |q|, omt)     */
    uint16_t nsc = adkv_o_hmul(*sc, f);         /* __hmul2(sc, .)              */
    *zp = nzp;
    *sc = nsc;
}

uint16_t adkv_o_dequant2_f16(int q, uint16_t zp, uint16_t sc)
{
    return adkv_o_hadd(adkv_o_hmul(int_to_h(q), sc), zp);
}

uint16_t adkv_o_dequant1_f16(int q, uint16_t zp, uint16_t sc)
{
    return adkv_o_hfma(int_to_h(q), sc, zp);
}

/* ------------------------------------------------------------------------------------------ */
/* packed layout                                                                                */
/* ------------------------------------------------------------------------------------------ */

/* [n_super, D/4, 4 (channel in group), 4 (byte row)] ; byte row br holds tokens 8sg+2br (low
 * nibble) and 8sg+2br+1 (high nibble).  gemv.cu:502-510, 91-146, 243-305.
 * 2-bit codes: a supergroup is 16 tokens, byte row br holds tokens 16sg+4br .. +3, token i of the
 * byte at bits 2i..2i+1; code = q + 2. */
int64_t adkv_o_byte_offset(int t, int c, int D)
{
    int tpw = tokens_per_word();
    int sg = t / tpw, br = (t % tpw) / (tpw / 4);
    return (((int64_t)sg * (D / 4) + c / 4) * 4 + c % 4) * 4 + br;
}

int adkv_o_get_code(const uint8_t *cache_bh, int t, int c, int D)
{
    uint8_t b = cache_bh[adkv_o_byte_offset(t, c, D)];
    int per_byte = 8 / g_bits, sh = (t % per_byte) * g_bits;
    return ((b >> sh) & ((1 << g_bits) - 1)) + q_lo();
}

void adkv_o_put_code(uint8_t *cache_bh, int t, int c, int D, int q)
{
    uint8_t *p = &cache_bh[adkv_o_byte_offset(t, c, D)];
    int per_byte = 8 / g_bits, sh = (t % per_byte) * g_bits;
    uint8_t m = (uint8_t)(((1 << g_bits) - 1) << sh);
    uint8_t n = (uint8_t)(((q - q_lo()) << sh) & m);
    *p = (uint8_t)((*p & ~m) | n);
}

/* ------------------------------------------------------------------------------------------ */
/* semantics B tensor operations                                                                */
/* ------------------------------------------------------------------------------------------ */

static inline int64_t bh_bytes(int D, int n_super_cap) { return (int64_t)n_super_cap * D * 4; }

void adkv_o_encode_kv_f16(uint8_t *cache, const uint16_t *kv_new,
                          const uint16_t *zp, const uint16_t *sc, const uint16_t *alpha,
                          const uint16_t *beta, const uint16_t *tgt,
                          int B, int H, int T, int D, int n_super_cap,
                          uint16_t *state_out)
{
    int n_super = (T + tokens_per_word() - 1) / tokens_per_word();
    for (int bx = 0; bx < B * H; bx++) {
        int h = bx % H;
        uint8_t *cb = cache + (int64_t)bx * bh_bytes(D, n_super_cap);
        /* the kernel builds each supergroup from zero and stores it whole (gemv.cu:243,300-305) */
        memset(cb, 0, (size_t)n_super * D * 4);
        for (int c = 0; c < D; c++) {
            int pi = h * D + c;
            uint16_t z = zp[pi], s = sc[pi];
            uint16_t omt = adkv_o_omt_f16(beta[pi], tgt[pi]);
            for (int t = 0; t < T; t++) {
                uint16_t x = kv_new[((int64_t)bx * T + t) * D + c];
                int q = adkv_o_quantize_f16(x, z, s);
                adkv_o_put_code(cb, t, c, D, q);
                adkv_o_update_f16(q, &z, &s, alpha[pi], beta[pi], omt);
            }
            if (state_out) {
                state_out[((int64_t)bx * D + c) * 2 + 0] = z;
                state_out[((int64_t)bx * D + c) * 2 + 1] = s;
            }
        }
    }
}

void adkv_o_replay_f16(const uint8_t *cache,
                       const uint16_t *zp, const uint16_t *sc, const uint16_t *alpha,
                       const uint16_t *beta, const uint16_t *tgt,
                       int B, int H, int T, int D, int n_super_cap,
                       uint16_t *khat_out, uint16_t *state_out)
{
    for (int bx = 0; bx < B * H; bx++) {
        int h = bx % H;
        const uint8_t *cb = cache + (int64_t)bx * bh_bytes(D, n_super_cap);
        for (int c = 0; c < D; c++) {
            int pi = h * D + c;
            uint16_t z = zp[pi], s = sc[pi];
            uint16_t omt = adkv_o_omt_f16(beta[pi], tgt[pi]);
            for (int t = 0; t < T; t++) {
                int q = adkv_o_get_code(cb, t, c, D);
                if (khat_out)
                    khat_out[((int64_t)bx * T + t) * D + c] = adkv_o_dequant2_f16(q, z, s);
                adkv_o_update_f16(q, &z, &s, alpha[pi], beta[pi], omt);
            }
            if (state_out) {
                state_out[((int64_t)bx * D + c) * 2 + 0] = z;
                state_out[((int64_t)bx * D + c) * 2 + 1] = s;
            }
        }
    }
}

/* 32-lane xor butterfly in fp16, masks 16,8,4,2,1 (gemv.cu:21-49); returns lane 0's value */
static uint16_t butterfly32(uint16_t *v)
{
    uint16_t n[32];
    for (int mask = 16; mask >= 1; mask >>= 1) {
        for (int l = 0; l < 32; l++)
            n[l] = adkv_o_hadd(v[l], v[l ^ mask]);
        memcpy(v, n, sizeof(n));
    }
    return v[0];
}

void adkv_o_forward_qk_f16(const uint16_t *q, uint8_t *cache, const uint16_t *k_new,
                           const uint16_t *zp, const uint16_t *sc, const uint16_t *alpha,
                           const uint16_t *beta, const uint16_t *tgt,
                           int B, int H, int T, int D, int n_super_cap,
                           double *logits_exact, uint16_t *logits_refemu)
{
    uint16_t *z = (uint16_t *)malloc(sizeof(uint16_t) * D);
    uint16_t *s = (uint16_t *)malloc(sizeof(uint16_t) * D);
    uint16_t *omt = (uint16_t *)malloc(sizeof(uint16_t) * D);
    uint16_t *kh = (uint16_t *)malloc(sizeof(uint16_t) * D);
    int emu = (logits_refemu != NULL) && (D == 128);
    for (int bx = 0; bx < B * H; bx++) {
        int h = bx % H;
        uint8_t *cb = cache + (int64_t)bx * bh_bytes(D, n_super_cap);
        const uint16_t *qv = q + (int64_t)bx * D;
        for (int c = 0; c < D; c++) {
            z[c] = zp[h * D + c];
            s[c] = sc[h * D + c];
            omt[c] = adkv_o_omt_f16(beta[h * D + c], tgt[h * D + c]);
        }
        for (int t = 0; t <= T; t++) {
            if (t < T) {
                for (int c = 0; c < D; c++) { /* gemv.cu:644-654 */
                    int qc = adkv_o_get_code(cb, t, c, D);
                    kh[c] = adkv_o_dequant2_f16(qc, z[c], s[c]);
                    adkv_o_update_f16(qc, &z[c], &s[c], alpha[h * D + c], beta[h * D + c], omt[c]);
                }
            } else {
                for (int c = 0; c < D; c++) { /* gemv.cu:744-798: state NOT advanced */
                    int qc = adkv_o_quantize_f16(k_new[(int64_t)bx * D + c], z[c], s[c]);
                    adkv_o_put_code(cb, T, c, D, qc);
                    kh[c] = adkv_o_dequant1_f16(qc, z[c], s[c]);
                }
            }
            double acc = 0.0;
            for (int c = 0; c < D; c++)
                acc += (double)adkv_o_h2f(qv[c]) * (double)adkv_o_h2f(kh[c]);
            logits_exact[(int64_t)bx * (T + 1) + t] = acc;
            if (emu) {
                /* lane l owns channels 4l..4l+3 as half2 pairs (4l,4l+1) then (4l+2,4l+3);
                 * per-lane: part = fma(q, k, part) over the two pairs with lo/hi halves kept
                 * apart, then lo+hi, then butterfly.  gemv.cu:647,678-686 / 797-802 */
                uint16_t lanes[32];
                for (int l = 0; l < 32; l++) {
                    uint16_t lo = 0, hi = 0;
                    for (int p = 0; p < 2; p++) {
                        int c0 = 4 * l + 2 * p;
                        lo = adkv_o_hfma(qv[c0], kh[c0], lo);
                        hi = adkv_o_hfma(qv[c0 + 1], kh[c0 + 1], hi);
                    }
                    lanes[l] = adkv_o_hadd(lo, hi);
                }
                logits_refemu[(int64_t)bx * (T + 1) + t] = butterfly32(lanes);
            }
        }
    }
    free(z);
    free(s);
    free(omt);
    free(kh);
}

void adkv_o_forward_ov_f16(const uint16_t *attn, uint8_t *cache, const uint16_t *v_new,
                           const uint16_t *zp, const uint16_t *sc, const uint16_t *alpha,
                           const uint16_t *beta, const uint16_t *tgt,
                           int B, int H, int T, int D, int n_super_cap,
                           double *out_exact, uint16_t *out_refemu)
{
    for (int bx = 0; bx < B * H; bx++) {
        int h = bx % H;
        uint8_t *cb = cache + (int64_t)bx * bh_bytes(D, n_super_cap);
        const uint16_t *w = attn + (int64_t)bx * (T + 1);
        for (int c = 0; c < D; c++) {
            int pi = h * D + c;
            uint16_t z = zp[pi], s = sc[pi];
            uint16_t omt = adkv_o_omt_f16(beta[pi], tgt[pi]);
            double acc = 0.0;
            uint16_t acc16 = 0;
            for (int t = 0; t < T; t++) { /* gemv.cu:1083-1099 */
                int qc = adkv_o_get_code(cb, t, c, D);
                uint16_t vh = adkv_o_dequant2_f16(qc, z, s);
                acc += (double)adkv_o_h2f(w[t]) * (double)adkv_o_h2f(vh);
                acc16 = adkv_o_hfma(w[t], vh, acc16);
                adkv_o_update_f16(qc, &z, &s, alpha[pi], beta[pi], omt);
            }
            { /* gemv.cu:1105-1157 */
                int qc = adkv_o_quantize_f16(v_new[(int64_t)bx * D + c], z, s);
                adkv_o_put_code(cb, T, c, D, qc);
                uint16_t vh = adkv_o_dequant1_f16(qc, z, s);
                acc += (double)adkv_o_h2f(w[T]) * (double)adkv_o_h2f(vh);
                acc16 = adkv_o_hfma(w[T], vh, acc16);
            }
            out_exact[(int64_t)bx * D + c] = acc;
            if (out_refemu)
                out_refemu[(int64_t)bx * D + c] = acc16;
        }
    }
}

/* ------------------------------------------------------------------------------------------ */
/* semantics A (fp32, unfused)                                                                  */
/* ------------------------------------------------------------------------------------------ */

static inline float clamp_keep_nan(float x, float lo, float hi)
{
    if (x != x)
        return x;
    if (x < lo)
        return lo;
    if (x > hi)
        return hi;
    return x;
}

/* train_model.py:8-22 (IntQuantSTE.forward) and :61-81 (_adkv_chunk_forward body).  Every
 * intermediate is rounded to fp32 (volatile stores keep gcc from carrying extra precision or
 * contracting).  The reference's torch.compile'd chunk function gives bit-identical results on
 * the recorded vectors of tests/golden/fp32_reference.npz (4-, 2- and 8-bit ranges). */
void adkv_o_quant_f32(const float *x, const float *zp0, const float *sc0,
                      const float *alpha, const float *beta, const float *tgt,
                      int B, int T, int C, int bits, float sc_min, float sc_max,
                      float *xhat, int8_t *codes, float *zp_seq, float *sc_seq,
                      float *zp_out, float *sc_out)
{
    const float QU = (float)((1 << (bits - 1)) - 1);
    const float QL = -(float)(1 << (bits - 1));
    const float eps = 1e-8f;
    for (int b = 0; b < B; b++) {
        for (int c = 0; c < C; c++) {
            volatile float zp = zp0[c], sc = sc0[c];
            for (int t = 0; t < T; t++) {
                int64_t i = ((int64_t)b * T + t) * C + c;
                if (zp_seq)
                    zp_seq[i] = zp;
                if (sc_seq)
                    sc_seq[i] = sc;
                volatile float s = (sc != sc) ? sc : (sc < eps ? eps : sc); /* clamp(min=eps) */
                volatile float r = x[i] - zp;
                volatile float u = r / s;
                float qf = clamp_keep_nan(nearbyintf(u), QL, QU);
                volatile float xr = qf * s;
                volatile float xh = xr + zp;
                if (xhat)
                    xhat[i] = xh;
                if (codes)
                    codes[i] = (qf != qf) ? 0 : (int8_t)qf;
                volatile float ax = alpha[c] * xr;
                volatile float nzp = zp + ax;
                volatile float e = fabsf(qf) - tgt[c];
                volatile float sb = sc * beta[c];
                volatile float sbe = sb * e;
                volatile float nsc = sc + sbe;
                zp = nzp;
                sc = clamp_keep_nan(nsc, sc_min, sc_max);
            }
            if (zp_out)
                zp_out[(int64_t)b * C + c] = zp;
            if (sc_out)
                sc_out[(int64_t)b * C + c] = sc;
        }
    }
}

void adkv_o_attention_f64(const float *q, const float *K, const float *V,
                          int B, int H, int T, int D, double scaling,
                          double *out, double *weights)
{
    double *l = (double *)malloc(sizeof(double) * (T > 0 ? T : 1));
    for (int bx = 0; bx < B * H; bx++) {
        const float *qv = q + (int64_t)bx * D;
        double m = -INFINITY;
        for (int t = 0; t < T; t++) {
            const float *k = K + ((int64_t)bx * T + t) * D;
            double a = 0.0;
            for (int c = 0; c < D; c++)
                a += (double)qv[c] * (double)k[c];
            l[t] = a * scaling;
            if (l[t] > m)
                m = l[t];
        }
        double z = 0.0;
        for (int t = 0; t < T; t++) {
            l[t] = exp(l[t] - m);
            z += l[t];
        }
        for (int c = 0; c < D; c++)
            out[(int64_t)bx * D + c] = 0.0;
        for (int t = 0; t < T; t++) {
            double w = l[t] / z;
            if (weights)
                weights[(int64_t)bx * T + t] = w;
            const float *v = V + ((int64_t)bx * T + t) * D;
            for (int c = 0; c < D; c++)
                out[(int64_t)bx * D + c] += w * (double)v[c];
        }
    }
    free(l);
}
