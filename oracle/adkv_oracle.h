/*
 * ADKV CPU oracle — TEST INFRASTRUCTURE ONLY.
 *
 * A scalar, single-threaded restatement of the reference's two recurrences:
 *   semantics B (fp16 deployment path)  src/adkv/kernel/gemv.cu
 *   semantics A (fp32 train/eval path)  src/adkv/train/train_model.py
 * Nothing in the shipped package may call into this library; only tests, the
 * smoke check and the bench's cpu_baseline leg do.
 *
 * Parity status: the reference holds no tests or golden vectors for this path; every function is
 * pinned by the independent checks in tests/test_oracle_*.py, and adkv_o_quant_f32 additionally by
 * vectors recorded from the reference's own (torch.compile'd) fp32 module
 * (tests/golden/fp32_reference.npz, tests/test_golden_fp32_reference.py).  Parity unpinned on one
 * point: CUDA hardware behaviour at NaN/denormal corners beyond its intrinsics' documentation.
 *
 * All fp16 values cross this interface as raw uint16_t bit patterns.
 */
#ifndef ADKV_ORACLE_H
#define ADKV_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- fp16 primitives (IEEE binary16, round-to-nearest-even, subnormals kept) ---- */
float    adkv_o_h2f(uint16_t h);
uint16_t adkv_o_f2h(float f);
uint16_t adkv_o_d2h(double d);
uint16_t adkv_o_hmul(uint16_t a, uint16_t b);
uint16_t adkv_o_hadd(uint16_t a, uint16_t b);
uint16_t adkv_o_hsub(uint16_t a, uint16_t b);
uint16_t adkv_o_hfma(uint16_t a, uint16_t b, uint16_t c); /* one rounding */

/* Code width used by every semantics-B function below: 4 (the reference's format, default) or 2
 * (this build's extension: codes in [-2, 1], 16 tokens per word).  Process-wide; returns 0, or
 * -1 for an unsupported width. */
int      adkv_o_set_bits(int bits);
int      adkv_o_get_bits(void);

/* ---- semantics B scalar steps ---- */
/* gemv.cu:150-154 */
int      adkv_o_quantize_f16(uint16_t x, uint16_t zp, uint16_t sc);
/* gemv.cu:220-221 */
uint16_t adkv_o_omt_f16(uint16_t beta, uint16_t tgt);
/* gemv.cu:158-164 ; q in [-8,7] */
void     adkv_o_update_f16(int q, uint16_t *zp, uint16_t *sc,
                           uint16_t alpha, uint16_t beta, uint16_t omt);
/* gemv.cu:644-645 (two roundings) */
uint16_t adkv_o_dequant2_f16(int q, uint16_t zp, uint16_t sc);
/* gemv.cu:796 (fused, one rounding) */
uint16_t adkv_o_dequant1_f16(int q, uint16_t zp, uint16_t sc);

/* ---- packed-cache layout  [B,H,n_super_cap,D/4,4,4] uint8  (llama_adkv.py:47-55) ---- */
int64_t adkv_o_byte_offset(int t, int c, int D); /* inside one (b,h) block */
int     adkv_o_get_code(const uint8_t *cache_bh, int t, int c, int D);      /* q in [-8,7] */
void    adkv_o_put_code(uint8_t *cache_bh, int t, int c, int D, int q);     /* RMW one nibble */

/* ---- semantics B whole-tensor operations ---- */
/* encode_kv: gemv.cu:168-308.  state_out (optional) = [B,H,D,2] fp16 (zp,sc) after T tokens.
 * Whole supergroups [0, ceil(T/8)) are overwritten, tail nibbles zero. */
void adkv_o_encode_kv_f16(uint8_t *cache, const uint16_t *kv_new,
                          const uint16_t *zp, const uint16_t *sc, const uint16_t *alpha,
                          const uint16_t *beta, const uint16_t *tgt,
                          int B, int H, int T, int D, int n_super_cap,
                          uint16_t *state_out);

/* Replay the cache: khat_out (optional) [B,H,T,D] fp16 two-rounding dequant (gemv.cu:644-645),
 * state_out (optional) [B,H,D,2] state after T tokens. */
void adkv_o_replay_f16(const uint8_t *cache,
                       const uint16_t *zp, const uint16_t *sc, const uint16_t *alpha,
                       const uint16_t *beta, const uint16_t *tgt,
                       int B, int H, int T, int D, int n_super_cap,
                       uint16_t *khat_out, uint16_t *state_out);

/* forward_qk: gemv.cu:435-815.  Appends k_new at slot T (in place).
 * logits_exact [B,H,T+1] double: exact sum of fp16 products over the bit-exact dequantised values.
 * logits_refemu (optional, D==128 only) [B,H,T+1] fp16: the reference's own fp16 accumulation
 * order (per-lane half2 fma, pair add, 32-lane xor butterfly). */
void adkv_o_forward_qk_f16(const uint16_t *q, uint8_t *cache, const uint16_t *k_new,
                           const uint16_t *zp, const uint16_t *sc, const uint16_t *alpha,
                           const uint16_t *beta, const uint16_t *tgt,
                           int B, int H, int T, int D, int n_super_cap,
                           double *logits_exact, uint16_t *logits_refemu);

/* forward_ov: gemv.cu:946-1178.  attn [B,H,T+1] fp16.  Appends v_new at slot T.
 * out_exact [B,H,D] double; out_refemu (optional) [B,H,D] fp16 sequential fp16 fma in t. */
void adkv_o_forward_ov_f16(const uint16_t *attn, uint8_t *cache, const uint16_t *v_new,
                           const uint16_t *zp, const uint16_t *sc, const uint16_t *alpha,
                           const uint16_t *beta, const uint16_t *tgt,
                           int B, int H, int T, int D, int n_super_cap,
                           double *out_exact, uint16_t *out_refemu);

/* ---- semantics A (fp32, unfused; train_model.py:8-22,61-81) ---- */
/* x [B,T,C] fp32; zp0/sc0/alpha/beta/tgt [C]; bits -> QU=2^(bits-1)-1, QL=-2^(bits-1).
 * Outputs (each optional): xhat [B,T,C], codes [B,T,C] int8, zp_seq/sc_seq [B,T,C] (state BEFORE
 * token t, as train_model.py:66-68), zp_out/sc_out [B,C] final state. */
void adkv_o_quant_f32(const float *x, const float *zp0, const float *sc0,
                      const float *alpha, const float *beta, const float *tgt,
                      int B, int T, int C, int bits, float sc_min, float sc_max,
                      float *xhat, int8_t *codes, float *zp_seq, float *sc_seq,
                      float *zp_out, float *sc_out);

/* Single-query attention in fp64 over fp32 K/V: out[b,h,:] = softmax(scaling * q.K^T) V.
 * q [B,H,D], K,V [B,H,T,D] -> out [B,H,D], weights (optional) [B,H,T]. */
void adkv_o_attention_f64(const float *q, const float *K, const float *V,
                          int B, int H, int T, int D, double scaling,
                          double *out, double *weights);

#ifdef __cplusplus
}
#endif
#endif
