/*
 * libadkv_hip — C ABI of the MI355X (gfx950) ADKV hot path.
 *
 * Plain pointers and sizes only: every pointer is a DEVICE pointer unless stated otherwise, every
 * fp16 tensor is IEEE binary16, `stream` is a hipStream_t passed as void* (NULL = default stream).
 * All calls are asynchronous with respect to the host and return 0 on success or a negative
 * ADKV_E_* code; adkv_strerror() names it.  Nothing here allocates device memory.
 *
 * Packed cache layout (reference: src/adkv/hf/llama_adkv.py:47-55, src/adkv/kernel/gemv.cu:502-510):
 *   uint8 [B, H, n_super_cap, D/4, 4, 4]; one supergroup = 8 tokens; viewed as 32-bit words, word
 *   (sg, c) holds channel c's eight 4-bit codes, code of token 8*sg+i at bits 4i..4i+3, code = q+8.
 * Parameter tensors zp/sc/alpha/beta/tgt are fp16 [H, D].
 */
#ifndef ADKV_HIP_H
#define ADKV_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ADKV_OK 0
#define ADKV_E_NULL (-1)       /* a required pointer is NULL */
#define ADKV_E_DIM (-2)        /* head dim not in {128, 256, 512} */
#define ADKV_E_SHAPE (-3)      /* negative / zero sizes */
#define ADKV_E_CAPACITY (-4)   /* cache has too few supergroups */
#define ADKV_E_ALIGN (-5)      /* pointer alignment requirement violated */
#define ADKV_E_UNSUPPORTED (-6)
#define ADKV_E_WORKSPACE (-7)  /* workspace missing or too small */
#define ADKV_E_SCRATCH_LIMIT (-8) /* adkv_forward_ov_noalloc: needs more than adkv_static_scratch_bytes() */
#define ADKV_E_DEVICE (-9)     /* a HIP device query failed; see adkv_last_hip_error() */
#define ADKV_E_LAUNCH (-100)   /* HIP reported a launch error; see adkv_last_hip_error() */

/* ABI version of this header; bumped on any signature change. */
int adkv_abi_version(void);

/* Tuning knob, no counterpart in the reference: which decode kernels a launch with as many query
 * heads as KV heads and head dim 128 uses: 0 = the vector kernels with the shared code table,
 * 1 = the matrix-core kernels (the ones grouped-query launches always use), 2 = the vector
 * kernels with a per-head table wherever they can run (4-bit codes; 3 = the same, always with
 * sixteen lanes per head, 4 = always with thirty-two), -1 = the library's choice
 * (the per-head table where its launch is the faster one, else the shared one; ADKV_MFMA=1 in the environment,
 * read once, makes it the matrix-core kernels).  Results agree to the tolerance of the fp32
 * accumulation order; appended codes, state and checkpoints are identical. */
void adkv_set_mha_kernel(int use_matrix_cores);
/* Tuning knob, no counterpart in the reference (whose module chains the three kernels,
 * llama_adkv.py:264-274): mode > 0 lets adkv_decode_step run forward_qk, the softmax and
 * forward_ov as ONE launch wherever both stages run the per-head-table kernels on four segments
 * per sequence, there is no mask and the context is at most 8703 tokens; 0 (the default) always
 * takes three launches.  The fused launch computes what the three launches compute (the softmax
 * sums in a different, fixed order: weights and outputs agree to an fp16 ulp; codes, state and
 * checkpoints are identical) in the same time, measured; it saves the host two launches.
 * adkv_decode_step_is_fused tells which a call with these sizes takes under the current mode. */
void adkv_set_fused_step(int mode);
int adkv_decode_step_is_fused(int B, int Hq, int H, int T, int D, int bits, int n_ckpt_cap,
                              int ckpt_interval, int masked);
const char *adkv_strerror(int code);
/* hipError_t (as int) of the last failed launch in this thread, 0 if none. */
int adkv_last_hip_error(void);

/*
 * Prefill quantise: tokens [0,T) of kv_new [B,H,T,D] fp16 -> codes, starting from (zp, sc).
 * Replaces encode_kv (src/adkv/kernel/gemv.cu:368-414, kernel :168-308; Python wrapper
 * src/adkv/kernel/gemv.py:100-132).  Whole supergroups [0, ceil(T/8)) are overwritten.
 * scale_min/scale_max are accepted for signature parity and ignored, as the reference kernel does.
 * state_out (optional, may be NULL): fp16 [B,H,D,2] = (zp, sc) after token T-1.
 */
int adkv_encode_kv(void *cache, const void *kv_new,
                   const void *zp, const void *sc, const void *alpha, const void *beta,
                   const void *tgt,
                   int B, int H, int T, int D, int n_super_cap,
                   float scale_min, float scale_max,
                   void *state_out, void *stream);

/*
 * Decode q.K^T over T cached tokens, then quantise k_new with the state after token T-1, write it
 * at slot T in place and emit its self logit.  logits: fp16 [B,H,T+1].
 * Replaces forward_qk (src/adkv/kernel/gemv.cu:883-939, kernel :435-815; gemv.py:16-55).
 * q, k_new: fp16 [B,H,D] (the reference's [B,H,1,D] made contiguous).
 * state_out (optional): fp16 [B,H,D,2] state after token T-1 (the state k_new was quantised with).
 */
int adkv_forward_qk(const void *q, void *k_cache, const void *k_new, void *logits,
                    const void *zp, const void *sc, const void *alpha, const void *beta,
                    const void *tgt,
                    int B, int H, int T, int D, int n_super_cap,
                    float scale_min, float scale_max,
                    void *state_out, void *stream);

/*
 * Decode P.V: out[b,h,:] = sum_{t<T} attn[t]*v_hat[t,:] + attn[T]*v_hat_new, appending v_new at
 * slot T in place.  attn: fp16 [B,H,T+1]; out: fp16 [B,H,D].
 * Replaces forward_ov (src/adkv/kernel/gemv.cu:1233-1288, kernel :946-1178; gemv.py:58-97).
 */
int adkv_forward_ov(const void *attn, void *v_cache, const void *v_new, void *out,
                    const void *zp, const void *sc, const void *alpha, const void *beta,
                    const void *tgt,
                    int B, int H, int T, int D, int n_super_cap,
                    float scale_min, float scale_max,
                    void *state_out, void *stream);

/*
 * weights = softmax(float(logits) * scaling + mask) over the last axis, written as fp16.
 * Replaces the torch ops between the two GEMVs (src/adkv/hf/llama_adkv.py:266-271).
 * logits, weights: fp16 [rows, n]; mask (optional, NULL = none): fp32 [mask_rows, n] with row r of
 * logits using mask row (r / rows_per_mask_row) — pass rows_per_mask_row = H for a [B,1,1,n] mask.
 */
int adkv_softmax(const void *logits, void *weights, const void *mask,
                 int rows, int n, int rows_per_mask_row, float scaling, void *stream);

/* The same with a workspace of adkv_softmax_workspace_bytes(rows, n) bytes (0 for rows of up to
 * 24576 elements, which one workgroup keeps in its registers): longer rows are then cut into
 * chunks that many workgroups process, instead of one workgroup walking the row three times.  ld: pitch of both
 * matrices in elements (0 = n); the mask stays packed. */
int64_t adkv_softmax_workspace_bytes(int rows, int n);
int adkv_softmax_ex(const void *logits, void *weights, const void *mask,
                    int rows, int n, int64_t ld, int rows_per_mask_row, float scaling,
                    void *workspace, int64_t workspace_bytes, void *stream);

/* Row pitch (in elements) this library recommends for a logits / attention-weight matrix with n
 * columns: the smallest odd multiple of 128.  The `ld` arguments of the entry points below are
 * such pitches (0 = rows packed back to back, n = T + 1).  With packed rows and n*2 bytes close
 * to a power of two (ctx 4096, 131072 ...), the rows of all heads start in the same memory
 * channel and the waves, which walk their rows in step, queue up on it. */
int64_t adkv_row_pitch(int n);

/*
 * ---- Extensions with state checkpoints (no counterpart in the reference's code; its paper sketches
 * them in App. I).  The fp16 recurrence rounds at every step, so a sequence can only be cut where
 * the exact state is known.  A checkpoint tensor is fp16 [B, H, n_ckpt_cap, D, 2]; entry j holds
 * (zp, sc) BEFORE token (j+1)*ckpt_interval (ckpt_interval a positive multiple of 8).  It belongs to
 * one cache tensor and is maintained by these calls: the encoder writes every entry up to T, the
 * decode calls write entry T/ckpt_interval-1 when the appended token T starts a new interval.
 * Given checkpoints, the decode calls split the time axis into independently replayed segments so
 * that small batches and long contexts still fill the GPU; results are bit-identical for codes and
 * state, and equal up to fp32 summation order for logits/outputs.  Passing ckpt = NULL gives exactly
 * the plain entry points above.
 */
int adkv_encode_kv_ex(void *cache, const void *kv_new,
                      const void *zp, const void *sc, const void *alpha, const void *beta,
                      const void *tgt,
                      int B, int H, int T, int D, int n_super_cap,
                      void *state_out, void *ckpt_out, int n_ckpt_cap, int ckpt_interval,
                      void *stream);

/*
 * Streaming append: quantise n_new further tokens of a stream whose first T0 tokens are already
 * in the cache, kv_new fp16 [B,H,n_new,D].  state_io fp16 [B,H,D,2] holds the state after token
 * T0-1 on entry (ignored when T0 == 0) and after token T0+n_new-1 on return, so appending costs
 * O(n_new) instead of the O(T0) replay that forward_qk/forward_ov pay to recover the state
 * (src/adkv/kernel/gemv.cu:744-764).  Byte-identical to one adkv_encode_kv over all T0+n_new tokens;
 * also lifts the reference's "prefill encodes from token 0" restriction
 * (src/adkv/hf/llama_adkv.py:195-197).  Checkpoint entries crossed by the new tokens are written.
 */
int adkv_append_kv(void *cache, const void *kv_new,
                   const void *zp, const void *sc, const void *alpha, const void *beta,
                   const void *tgt,
                   int B, int H, int T0, int n_new, int D, int n_super_cap, int bits,
                   void *state_io, void *ckpt, int n_ckpt_cap, int ckpt_interval, void *stream);

/*
 * adkv_append_kv for the K and the V rows of the same tokens in ONE launch: the two calls that
 * KVCacheLayer_ADKV._append_tokens makes back to back (src/adkv/hf/llama_adkv.py:144-153), with
 * the conversion and packing that precede them there (`.to(torch.float16).contiguous()`,
 * llama_adkv.py:141-142) folded in:
 *   kv_dtype   ADKV_DT_F16, or ADKV_DT_BF16: bfloat16 rows are rounded to fp16 (nearest even, as
 *              torch's .to(float16)) as they are read;
 *   k_strides / v_strides   NULL for packed [B,H,n_new,D] rows, else host arrays of three element
 *              strides {batch, head, token} (channels contiguous, all three even, token stride
 *              >= D, base pointers 4-byte aligned): a projection output laid out [B,T,H,D] is
 *              quantised where it lies.
 * Both tensors share every shape argument; k_params / v_params are host arrays of five device
 * pointers {zp, sc, alpha, beta, tgt}; the checkpoint tensors are both given or both NULL.
 * Results are byte-identical to two adkv_append_kv calls on packed fp16 copies.  Channels are the
 * only parallel axis of the encoder, so a long prompt at a small batch (B*H*D below ~130 000
 * channels) leaves half of the device idle per tensor; paired, both tensors finish in the time of
 * one.
 */
int adkv_append_kv_pair(void *k_cache, void *v_cache, const void *k_new, const void *v_new,
                        int kv_dtype, const int64_t *k_strides, const int64_t *v_strides,
                        const void *const *k_params, const void *const *v_params,
                        int B, int H, int T0, int n_new, int D, int n_super_cap, int bits,
                        void *k_state_io, void *v_state_io, void *k_ckpt, void *v_ckpt,
                        int n_ckpt_cap, int ckpt_interval, void *stream);

int adkv_forward_qk_ex(const void *q, void *k_cache, const void *k_new, void *logits,
                       const void *zp, const void *sc, const void *alpha, const void *beta,
                       const void *tgt,
                       int B, int H, int T, int D, int n_super_cap,
                       void *state_out, void *ckpt, int n_ckpt_cap, int ckpt_interval,
                       void *stream);

/* Bytes of fp32 workspace adkv_forward_ov_ex needs for these sizes (0 when it runs one segment). */
int64_t adkv_forward_ov_workspace_bytes(int B, int H, int T, int D, int n_ckpt_cap,
                                        int ckpt_interval);

int adkv_forward_ov_ex(const void *attn, void *v_cache, const void *v_new, void *out,
                       const void *zp, const void *sc, const void *alpha, const void *beta,
                       const void *tgt,
                       int B, int H, int T, int D, int n_super_cap,
                       void *state_out, void *ckpt, int n_ckpt_cap, int ckpt_interval,
                       void *workspace, int64_t workspace_bytes, void *stream);

/*
 * Grouped-query attention: Hq query heads share H KV heads (Hq % H == 0; query head j reads KV
 * head j / (Hq/H)).  The reference refuses this (src/adkv/hf/llama_adkv.py:235-238 requires
 * num_attention_heads == num_key_value_heads); here the state replay runs once per KV head and
 * the contraction with all of its query heads goes to the matrix cores.  Head dim 128 only when
 * Hq > H.  q: [B, Hq, D]; logits / attn: [B, Hq, T+1]; out: [B, Hq, D]; everything else as in the
 * _ex entry points.  The OV workspace is adkv_forward_ov_gqa_workspace_bytes(...) bytes.
 *
 * bits: 4 = the reference's code format.  2 = the same fp16 recurrence over codes in [-2, 1]
 * (QL/QU of src/adkv/train/train_model.py:96-97 for bits = 2), stored as q + 2 with 16 tokens per
 * 32-bit channel word, i.e. supergroups of 16 tokens in the same uint8 [B,H,n_super,D/4,4,4]
 * tensor; head dim 128 only, checkpoint intervals a multiple of 16.  The reference has no kernel
 * for it.  adkv_append_kv (T0 = 0 for a whole prompt) writes such caches.
 */
int adkv_forward_qk_gqa(const void *q, void *k_cache, const void *k_new, void *logits,
                        const void *zp, const void *sc, const void *alpha, const void *beta,
                        const void *tgt,
                        int B, int Hq, int H, int T, int D, int n_super_cap, int bits, int64_t ld,
                        void *state_out, void *ckpt, int n_ckpt_cap, int ckpt_interval,
                        void *stream);
int64_t adkv_forward_ov_gqa_workspace_bytes(int B, int Hq, int H, int T, int D, int n_ckpt_cap,
                                            int ckpt_interval);
int adkv_forward_ov_gqa(const void *attn, void *v_cache, const void *v_new, void *out,
                        const void *zp, const void *sc, const void *alpha, const void *beta,
                        const void *tgt,
                        int B, int Hq, int H, int T, int D, int n_super_cap, int bits, int64_t ld,
                        void *state_out, void *ckpt, int n_ckpt_cap, int ckpt_interval,
                        void *workspace, int64_t workspace_bytes, void *stream);

/*
 * adkv_forward_ov_gqa for callers that cannot allocate device memory and have no workspace to
 * hand over: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * No counterpart in the reference (its binding allocates its output with torch::zeros on every
 * call, src/adkv/kernel/gemv.cu:1272).  Same arguments and results as adkv_forward_ov_gqa without
 * `workspace`: the fp32 partial sums of a segmented launch go to a 32 MiB device array that is
 * part of the library (one copy per GPU, held until the process ends).  The call itself never
 * allocates or frees.  A launch whose segment plan needs more than adkv_static_scratch_bytes()
 * (= adkv_forward_ov_gqa_workspace_bytes(...) of the same sizes) is rejected with
 * ADKV_E_SCRATCH_LIMIT before anything is launched.  All calls on one GPU share that GPU's array:
 * calls that overlap in time on one GPU (different streams, different threads) race on it; calls
 * on one stream are safe.  The array needs no clearing between calls (every partial read was
 * written by the same launch).
 * adkv_init() resolves the array's address on the CURRENT device; call it once per device at
 * set-up (outside any graph capture).  adkv_forward_ov_noalloc does the same on its first call on
 * a device if adkv_init() was not called there.
 */
int adkv_init(void);
int64_t adkv_static_scratch_bytes(void);
int adkv_forward_ov_noalloc(const void *attn, void *v_cache, const void *v_new, void *out,
                            const void *zp, const void *sc, const void *alpha, const void *beta,
                            const void *tgt,
                            int B, int Hq, int H, int T, int D, int n_super_cap, int bits, int64_t ld,
                            void *state_out, void *ckpt, int n_ckpt_cap, int ckpt_interval,
                            void *stream);

/*
 * One decode-attention step of one layer in a single library call: the launches of forward_qk,
 * scale/mask/softmax and forward_ov (plus the sum of forward_ov's segments) issued back to back
 * on `stream`, appending k_new / v_new at slot T of both caches.  It is one CALL, not one kernel:
 * logits and weights pass through the workspace between the launches.  (A single kernel was
 * evaluated and not built: the softmax arithmetic costs the same vector instructions wherever it
 * runs, these kernels are bound by vector-instruction issue and not by the logits' round trip, and
 * the per-head table that the QK and OV kernels each build needs the whole LDS of a CU for itself.)
 * Replaces the body of KVCacheLayer_ADKV.decode (src/adkv/hf/llama_adkv.py:245-276).
 * q: fp16 [B, Hq, D] with Hq a multiple of the H KV heads (Hq == H is the reference's case).
 * k_params / v_params: host arrays of five device pointers {zp, sc, alpha, beta, tgt}, each
 * fp16 [H, D].  mask: optional fp32 additive mask as in adkv_softmax.  out: fp16 [B, Hq, D].
 * weights_out: optional fp16 [B, Hq, weights_ld] with weights_ld == adkv_row_pitch(T + 1), columns
 * 0..T valid (the attention weights the reference returns); when NULL they live in the workspace.  Checkpoint tensors as in the _ex entry points (NULL = none).
 * act_dtype: ADKV_DT_F16, or ADKV_DT_BF16 when q, k_new, v_new and out are bfloat16: they are
 * rounded to fp16 as they are read and the fp16 result to bf16 as it is written, the values of
 * the reference's .to(torch.float16) / .to(q.dtype) around its kernels (llama_adkv.py:248-250, 274)
 * without the four conversion launches.  Logits and weights stay fp16.
 * workspace: >= adkv_decode_step_workspace_bytes(...) bytes, 256-byte aligned.
 */
int64_t adkv_decode_step_workspace_bytes(int B, int Hq, int H, int T, int D, int n_ckpt_cap,
                                          int ckpt_interval);
int adkv_decode_step(const void *q, void *k_cache, void *v_cache, const void *k_new,
                      const void *v_new, const void *const *k_params, const void *const *v_params,
                      const void *mask, int rows_per_mask_row, float scaling,
                      void *out, void *weights_out, int64_t weights_ld,
                      int B, int Hq, int H, int T, int D, int n_super_cap, int bits, int act_dtype,
                      void *k_ckpt, void *v_ckpt, int n_ckpt_cap, int ckpt_interval,
                      void *workspace, int64_t workspace_bytes, void *stream);

/* Which of the library's decode kernels adkv_forward_qk_gqa / adkv_forward_ov_gqa /
 * adkv_decode_step launch for these sizes ("qk_" / "ov_" + the returned text): a static string,
 * for benchmark records and tests; "invalid" for sizes the entry points reject. */
const char *adkv_decode_kernel_name(int B, int Hq, int H, int T, int D, int bits, int n_ckpt_cap,
                                    int ckpt_interval);

/* How the context of such a launch is cut into independently replayed segments (no counterpart
 * in the reference, whose kernels replay every sequence from token 0: gemv.cu:565).  Returns the
 * number of segments n (1 without checkpoints; -1 for sizes the entry points reject) and, when
 * `bounds` has room (max_bounds > n), their token boundaries bounds[0] = 0 < ... < bounds[n] = T:
 * every inner boundary lies on a checkpoint.  Segments may differ in length: kernels in 16-wave
 * workgroups give the four wave slots of a SIMD unequal shares of the work, in groups of four
 * segments of which the last in time is the longest (the oldest slot takes it).  info, when not NULL,
 * receives {workgroups launched, virtual workgroups each of them walks through}. */
int adkv_decode_segments(int B, int Hq, int H, int T, int D, int bits, int n_ckpt_cap,
                         int ckpt_interval, int *bounds, int max_bounds, int *info);

/*
 * Measurement hook, no counterpart in the reference (its benchmark times whole steps with CUDA
 * events, tools/perf_kernel.py:65-74): `events` is a host array of four hipEvent_t created with
 * timing enabled, or NULL to switch the hook off.  While set, every adkv_decode_step call of
 * THIS host thread records them on its stream: [0] before the QK launch, [1] after it, [2] after
 * the softmax, [3] after the OV launch and the sum of its segments, so the stages of the product
 * path can be timed without taking it apart.
 */
void adkv_set_stage_events(void *const *events);

/*
 * fp32 ("train / eval") form of the recurrence: fake-quantise a token stream with the state kept
 * in fp32 and every operation separately rounded.  Replaces the forward pass of
 * _adkv_chunk_forward + IntQuantSTE (src/adkv/train/train_model.py:8-22,61-81) and the Triton
 * kernel _adkv_quant_kernel (src/adkv/hf/llama_adkv_eval.py:34-118, one call per K and per V).
 *   x         [B, T, C] of x_dtype (ADKV_DT_*), element strides stride_b / stride_t, channel
 *             stride 1;  xhat: same layout, may alias x (in-place, as the eval cache does) or NULL
 *   codes     optional int8 [B, T, C] contiguous, the integer q per element
 *   zp_state, sc_state   optional fp32 [B, C]: read as the starting state unless zp_init/sc_init
 *             are given, and always written with the state after the last token
 *   zp_init, sc_init     optional fp32 [C]: starting state broadcast over the batch
 *   alpha, beta, tgt     fp32 [C]
 *   zp_seq, sc_seq       optional fp32 [B, T, C] contiguous: the state BEFORE each token
 *             (train_model.py:66-68)
 *   lower_limit/upper_limit   integer code range (train_model.py:96-97), sc_min/sc_max the
 *             clamp of the scale (train_model.py:98-99).
 */
#define ADKV_DT_F32 0
#define ADKV_DT_F16 1
#define ADKV_DT_BF16 2
int adkv_quant_f32(const void *x, void *xhat, void *codes, void *zp_state, void *sc_state,
                   const void *zp_init, const void *sc_init, const void *alpha,
                   const void *beta, const void *tgt, void *zp_seq, void *sc_seq,
                   int B, int T, int C, int64_t stride_b, int64_t stride_t, int x_dtype,
                   int lower_limit, int upper_limit, float sc_min, float sc_max, void *stream);

/*
 * Rotary position embedding of the query and key rows in one launch: x * cos + rotate_half(x) * sin
 * with every operation rounded to the activations' type as torch rounds it, bit-identical to
 * transformers' apply_rotary_pos_emb that the attention module calls before the cache
 * (src/adkv/hf/llama_adkv.py:336-337; ten elementwise launches there).
 *   q [B, Hq, T, D], k [B, H, T, D]: fp16 (bf16 = 0) or bfloat16 (bf16 = 1), channels contiguous,
 *       element strides over batch / head / token given (the [B, T, H*D] projection output viewed
 *       head-first needs no copy);  cos, sin [B, T, D] in the same type, strides over batch / token
 *       (0 over the batch for a shared table);  q_out, k_out: contiguous [B, Hq, T, D] / [B, H, T, D].
 *   D a multiple of 4; every pointer 4-byte aligned and every stride even.
 */
int adkv_rope_qk(const void *q, const void *k, const void *cos, const void *sin, void *q_out, void *k_out,
                 int B, int Hq, int H, int T, int D,
                 int64_t q_sb, int64_t q_sh, int64_t q_st, int64_t k_sb, int64_t k_sh, int64_t k_st,
                 int64_t cs_sb, int64_t cs_st, int bf16, void *stream);

/* ---- comparator, not part of the drop-in boundary ----
 * fp16-KV single-query attention (split-K flash decoding), standing in for the uncompressed fp16
 * cache that ADKV's memory and latency claims are made against (tools/memory_comparison_fig.py:46-56
 * models its bytes; the reference ships no kernel for it).  q [B,H,128], K/V [B,H,T,128], out [B,H,128], all fp16;
 * out = softmax(scaling * q.K^T) V.  D must be 128. */
int64_t adkv_fp16_decode_workspace_bytes(int B, int H, int T);
int adkv_fp16_decode(const void *q, const void *K, const void *V, void *out, void *workspace,
                     int64_t workspace_bytes, int B, int H, int T, int D, float scaling, void *stream);

#ifdef __cplusplus
}
#endif
#endif
