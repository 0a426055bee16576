/*
 * mynn_oracle.h -- CPU restatement of the reference engine's quantized-LLM hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library may include, link or call this;
 * the only users are tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg, and
 * there it is the checker (or the timed CPU baseline), never the product.
 *
 * Every function restates one reference algorithm; the citation (path:line inside the
 * reference tree kcvlex/my-nn-engine) is on each declaration.  All arithmetic is IEEE f32
 * unless stated; storage types are f32, bf16 (RNE, as src/codegen/cpu/kernels/ftype.rs:41-50)
 * and fp16 (RNE; the reference has no fp16 -- it is the 16-bit type the new path adds).
 *
 * Summation order: the reference tags its dot products "fast" (translator.rs:284-288) and lets
 * LLVM vectorise them, so its own order depends on the host ISA.  The restatement fixes one
 * order instead: ORC_LANES interleaved partial sums (element i goes to lane i % lanes), lanes
 * combined by a fixed pairwise tree.  orc_set_lanes(1) gives the plain sequential order.
 *
 * Pin status (what checks each function besides its own formula; all in tests/test_oracle_*.py):
 *   orc_dequant_matmul        10 dequant_matmul* fixtures of tests/single_op.rs (mode 2 bit-exact), f64 closed form
 *   orc_quantized_matmul      5 quantized_matmul* fixtures (int32 part exact), integer brute force
 *   orc_dynquant_*            4 dyn_quantize_linear* fixtures, round-trip bound
 *   orc_dequantize_linear     dequantize_linear fixture
 *   orc_attention             5 attention* fixtures, f64 brute force of tests/session_state.rs, softmax invariants
 *   orc_kv_cache_update       kv_cache_update fixture + 3-step persistence
 *   orc_quantizing_kv_update  quantizing_kvcache_update fixture
 *   orc_rms_norm, orc_rope, orc_rope_table, orc_swish   closed forms of crates/llm/tests/builder_ops.rs, swish fixture
 *   orc_gather_rows           2 gather* fixtures
 *   orc_quantize_per_channel  known answers of crates/llm/tests/quantize.rs:106-159
 *   orc_f32_to_f16 / bf16     exhaustive against numpy
 *   orc_model_* (decoder executor and generate loop)   the reference's exact ids on its tiny random Llama
 *                             (crates/llm/tests/tinyllama_random.rs:20-24) in f32/bf16/f16 and three summation orders;
 *                             mock_decode expectations (crates/llm/tests/mock_decode.rs:30-87)
 *   orc_model_set_bias (q / k / v projection bias, decoder.rs:167-184)   no fixture in the reference (its only checkpoint is
 *                             a Llama): an independent float64 textbook decoder with one bias at a time and all three,
 *                             zero biases change no bit of the golden ids, token-by-token == prefill
 *   ring_phys_index, kv_cache_update_streaming, attention_streaming (numpy, oracle/__init__.py; sink + ring KV ops of the
 *                             reference's CUDA kernels)   brute-force ring simulation, reduction to the plain update /
 *                             attention when the ring has not wrapped, f64 attention over explicitly scattered rows
 * Parity unpinned: none.  What no offline check fixes bit for bit is the reference's own f32 summation
 * order (LLVM fast-math vectorisation, BLAS sgemm) and libm expf; those are covered by tolerance.
 */
#ifndef MYNN_ORACLE_H_
#define MYNN_ORACLE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* storage types; 0/1 match the reference's FType (ftype.rs:4-9), 2 is new */
enum { ORC_F32 = 0, ORC_BF16 = 1, ORC_F16 = 2 };

void orc_set_lanes(int lanes);   /* 1..64, power of two; default 16 */
int  orc_get_lanes(void);
void orc_set_threads(int n);     /* OpenMP threads for the N split (schedule/omp.rs:70-95) */
int  orc_get_threads(void);

/* scalar conversions (ftype.rs:22-50, quantize.rs:47-81) */
uint16_t orc_f32_to_bf16(float x);
float    orc_bf16_to_f32(uint16_t b);
uint16_t orc_f32_to_f16(float x);
float    orc_f16_to_f32(uint16_t h);
void orc_convert(void *dst, int dst_dtype, const void *src, int src_dtype, size_t n);

/* A1 DequantizeLinear axis 0 (translator.rs:206-282; cuda dequantize.cuh:5-19):
 * out[r,c] = (T)((f32)x[r,c] * (f32)scale[r]) */
void orc_dequantize_linear(void *out, const int8_t *x, const void *scale,
                           size_t rows, size_t cols, int dtype);

/* A2 DequantMatMul.  act [M,K] (act_dtype), wq [N,K] int8, scale [N] and out [M,N] (out_dtype).
 * mode 0: scale after the f32 sum  (translator.rs:3208-3313 M=1; cuda dequant_gemv.cuh:12-59,
 *         dequant_matmul.cuh:12-51)
 * mode 1: W_f32 = scale*wq, then f32 GEMM (translator.rs:3053-3114, CPU M>1)
 * mode 2: W_T = round_T(scale*wq), then f32-accumulate GEMM (cuda dequant_matmul_wmma.cuh:65-76)
 * mode -1: what the reference CPU backend does: M==1 -> 0, else 1. */
void orc_dequant_matmul(void *out, const void *act, const int8_t *wq, const void *scale,
                        size_t M, size_t N, size_t K, int act_dtype, int out_dtype, int mode);

/* A3 QuantizedMatMul (cpu/kernels/qgemv_i8i8.rs:38-80): exact i32 accumulator, then
 * (f32)acc * lhs_scale[m] * rhs_scale[n] (left to right), stored as dtype.
 * acc_out (optional, may be NULL) receives the [M,N] i32 accumulators. */
void orc_quantized_matmul(void *out, int32_t *acc_out, const int8_t *lhs, const void *lhs_scale,
                          const int8_t *rhs, const void *rhs_scale,
                          size_t M, size_t N, size_t K, int dtype);

/* A4 DynamicQuantizeLinear, symmetric per row (cpu/kernels/dynquant_i8.rs:13-37):
 * s = amax/127 (1 for a zero row), y = clamp(round_half_away(x * (1/s)), -127, 127) */
void orc_dynquant_i8(int8_t *y, void *scale, const void *x, size_t M, size_t K, int dtype);
/* the same rule with one scale for the whole tensor (per-tensor fixtures) */
void orc_dynquant_i8_per_tensor(int8_t *y, void *scale, const void *x, size_t n, int dtype);
/* ONNX asymmetric uint8 form (cuda dynamic_quantize_linear.cuh:39-153), per row */
void orc_dynquant_u8_asym(uint8_t *y, void *scale, uint8_t *zp, const void *x,
                          size_t M, size_t K, int dtype);

/* A5 Attention (translator.rs:4440-5008).  q,out [B,Hq,Sq,D]; k,v [B,Hkv,Sk,D] (kv_dtype is
 * dtype, or 3 = int8 with k_scale/v_scale [B,Hkv,Sk] of dtype); active < 0 means "no
 * active_seq_kv input" (= Sk).  Keys visited: [0, min(active, causal cap, Sk)) where the
 * causal cap is (active - Sq) + sq + 1.  Online softmax per key, f32. */
void orc_attention(void *out, const void *q, const void *k, const void *v,
                   const void *k_scale, const void *v_scale, long long active,
                   size_t B, size_t Hq, size_t Hkv, size_t Sq, size_t Sk, size_t D,
                   int is_causal, float scale, int dtype, int kv_int8);
/* the same result by the two-pass textbook form in f64 (tests/session_state.rs:122-152) */
void orc_attention_f64(double *out, const void *q, const void *k, const void *v,
                       long long active, size_t B, size_t Hq, size_t Hkv, size_t Sq, size_t Sk,
                       size_t D, int is_causal, double scale, int dtype);

/* A6 KVCacheUpdate (translator.rs:4374-4423; cuda kvcache_update.cuh:6-26):
 * cache[bh, offset+t, :] = new[bh, t, :], in place */
void orc_kv_cache_update(void *cache, const void *new_kv, long long offset,
                         size_t BH, size_t S_new, size_t max_seq, size_t D, size_t elem_bytes);

/* A7 QuantizingKVCacheUpdate, CPU rule (translator.rs:4090-4372):
 * s = amax*(1/127); inv = amax==0 ? 0 : 127/amax; q = clamp((int)(x*inv +/- 0.5), -128, 127) */
void orc_quantizing_kv_cache_update(int8_t *cache, void *scale, const void *new_kv,
                                    long long offset, size_t BH, size_t S_new, size_t max_seq,
                                    size_t D, int dtype);

/* A8 RMSNormalization (translator.rs:5896-6027): y = (x * (1/sqrt(mean(x^2)+eps))) * w */
void orc_rms_norm(void *out, const void *x, const void *w, size_t rows, size_t dim,
                  double eps, int dtype);

/* A9 RoPE.  rope_table (crates/llm/src/builder.rs:359-393): f64 cos/sin(p * base^(-2i/D)),
 * halves duplicated, rounded to dtype.  rope (builder.rs:402-438 decomposed ==
 * translator.rs:6029-6176 fused): lo' = lo*cos[p,j] - hi*sin[p,j];
 * hi' = hi*cos[p,j+D/2] + lo*sin[p,j+D/2]; one rounding at the store.
 * x [outer,S,D]; position [S] selects the table row. */
void orc_rope_table(void *cos_t, void *sin_t, size_t max_seq, size_t D, float base, int dtype);
void orc_rope(void *out, const void *x, const void *cos_t, const void *sin_t,
              const int64_t *position, size_t outer, size_t S, size_t D, int dtype);

/* A10 Gather axis 0 with negative-index wrap (cuda gather.cuh:5-21) */
void orc_gather_rows(void *out, const void *data, const int64_t *idx, size_t n_idx,
                     size_t rows, size_t row_bytes);

/* A11 elementwise groups, f32 compute, one rounding (schedule/kernel.rs, cuda/kernel.rs:952-957)
 * swish: x * (1/(1+exp(-x))) (translator.rs:459-476,994-1001) */
void orc_swish(void *out, const void *x, size_t n, int dtype);
void orc_swiglu(void *out, const void *gate, const void *up, size_t n, int dtype);
void orc_add(void *out, const void *a, const void *b, size_t n, int dtype);

/* A13 greedy argmax, last maximum wins (crates/llm/src/session.rs:683-690) */
int64_t orc_argmax_last(const void *logits, size_t n, int dtype);

/* A14 per-output-channel int8 weight quantiser (crates/llm/src/quantize.rs:124-169):
 * scale = amax/127 (1 for a zero row); q = clamp(round_half_away(x/scale), -128, 127);
 * scale stored in scale_dtype (bf16 RNE in the reference) */
void orc_quantize_per_channel(int8_t *q, void *scale, const float *w, size_t rows, size_t cols,
                              int scale_dtype);

/* streaming-KV helpers (cuda common.cuh:55-60; crates/llm/src/session.rs:604-635) */
int  orc_ring_phys_index(int rank, int sink, int window, int start);
void orc_streaming_kv_position(int64_t *out, size_t sink, size_t window, size_t stream_pos,
                               size_t max_seq);

/* The two cache updates and the attention with the ring inputs, as the reference's CUDA kernels apply them
 * (kvcache_update.cuh:12-26, quantizing_kvcache_update.cuh:24-36, attention.cuh:100-200, 386-420, 495-606):
 * the only backend that has the mechanism.  `offset` may lie past sink + window (the session passes the
 * unbounded stream position); kv_position (NULL = keys are used as stored) is indexed by rank. */
void orc_kv_cache_update_ring(void *cache, const void *new_kv, long long offset, size_t BH, size_t S_new,
                              size_t max_seq, size_t D, size_t eb, int sink, int window, int start);
void orc_quantizing_kv_cache_update_ring(int8_t *cache, void *scale, const void *new_kv, long long offset,
                                         size_t BH, size_t S_new, size_t max_seq, size_t D, int dtype,
                                         int sink, int window, int start);
void orc_attention_ring(void *out, const void *q, const void *k, const void *v, const void *k_scale,
                        const void *v_scale, long long active, size_t B, size_t Hq, size_t Hkv, size_t Sq,
                        size_t Sk, size_t D, int is_causal, float scale, int dtype, int kv_int8, int sink,
                        int window, int start, const void *cos_t, const void *sin_t, const int64_t *kv_position);

/* ---- A12/A13: whole decoder + generate loop (crates/llm/src/decoder.rs:222-865,
 * session.rs:311-537).  Weights are int8 [N,K] + scale[N] (dtype) when quantised, or plain
 * dtype matrices when `wq` is NULL for a tensor (un-quantised checkpoints such as the tiny
 * random Llama run through Gemm: f32 accumulate, one rounding). */
typedef struct {
    int n_layers, hidden, n_heads, n_kv_heads, head_dim, ffn, vocab, max_seq;
    double eps;
    float rope_theta;
    int dtype;            /* activation / scale / KV storage type */
} orc_model_cfg;

typedef struct {
    const int8_t *q;      /* int8 [N,K] or NULL */
    const void *scale;    /* [N] dtype, when q != NULL */
    const void *w;        /* dtype [N,K] when q == NULL */
} orc_linear;

typedef struct orc_model orc_model;

orc_model *orc_model_create(const orc_model_cfg *cfg);
void orc_model_destroy(orc_model *m);
/* tensors are referenced, not copied; they must outlive the model */
void orc_model_set_embed(orc_model *m, orc_linear w);
void orc_model_set_lm_head(orc_model *m, orc_linear w);
void orc_model_set_final_norm(orc_model *m, const void *w);
/* which: 0 q, 1 k, 2 v, 3 o, 4 gate, 5 up, 6 down */
void orc_model_set_linear(orc_model *m, int layer, int which, orc_linear w);
/* which: 0 input_layernorm, 1 post_attention_layernorm */
void orc_model_set_norm(orc_model *m, int layer, int which, const void *w);
/* q / k / v projection bias (which 0 / 1 / 2), [N] in the model's dtype; NULL = none (llama, mistral).
 * crates/llm/src/decoder.rs:167-184 (Add after the MatMul), 542-600 (model_type "qwen2") */
void orc_model_set_bias(orc_model *m, int layer, int which, const void *b);
void orc_model_reset(orc_model *m);                 /* past_len = 0 (session.rs:303-305) */
/* which backend's DequantMatMul kernel choice the linears follow: -1 the CPU backend's (default),
 * 2 the CUDA backend's (rows >= 16: weight rounded to the 16-bit type before the product) */
void orc_model_set_gemm_mode(orc_model *m, int mode);
/* BuildOptions::quant_kv_cache (crates/llm/src/decoder.rs:672, 405-470: int8 caches + per-token scales,
 * QuantizingKVCacheUpdate, attention scale slots) and Options::quantize_activations
 * (src/transform/optimize/quantize_activations.rs: DynamicQuantizeLinear + QuantizedMatMul for every
 * int8 linear with K % 32 == 0).  Call before the first forward. */
void orc_model_set_options(orc_model *m, int quant_kv_cache, int quantize_activations);
const void *orc_model_k_scale(const orc_model *m, int layer);
const void *orc_model_v_scale(const orc_model *m, int layer);
long long orc_model_past_len(const orc_model *m);
void orc_model_set_past_len(orc_model *m, long long p);
/* One graph run with S tokens: positions[s], writes KV rows past_len..past_len+S-1, attends
 * keys [0, min(active, causal cap)); logits [S,vocab] in cfg.dtype.  Does not move past_len. */
void orc_model_forward(orc_model *m, const int64_t *ids, const int64_t *positions, size_t S,
                       long long past_len, long long active, int is_causal, void *logits);
/* The same run of the streaming graph (BuildOptions::streaming_kv, decoder.rs:281-347, 472-487) with the
 * session's eight inputs (session.rs:539-597): positions = clamped query positions, past_len = the unbounded
 * stream position, active = min(.., sink + window), ring_start, kv_position [max_seq]. */
void orc_model_forward_streaming(orc_model *m, const int64_t *ids, const int64_t *positions, size_t S,
                                 long long past_len, long long active, int is_causal, int sink, int window,
                                 int ring_start, const int64_t *kv_position, void *logits);
/* DecodeKind::LlamaStreaming { sink, window }: decode_step / prefill / generate then build the streaming
 * inputs themselves and never report PromptTooLong (session.rs:350-366); window 0 switches it off */
void orc_model_set_streaming(orc_model *m, int sink, int window);
/* decode_step (session.rs:508-537): forward one token at past_len, argmax, past_len += 1 */
int64_t orc_model_decode_step(orc_model *m, int64_t token);
/* chunked, zero-padded prefill (session.rs:426-485); returns argmax of the last real row */
int64_t orc_model_prefill(orc_model *m, const int64_t *ids, size_t n, size_t prefill_len);
/* generate_ids (session.rs:333-401) without tokenizer/stop strings: feeds the prompt token by
 * token when prefill_len == 0, else by prefill chunks.  Returns the number of new ids, or -1
 * for PromptTooLong. */
long long orc_model_generate(orc_model *m, const int64_t *prompt, size_t n_prompt,
                             size_t max_new, size_t prefill_len, int64_t eos, int64_t *out);
/* read access for layer-level parity checks */
const void *orc_model_k_cache(const orc_model *m, int layer);
const void *orc_model_v_cache(const orc_model *m, int layer);
const void *orc_model_last_hidden(const orc_model *m);   /* [S,hidden] before final norm */

#ifdef __cplusplus
}
#endif
#endif
