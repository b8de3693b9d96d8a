/*
 * litenn_oracle.h -- CPU restatement of LiteNN's CPU semantics for the GGUF
 * quantized LLaMA path.  TEST INFRASTRUCTURE ONLY.
 *
 * This library is the checker the HIP kernels are compared against.  Nothing
 * in the shipped package may link, load or call it: only the tests, the smoke
 * check and the CPU-baseline leg of the benchmark do, and only as the
 * reference side of a comparison.
 *
 * Every function restates, in plain C and in the same evaluation order, what
 * the reference executes on Interpreter<CPU>; the citation next to each
 * declaration is the reference file:line it follows (paths relative to the
 * reference tree).
 *
 * Pinning status
 *   - fp16 <-> f32, MatMul, transpose, RMSNorm, RoPE, attention chain, SiLU,
 *     SwiGLU, get_rows, KV append, block order: pinned by the reference's own
 *     test vectors (tests/golden/reference_vectors.json) plus closed forms.
 *   - block sizes / raw payload layout: pinned (Quantization.h:190-211,
 *     tests/GGUFImporterTest.cpp:173-178).
 *   - dequantised VALUES of Q4_0 / Q4_1 / Q5_0 / Q5_1 / Q8_0 / Q2_K / Q3_K / Q4_K / Q5_K / Q6_K:
 *     PARITY UNPINNED against
 *     the reference.  The arithmetic lives in ggml (third_party/llama.cpp, an
 *     empty, un-pinned submodule; call site tools/gguf/LLaMABuilder.cpp:95,149)
 *     and no reference test holds a dequantised value.  The decoders here
 *     restate ggml's published block definitions (dequantize_row_q4_0, _q4_1,
 *     _q5_0, _q5_1, _q8_0, _q2_K, _q3_K, _q4_K and _q5_K + get_scale_min_k4,
 *     _q6_K) and are cross-checked against an independently
 *     written numpy decoder, hand-packed closed-form blocks and reduction
 *     invariants, which is everything short of a real ggml build.
 */
#ifndef LITENN_ORACLE_H
#define LITENN_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* QuantizedBlockFormat positional values, src/LiteNN/Quantization.h:31-62 */
enum {
	ORACLE_FMT_Q4_0 = 1,
	ORACLE_FMT_Q4_1 = 2,
	ORACLE_FMT_Q5_0 = 3,
	ORACLE_FMT_Q5_1 = 4,
	ORACLE_FMT_Q8_0 = 5,
	ORACLE_FMT_Q2_K = 7,
	ORACLE_FMT_Q3_K = 8,
	ORACLE_FMT_Q4_K = 9,
	ORACLE_FMT_Q5_K = 10,
	ORACLE_FMT_Q6_K = 11,
	ORACLE_FMT_F16 = 25,
	ORACLE_FMT_F32 = 27,
};

/* --- scalar types ------------------------------------------------------ */
/* src/LiteNN/DType.h:112-134 (Float16BitsToFloat32) */
float oracle_f16_to_f32(uint16_t bits);
/* src/LiteNN/DType.h:63-110 (Float32ToFloat16Bits; rounds half UP on the dropped bit) */
uint16_t oracle_f32_to_f16(float value);
void oracle_f16_to_f32_array(const uint16_t* src, float* dst, size_t n);
void oracle_f32_to_f16_array(const float* src, uint16_t* dst, size_t n);

/* --- block formats ----------------------------------------------------- */
/* src/LiteNN/Quantization.h:186-217 (GetQuantizedBlockLayout). 0 on unknown. */
int oracle_block_elements(int fmt);
int oracle_block_bytes(int fmt);
/* bytes of one row of k elements, or 0 if k is not a whole number of blocks */
size_t oracle_row_bytes(int fmt, size_t k);

/* ggml to_float as called at tools/gguf/LLaMABuilder.cpp:144-150.
 * Returns 0 on success, -1 on unsupported format / k not a block multiple. */
int oracle_dequantize_row(int fmt, const uint8_t* src, float* dst, size_t k);
/* whole tensor [rows, k] -> f32 [rows, k] (the loop at LLaMABuilder.cpp:146-150) */
int oracle_dequantize(int fmt, const uint8_t* src, float* dst, size_t rows, size_t k);

/* --- dense primitives -------------------------------------------------- */
/* 2-D transpose, src/LiteNN/Device.h:500-511: dst[c,r] = src[r,c] */
void oracle_transpose(const float* src, float* dst, size_t rows, size_t cols);
/* BinaryOp::MatMul, src/LiteNN/Device.h:628-660: zero-fill then i-k-j, f32 */
void oracle_matmul_ikj(const float* x, const float* w, float* y, size_t m, size_t k, size_t n);

/* Linear layer over a GGUF-layout weight [n, k] (raw blocks):
 * dequantise (LLaMABuilder.cpp:144-150) -> transpose to [k, n] (:225-230) ->
 * i-k-j MatMul (Device.h:645-658).  Materialises the f32 weight exactly as the
 * reference does.  y is [m, n]. */
int oracle_mul_mat_q(int fmt, const uint8_t* wq, size_t n, size_t k, const float* x, size_t m, float* y);
/* Same values bit for bit, computed one output column at a time with the row
 * dequantised on the fly (each y[i,j] still accumulates x[i,k]*W[k,j] for k
 * ascending in f32 with separate multiply and add).  Uses OpenMP threads over
 * j; thread count does not change any result. */
int oracle_mul_mat_q_rowwise(int fmt, const uint8_t* wq, size_t n, size_t k, const float* x, size_t m, float* y);

/* NormalizationMode::RMSNorm, src/LiteNN/ComputePrimitives.h:771-821 via
 * src/LiteNN/Layer/RMSNorm.h:41-57.  x,y [m,d]; w [d] (may be NULL). */
void oracle_rmsnorm(const float* x, const float* w, double eps, size_t m, size_t d, float* y);

/* RoPE on [m, d] rows at positions pos_offset + row, interleaved pairs over
 * the first rope_dims features, tail copied.  src/LiteNN/Layer/RoPE.h:24-41,
 * 75-116 and tools/gguf/LLaMABuilder.cpp:311-348. */
void oracle_rope(const float* x, float* y, size_t m, size_t d, size_t rope_dims, double base, double freq_scale,
                 size_t pos_offset);

/* One head of AddFlashAttnExt with scale + optional causal mask (no softcap,
 * ALiBi or sinks): src/LiteNN/Layer/FlashAttnExt.h:126-228,
 * src/LiteNN/Layer/CausalMask.h:16-34.  q [mq,d], k [l,d], v [l,dv], out [mq,dv]. */
void oracle_attention_head(const float* q, size_t mq, const float* k, const float* v, size_t l, size_t d, size_t dv,
                           double scale, int causal, size_t key_pos_offset, size_t query_pos_offset, float* out);

/* Detail::ComputeALiBiSlope, src/LiteNN/Layer/FlashAttnExt.h:69-96 */
double oracle_alibi_slope(size_t head_index, size_t head_count, double max_bias);
/* One head of AddFlashAttnExt with every option (src/LiteNN/Layer/FlashAttnExt.h:17-29,126-228):
 * logit softcap (tanh composed as in Activation.h:34-50), additive mask [mq, l] times mask_slope
 * (oracle_alibi_slope, 1 when maxBias is off; NULL = no mask), scalar sink (NULL = none), causal
 * mask with position offsets. */
void oracle_flash_attn_ext(const float* q, size_t mq, const float* k, const float* v, size_t l, size_t d, size_t dv,
                           double scale, double logit_softcap, const float* mask, double mask_slope,
                           const float* sink, int causal, size_t key_pos_offset, size_t query_pos_offset, float* out);

/* AddSiLU / AddSigmoid, src/LiteNN/Layer/Activation.h:22-63 */
void oracle_silu(const float* x, float* y, size_t n);
/* gated = silu(gate) * up, src/LiteNN/Layer/SwiGLU.h:59-69 */
void oracle_silu_mul(const float* gate, const float* up, float* y, size_t n);
/* DoGetRowsOp, src/LiteNN/Device.h:825-883.  -1 if an index is out of range. */
int oracle_get_rows(const float* table, size_t rows, size_t cols, const int32_t* idx, size_t n, float* out);
/* first maximal index (ties: lowest index, cf. src/LiteNN/Runtime/Interpreter.h:134-163) */
int32_t oracle_argmax(const float* x, size_t n);

/* --- LLaMA decoder ----------------------------------------------------- */
typedef struct oracle_llama oracle_llama;

enum {
	ORACLE_T_TOKEN_EMBD = 0, /* [vocab, d_model] */
	ORACLE_T_OUTPUT = 1,     /* [vocab, d_model]; absent => tied to token_embd */
	ORACLE_T_ATTN_Q = 2,     /* [n_head*head_dim, d_model] */
	ORACLE_T_ATTN_K = 3,     /* [n_kv_head*head_dim, d_model] */
	ORACLE_T_ATTN_V = 4,
	ORACLE_T_ATTN_OUTPUT = 5, /* [d_model, n_head*head_dim] */
	ORACLE_T_FFN_GATE = 6,    /* [d_ff, d_model] */
	ORACLE_T_FFN_UP = 7,
	ORACLE_T_FFN_DOWN = 8, /* [d_model, d_ff] */
	ORACLE_T_OUTPUT_NORM = 9, /* f32 [d_model] */
	ORACLE_T_ATTN_NORM = 10,
	ORACLE_T_FFN_NORM = 11,
};

/* Hyper-parameters as parsed at tools/gguf/GGUFImporter.cpp:505-642.
 * kv_f16 != 0 stores K (already rotated) and V rounded to Float16 with
 * oracle_f32_to_f16 (the harness's fp16 KV cache); 0 keeps f32 as the
 * reference graph does (tools/gguf/LLaMABuilder.cpp:848-849).
 * materialize != 0 dequantises every matrix to f32 [k,n] up front exactly like
 * the lowering; 0 uses the bit-identical row-wise form to bound host memory. */
oracle_llama* oracle_llama_new(int n_layer, int d_model, int n_head, int n_kv_head, int d_ff, int vocab, int ctx,
                               int rope_dims, double rms_eps, double rope_base, double rope_freq_scale, int kv_f16,
                               int materialize);
void oracle_llama_free(oracle_llama* m);
/* data must stay alive while the model is used (not copied unless materialize). */
int oracle_llama_set_tensor(oracle_llama* m, int which, int layer, int fmt, const void* data, size_t n, size_t k);
/* past length currently held in the KV cache */
int oracle_llama_past(const oracle_llama* m);
void oracle_llama_reset(oracle_llama* m);
/* LowerLLaMACausalLMDecode(sequenceLength=m_tokens, pastLength=positionOffset=past)
 * run on the cache held by the model; appends to the cache.  logits is
 * [m_tokens, vocab] or NULL; last_logits [vocab] or NULL.
 * tools/gguf/LLaMABuilder.cpp:568-668,774-800,826-872.  Returns 0, or -1 on
 * bad token id / context overflow / missing tensor. */
int oracle_llama_eval(oracle_llama* m, const int32_t* tokens, int m_tokens, float* logits, float* last_logits);
/* greedy loop of the harness: eval(prompt) then n_new times argmax->eval.
 * out_tokens [n_new]; margins [n_new] (top1 - top2 logit) may be NULL. */
int oracle_llama_generate(oracle_llama* m, const int32_t* prompt, int n_prompt, int n_new, int32_t* out_tokens,
                          float* margins);
/* copy of the cache: k,v [past, n_kv_head*head_dim] f32 (rounded values if kv_f16) */
int oracle_llama_get_kv(const oracle_llama* m, int layer, float* k, float* v);
/* Harness convenience, no counterpart in the reference: restore `rows` cache rows saved with
 * oracle_llama_get_kv, and set the position (resuming a long checker run). */
int oracle_llama_set_kv(oracle_llama* m, int layer, int rows, const float* k, const float* v);
int oracle_llama_set_past(oracle_llama* m, int past);

const char* oracle_last_error(void);
void oracle_set_threads(int n);

#ifdef __cplusplus
}
#endif
#endif
