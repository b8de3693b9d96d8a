/*
 * litenn_hip.h -- C ABI of the MI355X (gfx950) device backend for LiteNN's
 * GGUF-quantised LLaMA path.
 *
 * The first group of entry points is what a DeviceTraits<HIP> specialisation
 * binds, one call per static member of the reference's Device concept
 * (src/LiteNN/Device.h:17-69), modelled on DeviceTraits<CUDA>
 * (src/LiteNN/Device/CUDA.h:98-165).  The second group are extensions the
 * reference has no counterpart for, because it dequantises GGUF blocks to f32
 * on the host at lowering time (tools/gguf/LLaMABuilder.cpp:66-162): they
 * consume the raw block payload exactly as the importer stores it
 * (tools/gguf/GGUFImporter.cpp:478-491).  The third group is the decoder
 * runtime that replaces "lower a static graph per (sequenceLength,
 * pastLength) and interpret it" (tools/gguf/LLaMABuilder.cpp:826-872,
 * src/LiteNN/Runtime/Interpreter.h:35-43).
 *
 * Conventions
 *  - every function returns 0 on success and a non-zero status otherwise;
 *    litenn_hip_last_error() then holds "<action> failed: <message>" for the
 *    calling thread (the reference throws std::runtime_error with that text,
 *    src/LiteNN/Device/CUDA.cpp:89-95).
 *  - `dtype` uses DataType's positional values (src/LiteNN/DType.h:17-30),
 *    `fmt` uses QuantizedBlockFormat's (src/LiteNN/Quantization.h:31-62).
 *  - sizes are ELEMENT counts, never bytes (src/LiteNN/Device.h:28-31).
 *  - tensors are row-major and contiguous.
 *  - `opts` mirrors CUDAExecutionOptions (src/LiteNN/Device/CUDA.h:70-74):
 *    NULL means stream 0 and synchronise before returning.
 *  - the entry points of groups 1, 2 and 4 may be called from several host threads at
 *    once; each call selects `dev` for its own duration (cf. CUDADeviceGuard,
 *    src/LiteNN/Device/CUDA.cpp:734-761).  A litenn_hip_llama handle (group 3) is a
 *    mutable object -- cache position, scratch buffers, the captured step -- and must
 *    not be used by two threads at the same time; separate handles run side by side.
 *    litenn_hip_attn_decode_noalloc shares one scratch array per GPU between all its
 *    calls (see there).
 */
#ifndef LITENN_HIP_H
#define LITENN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* DataType, src/LiteNN/DType.h:17-30 */
enum litenn_dtype {
	LITENN_F32 = 0, LITENN_F64 = 1, LITENN_I32 = 2, LITENN_I64 = 3, LITENN_BOOL = 4, LITENN_F16 = 5,
	LITENN_BF16 = 6, LITENN_F8E4M3 = 7, LITENN_F8E5M2 = 8, LITENN_I8 = 9, LITENN_U8 = 10,
};

/* QuantizedBlockFormat, src/LiteNN/Quantization.h:31-62 (only the members this backend executes:
 * the ggml formats that have a dequantizer and a layout in the reference's table, :186-217; Q8_1 and
 * Q8_K have none in ggml and are refused, as tools/gguf/LLaMABuilder.cpp:95-101 refuses them).
 * All of them are decoded inside the streaming GEMV and the matrix-core GEMM. */
enum litenn_block_format {
	LITENN_FMT_Q4_0 = 1, LITENN_FMT_Q4_1 = 2, LITENN_FMT_Q5_0 = 3, LITENN_FMT_Q5_1 = 4, LITENN_FMT_Q8_0 = 5,
	LITENN_FMT_Q2_K = 7, LITENN_FMT_Q3_K = 8, LITENN_FMT_Q4_K = 9, LITENN_FMT_Q5_K = 10, LITENN_FMT_Q6_K = 11,
	LITENN_FMT_F16 = 25, LITENN_FMT_F32 = 27,
};

/* UnaryOp / BinaryOp / ReduceOp, src/LiteNN/Operators.h:12-51,237-242 */
enum litenn_unary_op {
	LITENN_UN_NEGATE = 0, LITENN_UN_ABS, LITENN_UN_SQRT, LITENN_UN_EXP, LITENN_UN_LOG, LITENN_UN_SIN, LITENN_UN_COS,
	LITENN_UN_TAN, LITENN_UN_ARCSIN, LITENN_UN_ARCCOS, LITENN_UN_ARCTAN, LITENN_UN_TRANSPOSE,
	LITENN_UN_LOGICAL_NEGATION, LITENN_UN_ERF,
};
enum litenn_binary_op {
	LITENN_BIN_ADD = 0, LITENN_BIN_SUBTRACT, LITENN_BIN_MULTIPLY, LITENN_BIN_DIVIDE, LITENN_BIN_MATMUL, LITENN_BIN_POW,
	LITENN_BIN_MAX, LITENN_BIN_MIN, LITENN_BIN_LESS, LITENN_BIN_GREATER, LITENN_BIN_EQUAL,
};
enum litenn_reduce_op { LITENN_RED_SUM = 0, LITENN_RED_MEAN = 1, LITENN_RED_MAX = 2 };

/* CUDAExecutionOptions, src/LiteNN/Device/CUDA.h:70-74 */
typedef struct litenn_hip_exec {
	void* stream;    /* hipStream_t, NULL = null stream */
	int synchronize; /* non-zero: hipStreamSynchronize before returning */
} litenn_hip_exec;

const char* litenn_hip_last_error(void);

/* ---- group 1: the Device concept ------------------------------------- */

/* CUDADeviceCount, src/LiteNN/Device/CUDA.cpp:1400-1416.  Never fails; 0 when no GPU. */
int litenn_hip_device_count(void);
/* DeviceTraits<CUDA>::Info, src/LiteNN/Device/CUDA.cpp:1735-1751 */
int litenn_hip_device_info(int dev, char* buf, size_t buf_len);
/* Allocate / Deallocate / ZeroFill, src/LiteNN/Device.h:28-34, CUDA.cpp:1753-1777.
 * Memory is uninitialised; the caller frees with the same (dtype, n). */
int litenn_hip_alloc(int dev, int dtype, size_t n, void** out);
int litenn_hip_free(int dev, void* ptr, int dtype, size_t n);
int litenn_hip_zero(int dev, void* ptr, int dtype, size_t n);
/* CopyToCPU / CopyFromCPU / ConvertTo, src/LiteNN/Device.h:35-39, CUDA.cpp:1785-1892.
 * Synchronous on return unless opts says otherwise; dtype may change: every pair of the eleven
 * element types converts as static_cast does on the CPU, Float16 / BFloat16 / Float8E4M3 /
 * Float8E5M2 through LiteNN's own constructors (src/LiteNN/DType.h:58-229). */
int litenn_hip_copy_to_host(int dev, int src_dtype, const void* src, size_t n, int dst_dtype, void* dst,
                            const litenn_hip_exec* opts);
int litenn_hip_copy_from_host(int dev, int dst_dtype, void* dst, int src_dtype, const void* src, size_t n,
                              const litenn_hip_exec* opts);
int litenn_hip_convert(int dev, int src_dtype, const void* src, size_t n, int dst_dtype, void* dst,
                       const litenn_hip_exec* opts);
/* DoUnaryOp, src/LiteNN/Device.h:42-44 (CPU semantics :393-511) */
int litenn_hip_unary(int dev, int op, void* dst, int dtype, const size_t* shape, size_t rank, const void* src,
                     const litenn_hip_exec* opts);
/* DoBinaryOp, src/LiteNN/Device.h:45-49 (CPU semantics :513-689; MatMul :628-660).
 * Broadcast aligns LEADING dimensions (src/LiteNN/Operators.h:173-188). */
int litenn_hip_binary(int dev, int op, void* dst, int dtype1, const size_t* shape1, size_t rank1, const void* src1,
                      int dtype2, const size_t* shape2, size_t rank2, const void* src2, const litenn_hip_exec* opts);
/* DoReduceOp, src/LiteNN/Device.h:50-52 (:691-759) */
int litenn_hip_reduce(int dev, int op, void* dst, int dtype, const size_t* shape, size_t rank, const void* src,
                      size_t axis, const litenn_hip_exec* opts);
/* DoConcatOp, src/LiteNN/Device.h:53-58 (:761-792).  shapes is input_count rows of `rank` extents. */
int litenn_hip_concat(int dev, void* dst, int dtype, const void* const* srcs, const size_t* shapes, size_t rank,
                      size_t input_count, size_t axis, const litenn_hip_exec* opts);
/* DoSliceOp, src/LiteNN/Device.h:59-60 (:794-823) */
int litenn_hip_slice(int dev, void* dst, int dtype, const size_t* src_shape, size_t rank, const void* src, size_t axis,
                     size_t start, size_t length, const litenn_hip_exec* opts);
/* DoGetRowsOp, src/LiteNN/Device.h:61-64 (:825-883).  index_dtype is I32 or I64; an
 * out-of-range index fails with "GetRows index out of range". */
int litenn_hip_get_rows(int dev, void* dst, int dtype, const size_t* data_shape, size_t data_rank, const void* data,
                        int index_dtype, const size_t* index_shape, size_t index_rank, const void* indices,
                        const litenn_hip_exec* opts);
/* DoPermuteOp, src/LiteNN/Device.h:65-68 (:885-966).  perm[d] = input axis of output axis d. */
int litenn_hip_permute(int dev, void* dst, int dtype, const size_t* src_shape, size_t rank, const void* src,
                       const size_t* perm, const litenn_hip_exec* opts);

/* ---- group 2: quantised extensions (no reference counterpart) -------- */

/* y[m, n] (f32) = x[m, k] . deq(wq)[n, k]^T with f32 accumulation, i.e. the value
 * AddLinear produces after the lowering's dequantise + transpose
 * (tools/gguf/LLaMABuilder.cpp:144-150,225-230; src/LiteNN/Layer/Linear.h:67-95).
 * wq is the raw GGUF payload: n rows of k/block blocks.  x_dtype is F32; F16 and BF16
 * activations are accepted too and widened exactly into a Float32 copy first (the copy is taken
 * from and returned to the device's memory pool in stream order, see below).
 * residual (f32 [m, n]) may be NULL; when given, y = residual + x.W
 * (the Add at tools/gguf/LLaMABuilder.cpp:652-653,661-663).  residual may alias y.
 * m == 1..3 runs the streaming GEMV, row by row (f32 operands).  m >= 4 (with k a multiple of 256;
 * the threshold was 16 in earlier versions of this library, and a caller that sized a workspace
 * for 4 <= m < 16 by that rule - zero bytes - must size it with
 * litenn_hip_mul_mat_q_workspace_bytes now) runs on the
 * matrix cores (the rows padded to a multiple of 16; one padded tile costs about as much as three
 * single-row launches): weights and activations are rounded to fp16 once each (activation rows are first scaled
 * by a power of two into the fp16 range), products accumulate in f32; relative L2 error about
 * 4e-4.  LITENN_HIP_MATMUL_PRECISE in `flags` keeps f32 operands (GEMV path) for any m.
 * The matrix-core path needs a device workspace of litenn_hip_mul_mat_q_workspace_bytes(m, k):
 * litenn_hip_mul_mat_q takes it from the device's memory pool in stream order (hipMallocAsync /
 * hipFreeAsync on the call's stream: no wait for the stream, opts->synchronize is honoured; only
 * where the device has no memory pools does the call fall back to hipMalloc and drain the stream);
 * litenn_hip_mul_mat_q_ws takes the caller's (16-byte aligned; NULL = as above).
 * m <= 32 against a single matrix whose k is a multiple of 2048 takes a streaming form of the
 * matrix-core kernel (one launch, every weight byte read once).
 * A workspace larger than that (rounded up to 16) by 4*m*n bytes, or by three times as much,
 * also lets a launch that would leave the card short of work walk K in two, or four, parts at
 * once (k >= 8192 with 128 x 128 tiles on half the card; m <= 32 or so, where the launch is a
 * stream of the weights); the parts are added in K order, so results do not depend on
 * scheduling. */
#define LITENN_HIP_MATMUL_PRECISE 1u
int litenn_hip_mul_mat_q(int dev, int fmt, const void* wq, size_t n, size_t k, const void* x, int x_dtype, size_t m,
                         void* y, const void* residual, unsigned flags, const litenn_hip_exec* opts);
size_t litenn_hip_mul_mat_q_workspace_bytes(size_t m, size_t k);
/* Measurement aid, no reference counterpart: writes into out (capacity bytes, always terminated)
 * which instance of the streaming single-row kernel the calling thread's last m == 1 matmul or
 * linear group launched and with what geometry, e.g.
 * "gemv_stream_kernel<Q4_KUnit, 2, true, 512> grid 256 x 512 threads, 83968 B LDS, runs of 8 and 6 rows"
 * ("none" before the first such launch).  The name is the one a kernel trace shows. */
int litenn_hip_gemv_last_launch(char* out, size_t capacity);
/* The same for the matrix cores: the calling thread's last launch for m >= 4 rows, e.g.
 * "gemm_q_kernel<4, 1, 8, 2> grid 224 x 1 x 1, 512 threads, 118784 B LDS" (activation tiles and
 * weight groups of a workgroup's tile, its wavefronts, the groups of them that split the tile's K
 * range; grid z = K ranges walked by separate workgroups), "gemm_stream_kernel<1, 1, 16> ..." for
 * the streaming form of few rows.  No reference counterpart. */
int litenn_hip_gemm_last_launch(char* out, size_t capacity);
int litenn_hip_mul_mat_q_ws(int dev, int fmt, const void* wq, size_t n, size_t k, const void* x, int x_dtype, size_t m,
                            void* y, const void* residual, unsigned flags, void* workspace, size_t workspace_bytes,
                            const litenn_hip_exec* opts);
/* One activation row through an operator group of the decoder block, fused into a single
 * launch when the shape allows and composed from separate launches otherwise:
 *   [RMSNorm(x, norm_w, eps)] -> count (1..3) linears of one format sharing that input
 *   -> [residual added to y[0]] or [SwiGLU: y[0] = silu(x.W0) * (x.W1)]
 * i.e. AddRMSNorm + AddLinear x3 (tools/gguf/LLaMABuilder.cpp:588-591), the front half of
 * AddSwiGLUMLP (src/LiteNN/Layer/SwiGLU.h:59-66), or AddLinear + Add (:652-653,661-663).
 * wq[i] is [n[i], k] raw payload, y[i] f32 [n[i]]; norm_w (f32 [k]) and residual (f32 [n[0]],
 * count == 1 only, may alias y[0]) may be NULL; with LITENN_HIP_GROUP_SILU_MUL count must be 2
 * with n[0] == n[1] and only y[0] is written. */
#define LITENN_HIP_GROUP_SILU_MUL 1u
int litenn_hip_linear_group(int dev, int fmt, size_t count, const void* const* wq, const size_t* n, size_t k,
                            const void* x, void* const* y, const void* residual, const void* norm_w, double eps,
                            unsigned flags, const litenn_hip_exec* opts);
/* f32 [rows, k] = dequantised rows of wq (ggml to_float as called at
 * tools/gguf/LLaMABuilder.cpp:144-150). */
int litenn_hip_dequantize(int dev, int fmt, const void* wq, size_t rows, size_t k, void* dst,
                          const litenn_hip_exec* opts);
/* out[i, :] = deq(table)[ids[i], :]; ids are I32 on the device
 * (AddLLaMATokenEmbedding, tools/gguf/LLaMABuilder.cpp:738-759). */
int litenn_hip_get_rows_q(int dev, int fmt, const void* table, size_t rows, size_t k, const void* ids, size_t n_ids,
                          void* out, const litenn_hip_exec* opts);
/* RMSNorm over the last axis with f64 accumulation: y = x / sqrt(mean(x^2) + eps) * w
 * (src/LiteNN/Layer/RMSNorm.h:41-57, src/LiteNN/ComputePrimitives.h:792-817).  w may be NULL. */
int litenn_hip_rmsnorm(int dev, const void* x, const void* w, double eps, size_t m, size_t d, void* y,
                       const litenn_hip_exec* opts);
/* Interleaved-pair RoPE on x[m, n_heads, head_dim] (f32) at positions pos_offset + row,
 * first rope_dims features of every head, tail copied
 * (src/LiteNN/Layer/RoPE.h:24-117, tools/gguf/LLaMABuilder.cpp:311-348). */
int litenn_hip_rope_interleaved(int dev, const void* x, void* y, size_t m, size_t n_heads, size_t head_dim,
                                size_t rope_dims, double base, double freq_scale, size_t pos_offset,
                                const litenn_hip_exec* opts);
/* cache[past + i, :] = convert(cur[i, :]) for i < m; cache dtype F16 or F32
 * (AddKVCacheAppend, src/LiteNN/Layer/KVCache.h:87-104; f32 -> Float16 rounding of
 * src/LiteNN/DType.h:63-110). */
int litenn_hip_kv_append(int dev, void* cache, int cache_dtype, size_t past, const void* cur, size_t m, size_t width,
                         const litenn_hip_exec* opts);
/* Causal attention of m query rows at positions past..past+m-1 against a cache holding
 * past+m rows: q [m, n_head, head_dim] f32 (already rotated), k/v cache
 * [>= past+m, n_kv_head, head_dim] F16 or F32, out [m, n_head, head_dim] f32; scale
 * 1/sqrt(head_dim); query head h reads kv head h / (n_head / n_kv_head)
 * (tools/gguf/LLaMABuilder.cpp:624-645, src/LiteNN/Layer/FlashAttnExt.h:126-228). */
int litenn_hip_attn_decode(int dev, const void* q, const void* kcache, const void* vcache, int cache_dtype, size_t m,
                           size_t past, size_t n_head, size_t n_kv_head, size_t head_dim, void* out,
                           const litenn_hip_exec* opts);
/* litenn_hip_attn_decode for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): same operands and the same
 * result, bit for bit, but the chunk triples and arrival counters that a single row against a
 * long cache needs live in a fixed array of 1 MiB + 4 KiB inside the library's code object (one copy per
 * GPU, held until the process ends) instead of memory allocated and freed by the call.  No
 * counterpart in the reference.  The call allocates nothing, records no memset node, and honours
 * opts->synchronize like every other entry point.  It refuses a launch whose chunks do not fit:
 * a single row (m == 1) is cut into c = min(16, max(1, round(2.2 * sqrt(keys / 64))),
 * ceil(1024 / n_head)) chunks (2 from 30 keys on, 3 at 128, 6 at 512, 16 from 3400 on) and needs n_head * c * (head_dim + 2) <= 262144 floats, which holds
 * for every head_dim <= 128 and, at the 16 chunks of a long cache, e.g. for 48 heads of 256
 * features but not for 64.  Every call on one GPU shares that GPU's array:
 * calls that overlap on one GPU (two streams, two threads) race and must be serialised by the
 * caller. */
int litenn_hip_attn_decode_noalloc(int dev, const void* q, const void* kcache, const void* vcache, int cache_dtype,
                                   size_t m, size_t past, size_t n_head, size_t n_kv_head, size_t head_dim, void* out,
                                   const litenn_hip_exec* opts);
/* The same attention for a prompt's rows (the multi-row lowering of
 * tools/gguf/LLaMABuilder.cpp:350-404,502-557; mask of src/LiteNN/Layer/CausalMask.h:16-56):
 * with m >= 16, an F16 cache, 128-wide heads and 16-byte aligned buffers both contractions
 * run on the matrix cores (fp16 operands: q / sqrt(d)
 * and the softmax weights are rounded once, f32 accumulation and softmax; relative L2 error
 * about 3e-4), tiled so that the keys are read once per 64 rows instead of once per row.
 * flags: LITENN_HIP_MATMUL_PRECISE keeps the f32 row kernel of litenn_hip_attn_decode, which
 * every other shape uses as well. */
int litenn_hip_attn_rows(int dev, const void* q, const void* kcache, const void* vcache, int cache_dtype, size_t m,
                         size_t past, size_t n_head, size_t n_kv_head, size_t head_dim, void* out, unsigned flags,
                         const litenn_hip_exec* opts);
/* The options of the reference's attention layer (FlashAttnExtOptions,
 * src/LiteNN/Layer/FlashAttnExt.h:17-29) for all heads of one call; headIndex / headCount are the
 * head's index and n_head. */
typedef struct litenn_hip_attn_ext_opts
{
	double scale;         /* multiplies q.k; 1 = none */
	double max_bias;      /* > 0: the mask is multiplied by the head's ALiBi slope; needs a mask */
	double logit_softcap; /* != 0: scores become softcap * tanh(scale * q.k / softcap) */
	const void* mask;     /* additive F32 [m, keys] on the device, shared by the heads, or NULL */
	const void* sinks;    /* F32 [n_head] on the device, one scalar sink per head, or NULL */
	int causal;           /* adds -1e9 where key_position_offset + key > query_position_offset + row */
	size_t key_position_offset;
	size_t query_position_offset;
} litenn_hip_attn_ext_opts;
/* AddFlashAttnExt with its options for every head at once
 * (src/LiteNN/Layer/FlashAttnExt.h:100-228; causal mask src/LiteNN/Layer/CausalMask.h:16-34; tanh
 * as the layer composes it, src/LiteNN/Layer/Activation.h:34-50): q [m, n_head, head_dim] F32,
 * k / v [keys, n_kv_head, head_dim] F16 or F32, out [m, n_head, head_dim] F32; query head h reads kv
 * head h / (n_head / n_kv_head).  o == NULL means no option (scale 1, no mask).  The LLaMA lowering
 * uses none of the options and goes through litenn_hip_attn_decode / litenn_hip_attn_rows; this
 * entry point is a plain f32 row kernel.  The tanh is (exp(2x) - 1) / (exp(2x) + 1) in f32 as in the
 * reference, NaN once 2x exceeds 88.  Refused: max_bias without a mask (the reference's text), a
 * causal mask that hides every key from the first row (key_position_offset beyond
 * query_position_offset; the reference computes a softmax over scores of -1e9 there), more than
 * 65535 query rows or heads.  Keys hidden by the causal mask are skipped, where the reference adds
 * -1e9 to their scores (src/LiteNN/Layer/FlashAttnExt.h:169): the same result whenever a row keeps
 * a visible key whose score is far above -1e9; a user mask that drives every visible key of a row to
 * about -1e9 or to -inf is outside what the tests pin against the reference. */
int litenn_hip_flash_attn_ext(int dev, const void* q, const void* k, const void* v, int kv_dtype, size_t m, size_t keys,
                              size_t n_head, size_t n_kv_head, size_t head_dim, const litenn_hip_attn_ext_opts* o,
                              void* out, const litenn_hip_exec* opts);
/* y = silu(gate) * up (src/LiteNN/Layer/SwiGLU.h:59-69, Activation.h:22-63) */
int litenn_hip_silu_mul(int dev, const void* gate, const void* up, void* y, size_t n, const litenn_hip_exec* opts);
/* out_index[row] (I32) = first maximal index of x[row, :] (f32); ties pick the lowest index
 * (cf. the stable sort at src/LiteNN/Runtime/Interpreter.h:134-163). */
int litenn_hip_argmax(int dev, const void* x, size_t rows, size_t n, void* out_index, const litenn_hip_exec* opts);

/* ---- group 3: LLaMA decoder runtime ----------------------------------- */

typedef struct litenn_hip_llama litenn_hip_llama;

/* tensor ids for litenn_hip_llama_set_tensor; shapes are GGUF [n, k] = [out, in] */
enum litenn_llama_tensor {
	LITENN_T_TOKEN_EMBD = 0, LITENN_T_OUTPUT = 1, LITENN_T_ATTN_Q = 2, LITENN_T_ATTN_K = 3, LITENN_T_ATTN_V = 4,
	LITENN_T_ATTN_OUTPUT = 5, LITENN_T_FFN_GATE = 6, LITENN_T_FFN_UP = 7, LITENN_T_FFN_DOWN = 8,
	LITENN_T_OUTPUT_NORM = 9, LITENN_T_ATTN_NORM = 10, LITENN_T_FFN_NORM = 11,
};

/* Hyper-parameters as ParseLLaMAHyperparameters yields them
 * (tools/gguf/GGUFImporter.cpp:505-642).  kv_dtype is F16 or F32.  context_length is bounded by
 * 2^30 positions and by the memory of the caches it sizes
 * (2 * block_count * context_length * head_count_kv * head_dim elements of kv_dtype). */
typedef struct litenn_hip_llama_params {
	int32_t block_count, embedding_length, head_count, head_count_kv, feed_forward_length, vocab_size,
	    context_length, rope_dimension_count;
	double rms_norm_epsilon, rope_freq_base, rope_freq_scale;
	int32_t kv_dtype;
} litenn_hip_llama_params;

int litenn_hip_llama_create(int dev, const litenn_hip_llama_params* params, litenn_hip_llama** out);
int litenn_hip_llama_free(litenn_hip_llama* model);
/* `data` is DEVICE memory holding the raw payload (or f32 for the norm weights); it is
 * referenced, not copied, and must outlive the model.  LITENN_T_OUTPUT may be left unset:
 * the head is then tied to token_embd (tools/gguf/LLaMABuilder.cpp:719-733). */
int litenn_hip_llama_set_tensor(litenn_hip_llama* model, int which, int layer, int fmt, const void* data, size_t n,
                                size_t k);
int litenn_hip_llama_reset(litenn_hip_llama* model);
int litenn_hip_llama_past(const litenn_hip_llama* model);
/* How the single-token step runs a decoder block's attention half (no reference counterpart): 1 = as
 * one launch (norm + q/k/v, rotation + append + attention, output projection; models 4096 wide
 * with 32 heads of 128, a Float16 cache and Q4_0 / Q4_K weights on a card of 256 CUs), -1 = as
 * separate launches (the shape is another, LITENN_HIP_ATTN_BLOCK=0 was set when the step was first
 * built, or a bounded wait inside the launch once ran out and the step was repeated), 0 = not yet
 * decided (no single-token step has run since the model's tensors were set). */
int litenn_hip_llama_block_form(const litenn_hip_llama* m);
/* LowerLLaMACausalLMDecode(sequenceLength = m, pastLength = positionOffset = past) executed
 * against the cache the model holds (tools/gguf/LLaMABuilder.cpp:826-872); tokens are host
 * I32.  logits (host f32 [m, vocab]) and last_logits (host f32 [vocab]) may be NULL.
 * flags: LITENN_HIP_MATMUL_PRECISE keeps f32 activations for m >= 4. */
int litenn_hip_llama_eval(litenn_hip_llama* model, const int32_t* tokens, size_t m, float* logits, float* last_logits,
                          unsigned flags);
/* Greedy loop kept on the device: eval(prompt), then n_new times argmax -> eval of that
 * token.  out_tokens is host I32 [n_new].  decode_ms (may be NULL) receives the
 * device time of the n_new - 1 single-token steps. */
int litenn_hip_llama_generate(litenn_hip_llama* model, const int32_t* prompt, size_t n_prompt, size_t n_new,
                              int32_t* out_tokens, unsigned flags, double* prefill_ms, double* decode_ms);
/* Copies the first `past` cache rows of one layer to host as f32 [past, n_kv_head*head_dim]. */
int litenn_hip_llama_get_kv(litenn_hip_llama* model, int layer, float* k, float* v);

/* ---- group 4: weight container readers (host side) --------------------- */

/* A dependency-free reader of the GGUF container (versions 2 and 3), producing what
 * ImportGGUFArchive produces (tools/gguf/GGUFImporter.cpp:644-678) without ggml: metadata
 * widened to u64 / i64 / f64 / bool / string (:339-437), tensors as (type, shape with the
 * slowest dimension first, :206-221, raw payload, :457-502), LLaMA hyper-parameters with the
 * defaults and checks of ParseLLaMAHyperparameters (:505-642).  The file is mapped read-only;
 * pointers handed out stay valid until litenn_gguf_close.  Error texts are the reference's.
 *
 * litenn_gguf_open also takes a LiteNN model archive (.ltnn, magic "LTNNMDL\0", versions 6..18,
 * src/LiteNN/Serialization/ModelIO.h:25-26,1291-1341), the reference's own on-disk form of an
 * imported model: its variable table (names, tensors, quantisation records with block format and
 * expressed shape, :281-338,592-612) and metadata entries (:27-39,447-505) come before the graph
 * and are exposed through the same handle and accessors; the graph itself is not read.  For such
 * a file litenn_gguf_version returns the archive version and a tensor's ggml_type is the id of
 * its block format's ggml type (negative for plain types ggml has no id for). */
typedef struct litenn_gguf litenn_gguf;

typedef struct litenn_gguf_tensor {
	const char* name;
	int ggml_type;      /* id of the published ggml_type enum */
	int fmt;            /* QuantizedBlockFormat this backend executes, or -1 */
	int dtype;          /* DataType of a plain tensor, or -1 */
	int quantized;      /* non-zero for block formats */
	size_t rank;
	size_t shape[4];    /* slowest dimension first: a [N, K] weight has shape {N, K} */
	size_t file_offset; /* of the payload, from the start of the file */
	size_t bytes;
	const void* data;   /* the payload inside the mapping */
} litenn_gguf_tensor;

int litenn_gguf_open(const char* path, litenn_gguf** out);
void litenn_gguf_close(litenn_gguf* file);
unsigned litenn_gguf_version(const litenn_gguf* file);
size_t litenn_gguf_tensor_count(const litenn_gguf* file);
size_t litenn_gguf_metadata_count(const litenn_gguf* file);
int litenn_gguf_tensor_info(const litenn_gguf* file, size_t index, litenn_gguf_tensor* out);
int litenn_gguf_find_tensor(const litenn_gguf* file, const char* name, litenn_gguf_tensor* out);
const char* litenn_gguf_metadata_key(const litenn_gguf* file, size_t index);
/* ReadSizeValue / ReadDoubleValue / ReadStringValue / ReadBoolValue,
 * tools/gguf/GGUFImporter.cpp:66-147: any integer type for sizes (negative values refused),
 * any numeric type for doubles. */
int litenn_gguf_metadata_u64(const litenn_gguf* file, const char* key, uint64_t* out);
int litenn_gguf_metadata_f64(const litenn_gguf* file, const char* key, double* out);
int litenn_gguf_metadata_str(const litenn_gguf* file, const char* key, const char** out);
int litenn_gguf_metadata_bool(const litenn_gguf* file, const char* key, int* out);
int litenn_gguf_metadata_array(const litenn_gguf* file, const char* key, unsigned* elem_type, size_t* count);
/* Fills every field but kv_dtype; vocab_size comes from token_embd.weight
 * (tools/gguf/LLaMABuilder.cpp:685-703). */
int litenn_gguf_llama_params(const litenn_gguf* file, litenn_hip_llama_params* out);
/* Reads the file (.gguf or .ltnn), uploads the tensors of the decoder (token_embd, output_norm, optional output,
 * and per block attn_norm, attn_q/k/v/output, ffn_norm, ffn_gate/up/down: the names of
 * tools/gguf/LLaMABuilder.cpp:171-178,466-500) and returns a resident model that owns them.
 * context_length > 0 overrides the file's; kv_dtype is F16 or F32. */
int litenn_hip_llama_load_gguf(int dev, const char* path, int kv_dtype, int32_t context_length,
                               litenn_hip_llama** out);

#ifdef __cplusplus
}
#endif
#endif
