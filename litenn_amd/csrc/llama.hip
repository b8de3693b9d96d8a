// LLaMA decoder runtime on one GPU.
//
// The reference lowers a new static graph for every (sequenceLength, pastLength) pair and
// interprets it node by node, re-dequantising every weight to f32 each time
// (tools/gguf/LLaMABuilder.cpp:826-872, src/LiteNN/Runtime/Interpreter.h:89-104,325-329).
// Here the same operator sequence (LLaMABuilder.cpp:568-668,774-800) runs as a fixed list of
// kernel launches over weights that stay in their .gguf block layout in HBM, with a
// preallocated KV cache, the current length kept in device memory, and the single-token
// step captured once into a HIP graph so that a greedy loop never returns to the host.
#include "common.hpp"

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <exception>
#include <string>
#include <vector>

namespace litenn_hip
{
	int launch_gemv(int fmt, const void* wq, size_t n, size_t k, const float* x, size_t m, float* y,
	                const float* residual, hipStream_t stream);
	size_t gemm_scratch_halves(size_t m, size_t k);
	bool launch_gemm_group(int fmt, int count, const void* const* wq, const size_t* n, size_t k, const float* x,
	                       size_t m, float* const* y, const float* residual, const float* norm_w, double eps,
	                       const float* up, void* scratch_halves, float* partial, size_t partial_floats,
	                       hipStream_t stream);
	bool launch_gemm_gated(int fmt, const void* w_gate, const void* w_up, size_t n, size_t k, const float* x, size_t m,
	                       float* h, const float* norm_w, double eps, void* scratch_halves, hipStream_t stream);
	bool launch_gemm_group_mixed(const int* fmts, int count, const void* const* wq, const size_t* n, size_t k,
	                             const float* x, size_t m, float* const* y, const float* norm_w, double eps,
	                             void* scratch_halves, size_t scratch_capacity, hipStream_t stream);
	bool launch_gemm(int fmt, const void* wq, size_t n, size_t k, const float* x, size_t m, float* y,
	                 const float* residual, void* scratch_halves, float* partial, size_t partial_floats,
	                 hipStream_t stream);
	bool launch_linear_group(int fmt, int count, const void* const* w, float* const* y, const size_t* n, size_t k,
	                         const float* x, const float* residual, const float* norm_w, double eps, bool silu_mul,
	                         float* scratch_x, float* scratch_gate, float* scratch_up, hipStream_t stream);
	bool launch_gemv_fused_partials(int fmt, int count, const void* const* w, float* const* y, const size_t* n, size_t k,
	                                const float* x, const float* residual, const float* norm_w, double eps, bool silu_mul,
	                                const float* partials, size_t stride, bool on_x, bool plan_only, hipStream_t stream);
	bool launch_attn_block(const int* fmts, const void* const* wqkv, const size_t* n_qkv, int fmt_o, const void* wo,
	                       size_t d, const float* x, const float* norm_w, double eps, float* q, float* k, float* v,
	                       void* kcache, void* vcache, int cache_dtype, const float* cos_t, const float* sin_t,
	                       size_t rope_dims, const int* counters, int layer, size_t n_head, size_t n_kv_head,
	                       size_t head_dim, float* triples, unsigned* flags, float* y_partial, int* err, int spin_limit,
	                       bool plan_only, hipStream_t stream);
	bool launch_gemv_fused_mixed(const int* fmts, int count, const void* const* w, float* const* y, const size_t* n,
	                             size_t k, const float* x, const float* norm_w, double eps, hipStream_t stream);
	void launch_get_rows_q(int fmt, const void* table, size_t rows, size_t k, const int32_t* ids, size_t n_ids,
	                       float* out, int* err_flag, hipStream_t stream);
	void launch_rmsnorm(const float* x, const float* w, double eps, size_t m, size_t d, float* y, hipStream_t s);
	void launch_rope_qkv_append(float* q, const float* k, const float* v, void* kcache, void* vcache, int cache_dtype,
	                            const int* past_dev, size_t m, size_t n_head, size_t n_kv_head, size_t head_dim,
	                            size_t rope_dims, const float* cos_t, const float* sin_t, hipStream_t s);
	bool attn_step_fusable(const float* q, const float* k, const float* v, const void* kcache, const void* vcache,
	                       size_t head_dim, size_t rope_dims, const float* cos_t, const float* sin_t);
	void launch_attn_step(const float* q, const float* k, const float* v, void* kcache, void* vcache, int cache_dtype,
	                      const int* past_dev, size_t n_head, size_t n_kv_head, size_t head_dim, size_t rope_dims,
	                      const float* cos_t, const float* sin_t, float* out, size_t splits, float* partial,
	                      int* counters, hipStream_t s);
	size_t attn_splits(size_t m, size_t max_len, size_t n_head);
	size_t attn_partial_floats(size_t m, size_t n_head, size_t head_dim, size_t splits);
	bool launch_attn_tile(const float* q, const void* kcache, const void* vcache, int cache_dtype, size_t m,
	                      const int* past_dev, size_t past_host, size_t n_head, size_t n_kv_head, size_t head_dim,
	                      float* out, hipStream_t s);
	void launch_attn_decode(const float* q, const void* kcache, const void* vcache, int cache_dtype, size_t m,
	                        const int* past_dev, size_t past_host, size_t n_head, size_t n_kv_head, size_t head_dim,
	                        float* out, size_t splits, float* partial, int* counters, hipStream_t s);
	void launch_silu_mul(const float* gate, const float* up, float* y, size_t n, hipStream_t s);
	void launch_argmax(const float* x, size_t rows, size_t n, int32_t* out, hipStream_t s);
	size_t argmax_step_scratch_bytes(size_t n);
	void launch_argmax_step(const float* x, size_t n, void* scratch, int32_t* next, int* counters, int past_inc,
	                        int32_t* out, hipStream_t s);
	bool launch_convert(int src_dtype, const void* src, size_t n, int dst_dtype, void* dst, hipStream_t s);

	namespace
	{
		// counters[0] = past length, counters[1] = tokens emitted so far, counters[2] = steps this model
		// has run (never reset: it names a step in the values its workgroups hand to each other)
		__global__ void set_counters_kernel(int* counters, int past, int emitted)
		{
			counters[0] = past;
			counters[1] = emitted;
			counters[2] += 1;
		}

		struct Weight
		{
			int fmt = 0;
			const void* data = nullptr;
			size_t n = 0, k = 0;
		};

		struct Layer
		{
			Weight wq, wk, wv, wo, gate, up, down;
			const float* attn_norm = nullptr;
			const float* ffn_norm = nullptr;
			void* kcache = nullptr;
			void* vcache = nullptr;
		};
	} // namespace
} // namespace litenn_hip

using namespace litenn_hip;

struct litenn_hip_llama
{
	int dev = 0;
	litenn_hip_llama_params p{};
	int head_dim = 0;
	Weight tok_embd, output;
	const float* output_norm = nullptr;
	std::vector<Layer> layers;
	hipStream_t stream = nullptr;
	float* cos_t = nullptr; // [context_length, rope_dims/2]
	float* sin_t = nullptr;
	// activations for `cap_rows` rows
	size_t cap_rows = 0, cap_logit_rows = 0;
	float *x = nullptr, *xn = nullptr, *q = nullptr, *k = nullptr, *v = nullptr, *attn = nullptr, *gate = nullptr,
	      *gate2 = nullptr, *up = nullptr, *logits = nullptr;
	size_t xn_floats = 0; // what xn holds (rows x embedding_length, three times that for short prompts)
	void* xh = nullptr; // fp16 copy of a matmul's activations (multi-row path), 16-row padded
	size_t xh_halves = 0; // its size: room for the widest matmul, and for two copies of the embedding width
	void* argmax_scratch = nullptr; // per-chunk (value, index) pairs of the vocabulary arg-max
	std::vector<void*> owned; // device buffers freed with the model (tensors uploaded by the GGUF loader)
	int32_t* d_tokens = nullptr;
	int32_t* d_next = nullptr; // token produced by the last arg-max
	int32_t* d_out = nullptr;  // generated tokens
	size_t cap_out = 0;
	int* d_counters = nullptr; // {past, emitted, steps run}
	int* d_err = nullptr;
	// single-row attention: key chunks per head, their meeting place and arrival counters
	size_t attn_splits = 1;
	float* attn_partial = nullptr;
	int* attn_counters = nullptr;
	// The attention half of a block as one launch (launch_attn_block): 0 = not yet decided, 1 = every
	// block of this model takes it, -1 = it does not apply, or a wait inside it once ran out
	int block_fused = 0;
	float* blk_triples = nullptr;  // [head_count][8][132] chunk triples of the launch's second phase
	unsigned* blk_flags = nullptr; // [2][256] tags of the launch's two meetings
	float* blk_partial = nullptr; // [8][embedding_length] the launch's result, one vector per team
	int blk_spins = 8192;         // polls a wait inside the launch may take before it gives up
	int past = 0;
	hipGraphExec_t step_exec = nullptr;
	hipGraph_t step_graph = nullptr;
};

namespace
{
	const char* kAction = "HIP LLaMA";

	void free_scratch(litenn_hip_llama* m)
	{
		float** bufs[] = { &m->x, &m->xn, &m->q, &m->k, &m->v, &m->attn, &m->gate, &m->gate2, &m->up };
		for (float** b : bufs)
		{
			if (*b)
			{
				(void)hipFree(*b);
				*b = nullptr;
			}
		}
		if (m->d_tokens)
		{
			(void)hipFree(m->d_tokens);
			m->d_tokens = nullptr;
		}
		if (m->xh)
		{
			(void)hipFree(m->xh);
			m->xh = nullptr;
		}
		m->cap_rows = 0;
	}

	void drop_graph(litenn_hip_llama* m)
	{
		if (m->step_exec)
		{
			(void)hipGraphExecDestroy(m->step_exec);
			m->step_exec = nullptr;
		}
		if (m->step_graph)
		{
			(void)hipGraphDestroy(m->step_graph);
			m->step_graph = nullptr;
		}
	}

	int ensure_rows(litenn_hip_llama* m, size_t rows, size_t logit_rows)
	{
		const size_t d = m->p.embedding_length;
		const size_t qw = static_cast<size_t>(m->p.head_count) * m->head_dim;
		const size_t kvw = static_cast<size_t>(m->p.head_count_kv) * m->head_dim;
		const size_t ff = m->p.feed_forward_length;
		if (rows > m->cap_rows)
		{
			drop_graph(m); // the captured step references the old buffers
			free_scratch(m);
			// xn also takes the products of K's later ranges when a GEMM on few weight rows walks K in up to
			// four ranges at once: room for three, for prompts where that is used
			const size_t xn_width = rows <= 1024 ? 3 * d : d;
			m->xn_floats = rows * xn_width;
			struct { float** p; size_t n; } bufs[] = { { &m->x, d }, { &m->xn, xn_width }, { &m->q, qw }, { &m->k, kvw },
				                                        { &m->v, kvw }, { &m->attn, qw }, { &m->gate, ff }, { &m->gate2, ff },
				                                        { &m->up, ff } };
			for (auto& b : bufs)
			{
				LITENN_HIP_TRY(kAction, hipMalloc(reinterpret_cast<void**>(b.p), sizeof(float) * rows * b.n));
			}
			LITENN_HIP_TRY(kAction, hipMalloc(reinterpret_cast<void**>(&m->d_tokens), sizeof(int32_t) * rows));
			// (q/k/v projections in two formats share a launch that wants the rows in both fragment orders)
			m->xh_halves = std::max(gemm_scratch_halves(rows, std::max({ d, qw, ff })), 2 * gemm_scratch_halves(rows, d));
			LITENN_HIP_TRY(kAction, hipMalloc(&m->xh, 2 * m->xh_halves));
			m->cap_rows = rows;
		}
		if (logit_rows > m->cap_logit_rows)
		{
			drop_graph(m);
			if (m->logits)
			{
				(void)hipFree(m->logits);
				m->logits = nullptr;
			}
			LITENN_HIP_TRY(kAction, hipMalloc(reinterpret_cast<void**>(&m->logits),
			                                  sizeof(float) * logit_rows * static_cast<size_t>(m->p.vocab_size)));
			m->cap_logit_rows = logit_rows;
		}
		return 0;
	}

	int check_complete(const litenn_hip_llama* m)
	{
		if (!m->tok_embd.data || !m->output_norm)
		{
			return fail(kAction, "Missing GGUF tensor 'token_embd.weight' or 'output_norm.weight'");
		}
		for (const Layer& L : m->layers)
		{
			if (!L.wq.data || !L.wk.data || !L.wv.data || !L.wo.data || !L.gate.data || !L.up.data || !L.down.data ||
			    !L.attn_norm || !L.ffn_norm)
			{
				return fail(kAction, "Missing GGUF tensor in a decoder block");
			}
		}
		return 0;
	}

	// From this many rows on (and unless f32 operands are asked for) a matmul goes to the matrix cores:
	// one padded 16-row tile costs about as much as three single-row GEMVs.
	constexpr size_t kGemmMinRows = 4;
	// From this many rows on the prompt's attention runs tiled on the matrix cores.
	constexpr size_t kAttnTileMinRows = 16;

	// partial: null, or m->xn while it is idle (the GEMM may leave the products of K's later ranges there)
	void matmul(litenn_hip_llama* m, const Weight& w, const float* x, size_t rows, float* y, const float* residual,
	            float* partial, unsigned flags, hipStream_t s)
	{
		const bool quant = w.fmt != LITENN_FMT_F16 && w.fmt != LITENN_FMT_F32;
		if (rows >= kGemmMinRows && !(flags & LITENN_HIP_MATMUL_PRECISE) && quant && w.k % 256 == 0 &&
		    launch_gemm(w.fmt, w.data, w.n, w.k, x, rows, y, residual, m->xh, partial, partial ? m->xn_floats : 0, s))
		{
			return;
		}
		launch_gemv(w.fmt, w.data, w.n, w.k, x, rows, y, residual, s);
	}

	// Multi-row form of an operator group: y_i = X' . W_i^T (+ residual) with X' = x, RMSNorm(x) * norm_w
	// or silu(x) * up.  On the matrix cores the producer runs inside the fp16 pre-pass and matrices of
	// one format share a launch; otherwise it is composed from the stand-alone kernels (`tmp` takes
	// the producer's result).
	void matmul_group(litenn_hip_llama* m, int count, const Weight* const* ws, float* const* ys, const float* x,
	                  size_t rows, const float* residual, const float* norm_w, const float* up, float* tmp,
	                  float* partial, unsigned flags, hipStream_t s)
	{
		const Weight& w0 = *ws[0];
		bool same = true;
		for (int i = 1; i < count; ++i)
		{
			same = same && ws[i]->fmt == w0.fmt && ws[i]->k == w0.k;
		}
		const bool quant = w0.fmt != LITENN_FMT_F16 && w0.fmt != LITENN_FMT_F32;
		if (same && rows >= kGemmMinRows && !(flags & LITENN_HIP_MATMUL_PRECISE) && quant && w0.k % 256 == 0)
		{
			const void* w[3] = { nullptr, nullptr, nullptr };
			size_t n[3] = { 0, 0, 0 };
			for (int i = 0; i < count; ++i)
			{
				w[i] = ws[i]->data;
				n[i] = ws[i]->n;
			}
			if (launch_gemm_group(w0.fmt, count, w, n, w0.k, x, rows, ys, residual, norm_w, m->p.rms_norm_epsilon, up,
			                      m->xh, partial, partial ? m->xn_floats : 0, s))
			{
				return;
			}
		}
		const float* in = x;
		if (norm_w)
		{
			launch_rmsnorm(x, norm_w, m->p.rms_norm_epsilon, rows, w0.k, tmp, s);
			in = tmp;
		}
		else if (up)
		{
			launch_silu_mul(x, up, tmp, rows * w0.k, s);
			in = tmp;
		}
		for (int i = 0; i < count; ++i)
		{
			matmul(m, *ws[i], in, rows, ys[i], residual, nullptr, flags, s);
		}
	}

	// One operator group of the single-token step (see launch_linear_group).
	void group(litenn_hip_llama* m, int count, const Weight* const* ws, float* const* ys, const float* x,
	           const float* residual, const float* norm_w, bool silu_mul, hipStream_t s)
	{
		const void* w[3] = { nullptr, nullptr, nullptr };
		size_t n[3] = { 0, 0, 0 };
		for (int i = 0; i < count; ++i)
		{
			w[i] = ws[i]->data;
			n[i] = ws[i]->n;
		}
		// scratch used only when the fused kernel does not take the shape: xn for the normalised
		// activations, gate2 / up for the separate gate and up projections
		launch_linear_group(ws[0]->fmt, count, w, ys, n, ws[0]->k, x, residual, norm_w, m->p.rms_norm_epsilon, silu_mul,
		                    m->xn, m->gate2, m->up, s);
	}

	// the three launches of a block's single-token step when its attention half is one launch
	bool block_step(litenn_hip_llama* m, const Layer& L, int layer, bool plan_only, hipStream_t s)
	{
		const size_t d = m->p.embedding_length, ff = m->p.feed_forward_length;
		const int qkv_fmt[3] = { L.wq.fmt, L.wk.fmt, L.wv.fmt };
		const void* qkv_w[3] = { L.wq.data, L.wk.data, L.wv.data };
		const size_t qkv_n[3] = { L.wq.n, L.wk.n, L.wv.n };
		if (L.wq.k != d || L.wk.k != d || L.wv.k != d || L.wo.k != d || L.wo.n != d || L.gate.fmt != L.up.fmt ||
		    L.gate.k != d || L.up.k != d || L.gate.n != ff || L.up.n != ff || L.down.k != ff || L.down.n != d)
		{
			return false;
		}
		if (!launch_attn_block(qkv_fmt, qkv_w, qkv_n, L.wo.fmt, L.wo.data, d, m->x, L.attn_norm, m->p.rms_norm_epsilon, m->q,
		                       m->k, m->v, L.kcache, L.vcache, m->p.kv_dtype, m->cos_t, m->sin_t,
		                       static_cast<size_t>(m->p.rope_dimension_count), m->d_counters, layer, m->p.head_count,
		                       m->p.head_count_kv, m->head_dim, m->blk_triples, m->blk_flags, m->blk_partial, m->d_err,
		                       m->blk_spins, plan_only, s))
		{
			return false;
		}
		// gate = silu(x' . Wg) * (x' . Wu) with x' = RMSNorm(x + the eight partial vectors)
		const void* gu_w[2] = { L.gate.data, L.up.data };
		const size_t gu_n[2] = { L.gate.n, L.up.n };
		float* gu_y[2] = { m->gate, nullptr };
		if (!launch_gemv_fused_partials(L.gate.fmt, 2, gu_w, gu_y, gu_n, d, m->x, nullptr, L.ffn_norm, m->p.rms_norm_epsilon,
		                                true, m->blk_partial, d, true, plan_only, s))
		{
			return false;
		}
		// x = (x + the eight partial vectors) + mlp
		const void* dn_w[1] = { L.down.data };
		const size_t dn_n[1] = { L.down.n };
		float* dn_y[1] = { m->x };
		return launch_gemv_fused_partials(L.down.fmt, 1, dn_w, dn_y, dn_n, ff, m->gate, m->x, nullptr, 0.0, false,
		                                  m->blk_partial, d, false, plan_only, s);
	}

	// Decides once per model (and again after a tensor changed) whether its blocks take that form, and
	// allocates what the launch needs.
	bool block_fused_ready(litenn_hip_llama* m)
	{
		if (m->block_fused != 0)
		{
			return m->block_fused > 0;
		}
		m->block_fused = -1;
		// LITENN_HIP_ATTN_BLOCK=0 keeps the separate launches; LITENN_HIP_ATTN_BLOCK_SPINS bounds the
		// launch's waits (read when the model's step is decided, not per launch)
		const char* off = getenv("LITENN_HIP_ATTN_BLOCK");
		if (off && off[0] == '0')
		{
			return false;
		}
		if (const char* spins = getenv("LITENN_HIP_ATTN_BLOCK_SPINS"))
		{
			m->blk_spins = std::max(0, atoi(spins));
		}
		const size_t d = m->p.embedding_length;
		if (!m->blk_partial)
		{
			// flags start at 0, which no launch's tag equals
			const size_t triples = sizeof(float) * static_cast<size_t>(m->p.head_count) * 8 * 132;
			if (hipMalloc(reinterpret_cast<void**>(&m->blk_triples), triples) != hipSuccess ||
			    hipMalloc(reinterpret_cast<void**>(&m->blk_flags), sizeof(unsigned) * 512) != hipSuccess ||
			    hipMalloc(reinterpret_cast<void**>(&m->blk_partial), sizeof(float) * 8 * d) != hipSuccess ||
			    hipMemsetAsync(m->blk_flags, 0, sizeof(unsigned) * 512, m->stream) != hipSuccess ||
			    hipStreamSynchronize(m->stream) != hipSuccess)
			{
				(void)hipGetLastError();
				return false;
			}
		}
		for (size_t i = 0; i < m->layers.size(); ++i)
		{
			if (!block_step(m, m->layers[i], static_cast<int>(i), true, m->stream))
			{
				return false;
			}
		}
		m->block_fused = 1;
		return true;
	}

	// The single-token step: six fused launches per decoder block
	//   [RMSNorm + q/k/v] [RoPE + cache append] [attention] [o + residual] [RMSNorm + gate/up + SwiGLU]
	//   [down + residual]
	// (matrices of different formats cannot share a launch and go out one by one).
	void forward_token(litenn_hip_llama* m, const int32_t* ids)
	{
		hipStream_t s = m->stream;
		const size_t d = m->p.embedding_length;
		const size_t H = m->p.head_count, KH = m->p.head_count_kv, hd = m->head_dim;
		const int* past_dev = m->d_counters;
		launch_get_rows_q(m->tok_embd.fmt, m->tok_embd.data, m->tok_embd.n, d, ids, 1, m->x, m->d_err, s);
		// three launches per block where the attention half is one launch (block_step), else five;
		// decided (and its buffers allocated) by the entry points before anything is queued or captured
		const bool fused_blocks = m->block_fused > 0;
		for (Layer& L : m->layers)
		{
			if (fused_blocks && block_step(m, L, static_cast<int>(&L - m->layers.data()), false, s))
			{
				continue;
			}
			const Weight* qkv[3] = { &L.wq, &L.wk, &L.wv };
			float* qkv_out[3] = { m->q, m->k, m->v };
			// one launch when the three share a format or are one of the two-format mixes the GEMV
			// takes (q/k in Q4_K or Q5_K beside a Q6_K v); otherwise one per run of equal formats
			const int qkv_fmt[3] = { L.wq.fmt, L.wk.fmt, L.wv.fmt };
			const void* qkv_w[3] = { L.wq.data, L.wk.data, L.wv.data };
			const size_t qkv_n[3] = { L.wq.n, L.wk.n, L.wv.n };
			const bool mixed = L.wq.fmt != L.wk.fmt || L.wk.fmt != L.wv.fmt;
			if (!(mixed && L.wq.k == L.wk.k && L.wk.k == L.wv.k &&
			      launch_gemv_fused_mixed(qkv_fmt, 3, qkv_w, qkv_out, qkv_n, L.wq.k, m->x, L.attn_norm,
			                              m->p.rms_norm_epsilon, s)))
			{
				for (int i = 0; i < 3;)
				{
					int j = i + 1;
					while (j < 3 && qkv[j]->fmt == qkv[i]->fmt)
					{
						++j;
					}
					group(m, j - i, qkv + i, qkv_out + i, m->x, nullptr, L.attn_norm, false, s);
					i = j;
				}
			}
			const size_t rope_dims = m->p.rope_dimension_count;
			if (attn_step_fusable(m->q, m->k, m->v, L.kcache, L.vcache, hd, rope_dims, m->cos_t, m->sin_t))
			{
				launch_attn_step(m->q, m->k, m->v, L.kcache, L.vcache, m->p.kv_dtype, past_dev, H, KH, hd, rope_dims,
				                 m->cos_t, m->sin_t, m->attn, m->attn_splits, m->attn_partial, m->attn_counters, s);
			}
			else
			{
				launch_rope_qkv_append(m->q, m->k, m->v, L.kcache, L.vcache, m->p.kv_dtype, past_dev, 1, H, KH, hd,
				                       rope_dims, m->cos_t, m->sin_t, s);
				launch_attn_decode(m->q, L.kcache, L.vcache, m->p.kv_dtype, 1, past_dev, 0, H, KH, hd, m->attn,
				                   m->attn_splits, m->attn_partial, m->attn_counters, s);
			}
			const Weight* wo[1] = { &L.wo };
			float* xo[1] = { m->x };
			group(m, 1, wo, xo, m->attn, m->x, nullptr, false, s); // x = x + attn . Wo
			if (L.gate.fmt == L.up.fmt)
			{
				const Weight* gu[2] = { &L.gate, &L.up };
				float* h[1] = { m->gate };
				group(m, 2, gu, h, m->x, nullptr, L.ffn_norm, true, s); // gate = silu(x'.Wg) * (x'.Wu)
			}
			else
			{
				const Weight* wg[1] = { &L.gate };
				const Weight* wu[1] = { &L.up };
				float* og[1] = { m->gate };
				float* ou[1] = { m->up };
				group(m, 1, wg, og, m->x, nullptr, L.ffn_norm, false, s);
				group(m, 1, wu, ou, m->x, nullptr, L.ffn_norm, false, s);
				launch_silu_mul(m->gate, m->up, m->gate, m->p.feed_forward_length, s);
			}
			const Weight* wd[1] = { &L.down };
			group(m, 1, wd, xo, m->gate, m->x, nullptr, false, s); // x = x + mlp
		}
		const Weight* head[1] = { m->output.data ? &m->output : &m->tok_embd };
		float* lg[1] = { m->logits };
		group(m, 1, head, lg, m->x, nullptr, m->output_norm, false, s);
	}

	// Enqueues the decoder over `rows` tokens whose ids are at `ids` (device); positions start at
	// counters[0].  Logits are produced for the last `logit_rows` rows into m->logits.
	void forward(litenn_hip_llama* m, const int32_t* ids, size_t rows, size_t logit_rows, unsigned flags)
	{
		static const bool fuse_token = !(getenv("LITENN_HIP_FUSE") && getenv("LITENN_HIP_FUSE")[0] == '0');
		if (rows == 1 && logit_rows == 1 && fuse_token)
		{
			forward_token(m, ids);
			return;
		}
		hipStream_t s = m->stream;
		const size_t d = m->p.embedding_length;
		const size_t H = m->p.head_count, KH = m->p.head_count_kv, hd = m->head_dim;
		const int* past_dev = m->d_counters;
		launch_get_rows_q(m->tok_embd.fmt, m->tok_embd.data, m->tok_embd.n, d, ids, rows, m->x, m->d_err, s);
		for (Layer& L : m->layers)
		{
			const Weight* qkv[3] = { &L.wq, &L.wk, &L.wv };
			float* qkv_out[3] = { m->q, m->k, m->v };
			// consecutive projections of one format share a launch (and its fused norm), and so do q and
			// k in Q4_K or Q5_K beside a Q6_K v
			const int qkv_fmt[3] = { L.wq.fmt, L.wk.fmt, L.wv.fmt };
			const void* qkv_w[3] = { L.wq.data, L.wk.data, L.wv.data };
			const size_t qkv_n[3] = { L.wq.n, L.wk.n, L.wv.n };
			const bool mixed = L.wq.fmt != L.wk.fmt || L.wk.fmt != L.wv.fmt;
			const bool one_launch = mixed && rows >= kGemmMinRows && !(flags & LITENN_HIP_MATMUL_PRECISE) &&
			                        L.wq.k == L.wk.k && L.wk.k == L.wv.k &&
			                        launch_gemm_group_mixed(qkv_fmt, 3, qkv_w, qkv_n, L.wq.k, m->x, rows, qkv_out, L.attn_norm,
			                                                m->p.rms_norm_epsilon, m->xh, m->xh_halves, s);
			for (int i = 0; i < 3 && !one_launch;)
			{
				int j = i + 1;
				while (j < 3 && qkv[j]->fmt == qkv[i]->fmt && qkv[j]->k == qkv[i]->k)
				{
					++j;
				}
				matmul_group(m, j - i, qkv + i, qkv_out + i, m->x, rows, nullptr, L.attn_norm, nullptr, m->xn, nullptr,
				             flags, s);
				i = j;
			}
			launch_rope_qkv_append(m->q, m->k, m->v, L.kcache, L.vcache, m->p.kv_dtype, past_dev, rows, H, KH, hd,
			                       m->p.rope_dimension_count, m->cos_t, m->sin_t, s);
			// a prompt's rows go through the matrix cores (fp16 operands) unless f32 operands are asked for
			if (rows < kAttnTileMinRows || (flags & LITENN_HIP_MATMUL_PRECISE) ||
			    !launch_attn_tile(m->q, L.kcache, L.vcache, m->p.kv_dtype, rows, past_dev, 0, H, KH, hd, m->attn, s))
			{
				launch_attn_decode(m->q, L.kcache, L.vcache, m->p.kv_dtype, rows, past_dev, 0, H, KH, hd, m->attn,
				                   rows == 1 ? m->attn_splits : 1, m->attn_partial, m->attn_counters, s);
			}
			matmul(m, L.wo, m->attn, rows, m->x, m->x, m->xn, flags, s); // x = x + attn . Wo (xn is idle here)
			const Weight* gu[2] = { &L.gate, &L.up };
			float* gu_out[2] = { m->gate, m->up };
			// gate = silu(x' . Wg) * (x' . Wu) straight from the launch's epilogue where the shape allows,
			// else the two projections, whose product the down projection's pre-pass then forms
			const bool gated = rows >= kGemmMinRows && !(flags & LITENN_HIP_MATMUL_PRECISE) && L.gate.fmt == L.up.fmt &&
			                   L.gate.k == L.up.k && L.gate.n == L.up.n &&
			                   launch_gemm_gated(L.gate.fmt, L.gate.data, L.up.data, L.gate.n, L.gate.k, m->x, rows, m->gate,
			                                     L.ffn_norm, m->p.rms_norm_epsilon, m->xh, s);
			if (!gated)
			{
				matmul_group(m, 2, gu, gu_out, m->x, rows, nullptr, L.ffn_norm, nullptr, m->xn, nullptr, flags, s);
			}
			const Weight* wd[1] = { &L.down };
			float* xo[1] = { m->x };
			// xn is idle here: the GEMM may leave the product of K's second half there
			matmul_group(m, 1, wd, xo, m->gate, rows, m->x, nullptr, gated ? nullptr : m->up, m->gate2, m->xn, flags,
			             s); // x = x + mlp
		}
		const size_t first = rows - logit_rows;
		launch_rmsnorm(m->x + first * d, m->output_norm, m->p.rms_norm_epsilon, logit_rows, d, m->xn, s);
		const Weight& head = m->output.data ? m->output : m->tok_embd;
		matmul(m, head, m->xn, logit_rows, m->logits, nullptr, nullptr, flags, s);
	}

	constexpr int kBlockWaitRanOut = -2;

	int check_error_flag(litenn_hip_llama* m)
	{
		int flag = 0;
		LITENN_HIP_TRY(kAction, hipMemcpyAsync(&flag, m->d_err, sizeof(int), hipMemcpyDeviceToHost, m->stream));
		LITENN_HIP_TRY(kAction, hipStreamSynchronize(m->stream));
		if (flag)
		{
			const int zero = 0;
			(void)hipMemcpy(m->d_err, &zero, sizeof(int), hipMemcpyHostToDevice);
			if (flag & 2)
			{
				return kBlockWaitRanOut;
			}
			return fail(kAction, "GetRows index out of range");
		}
		return 0;
	}

	// A wait inside the one-launch attention half ran out (its workgroups were not all running at
	// once: the card was shared, or is not the one the launch is shaped for).  What that step
	// computed is void; the model takes the separate launches from now on and the caller repeats
	// the step.  The flags the launch left behind are never read again.
	void give_up_block_launch(litenn_hip_llama* m)
	{
		m->block_fused = -1;
		drop_graph(m);
	}
} // namespace

namespace
{
	int llama_create_impl(int dev, const litenn_hip_llama_params* params, litenn_hip_llama** out, litenn_hip_llama*& m);
}

extern "C" int litenn_hip_llama_create(int dev, const litenn_hip_llama_params* params, litenn_hip_llama** out)
{
	// host containers sized by the caller's context length live in the body: an allocation that
	// fails there must come back as a status, not leave through the C boundary
	litenn_hip_llama* m = nullptr;
	try
	{
		return llama_create_impl(dev, params, out, m);
	}
	catch (const std::exception& ex)
	{
		if (m)
		{
			litenn_hip_llama_free(m);
		}
		return fail(kAction, std::string("host memory for the model's tables: ") + ex.what());
	}
}

namespace
{
int llama_create_impl(int dev, const litenn_hip_llama_params* params, litenn_hip_llama** out, litenn_hip_llama*& m)
{
	if (!params || !out)
	{
		return fail(kAction, "null argument");
	}
	const litenn_hip_llama_params& p = *params;
	// the checks of ParseLLaMAHyperparameters (tools/gguf/GGUFImporter.cpp:603-640)
	if (p.context_length <= 0 || p.embedding_length <= 0 || p.block_count <= 0 || p.feed_forward_length <= 0 ||
	    p.vocab_size <= 0)
	{
		return fail(kAction, "LLaMA hyperparameters must be greater than zero");
	}
	if (p.head_count <= 0 || p.head_count_kv <= 0 || p.embedding_length % p.head_count != 0 ||
	    p.head_count % p.head_count_kv != 0)
	{
		return fail(kAction, "LLaMA head counts must divide the embedding length and each other");
	}
	if (!(p.rms_norm_epsilon > 0.0))
	{
		return fail(kAction, "LLaMA attention.layer_norm_rms_epsilon must be greater than zero");
	}
	if (!(p.rope_freq_base > 0.0) || !(p.rope_freq_scale > 0.0))
	{
		return fail(kAction, "LLaMA rope.freq_base and rope.freq_scale must be greater than zero");
	}
	const int head_dim = p.embedding_length / p.head_count;
	int rope_dims = p.rope_dimension_count == 0 ? head_dim : p.rope_dimension_count;
	if (rope_dims > head_dim || rope_dims % 2 != 0 || rope_dims < 0)
	{
		return fail(kAction, "LLaMA rope.dimension_count must be an even value in [2, headDim]");
	}
	if (head_dim > 256 || head_dim % 2 != 0)
	{
		return fail(kAction, "head dimension must be even and at most 256");
	}
	// The attention kernels keep no per-key storage (online softmax), so the context is bounded only
	// by the 2^30 positions their int arithmetic takes and by the memory the caches need (an
	// allocation failure below reports that).
	if (p.context_length > (1 << 30))
	{
		return fail(kAction, "context length exceeds 2^30 positions");
	}
	if (p.kv_dtype != LITENN_F16 && p.kv_dtype != LITENN_F32)
	{
		return fail(kAction, "KV cache dtype must be Float16 or Float32");
	}
	DeviceGuard guard(dev);
	if (!guard.ok())
	{
		return fail_hip(kAction, guard.error());
	}
	m = new litenn_hip_llama();
	m->dev = dev;
	m->p = p;
	m->p.rope_dimension_count = rope_dims;
	m->head_dim = head_dim;
	m->layers.resize(static_cast<size_t>(p.block_count));
	auto bail = [&](hipError_t e) {
		litenn_hip_llama_free(m);
		m = nullptr;
		return fail_hip(kAction, e);
	};
	// Non-blocking: a stream that synchronises with the legacy default stream would, while its
	// decode step is being captured, make every default-stream call of another host thread fail
	// ("would make the legacy stream depend on a capturing blocking stream").
	hipError_t e = hipStreamCreateWithFlags(&m->stream, hipStreamNonBlocking);
	if (e != hipSuccess)
	{
		m->stream = nullptr;
		return bail(e);
	}
	const size_t kv_bytes = static_cast<size_t>(p.context_length) * p.head_count_kv * head_dim * dtype_size(p.kv_dtype);
	for (Layer& L : m->layers)
	{
		if ((e = hipMalloc(&L.kcache, kv_bytes)) != hipSuccess || (e = hipMalloc(&L.vcache, kv_bytes)) != hipSuccess)
		{
			return bail(e);
		}
	}
	// angle tables in f64 on the host, stored as f32: MakeRoPEAngleTable (Layer/RoPE.h:24-41)
	const size_t half = static_cast<size_t>(rope_dims) / 2;
	if (half)
	{
		std::vector<float> c(static_cast<size_t>(p.context_length) * half), s(c.size());
		std::vector<double> inv_freqs(half);
		for (size_t dim = 0; dim < half; ++dim)
		{
			const double exponent = -2.0 * static_cast<double>(dim) / static_cast<double>(half * 2);
			inv_freqs[dim] = std::pow(p.rope_freq_base, exponent);
		}
		for (size_t pos = 0; pos < static_cast<size_t>(p.context_length); ++pos)
		{
			for (size_t dim = 0; dim < half; ++dim)
			{
				const double inv_freq = inv_freqs[dim];
				const double angle = static_cast<double>(pos) * inv_freq * p.rope_freq_scale;
				c[pos * half + dim] = static_cast<float>(std::cos(angle));
				s[pos * half + dim] = static_cast<float>(std::sin(angle));
			}
		}
		if ((e = hipMalloc(reinterpret_cast<void**>(&m->cos_t), sizeof(float) * c.size())) != hipSuccess ||
		    (e = hipMalloc(reinterpret_cast<void**>(&m->sin_t), sizeof(float) * c.size())) != hipSuccess ||
		    (e = hipMemcpy(m->cos_t, c.data(), sizeof(float) * c.size(), hipMemcpyHostToDevice)) != hipSuccess ||
		    (e = hipMemcpy(m->sin_t, s.data(), sizeof(float) * s.size(), hipMemcpyHostToDevice)) != hipSuccess)
		{
			return bail(e);
		}
	}
	if ((e = hipMalloc(reinterpret_cast<void**>(&m->d_counters), 4 * sizeof(int))) != hipSuccess ||
	    (e = hipMalloc(reinterpret_cast<void**>(&m->d_err), sizeof(int))) != hipSuccess ||
	    (e = hipMalloc(reinterpret_cast<void**>(&m->d_next), sizeof(int32_t))) != hipSuccess ||
	    (e = hipMemsetAsync(m->d_counters, 0, 4 * sizeof(int), m->stream)) != hipSuccess ||
	    (e = hipMemsetAsync(m->d_err, 0, sizeof(int), m->stream)) != hipSuccess ||
	    (e = hipMemsetAsync(m->d_next, 0, sizeof(int32_t), m->stream)) != hipSuccess)
	{
		return bail(e);
	}
	if ((e = hipMalloc(&m->argmax_scratch, argmax_step_scratch_bytes(static_cast<size_t>(p.vocab_size)))) != hipSuccess)
	{
		return bail(e);
	}
	m->attn_splits = attn_splits(1, static_cast<size_t>(p.context_length), static_cast<size_t>(p.head_count));
	if (m->attn_splits > 1)
	{
		const size_t heads = static_cast<size_t>(p.head_count);
		const size_t floats = attn_partial_floats(1, heads, static_cast<size_t>(head_dim), m->attn_splits);
		if ((e = hipMalloc(reinterpret_cast<void**>(&m->attn_partial), sizeof(float) * floats)) != hipSuccess ||
		    (e = hipMalloc(reinterpret_cast<void**>(&m->attn_counters), sizeof(int) * heads)) != hipSuccess ||
		    (e = hipMemsetAsync(m->attn_counters, 0, sizeof(int) * heads, m->stream)) != hipSuccess)
		{
			return bail(e);
		}
	}
	*out = m;
	return 0;
}
} // namespace

// Hands a device allocation to the model: it is released by litenn_hip_llama_free.  Used by
// the GGUF loader; not part of the C ABI.
namespace litenn_hip
{
	int llama_adopt(litenn_hip_llama* m, void* device_ptr)
	{
		if (!m || !device_ptr)
		{
			return fail(kAction, "null argument");
		}
		m->owned.push_back(device_ptr);
		return 0;
	}
} // namespace litenn_hip

extern "C" int litenn_hip_llama_free(litenn_hip_llama* m)
{
	if (!m)
	{
		return 0;
	}
	DeviceGuard guard(m->dev);
	if (m->stream)
	{
		(void)hipStreamSynchronize(m->stream);
	}
	drop_graph(m);
	free_scratch(m);
	for (void* p : { static_cast<void*>(m->blk_triples), static_cast<void*>(m->blk_flags), static_cast<void*>(m->blk_partial) })
	{
		if (p)
		{
			(void)hipFree(p);
		}
	}
	for (Layer& L : m->layers)
	{
		if (L.kcache)
		{
			(void)hipFree(L.kcache);
		}
		if (L.vcache)
		{
			(void)hipFree(L.vcache);
		}
	}
	for (void* ptr : m->owned)
	{
		(void)hipFree(ptr);
	}
	void* singles[] = { m->cos_t, m->sin_t,      m->logits,       m->d_next,       m->d_out,
	                    m->d_counters, m->d_err, m->attn_partial, m->attn_counters,
	                    m->argmax_scratch };
	for (void* ptr : singles)
	{
		if (ptr)
		{
			(void)hipFree(ptr);
		}
	}
	if (m->stream)
	{
		(void)hipStreamDestroy(m->stream);
	}
	delete m;
	return 0;
}

extern "C" int litenn_hip_llama_set_tensor(litenn_hip_llama* m, int which, int layer, int fmt, const void* data,
                                           size_t n, size_t k)
{
	if (!m || !data)
	{
		return fail(kAction, "null argument");
	}
	const size_t d = m->p.embedding_length, hd = m->head_dim;
	const size_t qw = m->p.head_count * hd, kvw = m->p.head_count_kv * hd, ff = m->p.feed_forward_length;
	const size_t vocab = m->p.vocab_size;
	const bool per_layer = which >= LITENN_T_ATTN_Q && which != LITENN_T_OUTPUT_NORM;
	if (per_layer && (layer < 0 || layer >= m->p.block_count))
	{
		return fail(kAction, "layer index out of range");
	}
	Layer* L = per_layer ? &m->layers[static_cast<size_t>(layer)] : nullptr;
	Weight* target = nullptr;
	size_t want_n = 0, want_k = 0;
	switch (which)
	{
	case LITENN_T_TOKEN_EMBD: target = &m->tok_embd; want_n = vocab; want_k = d; break;
	case LITENN_T_OUTPUT: target = &m->output; want_n = vocab; want_k = d; break;
	case LITENN_T_ATTN_Q: target = &L->wq; want_n = qw; want_k = d; break;
	case LITENN_T_ATTN_K: target = &L->wk; want_n = kvw; want_k = d; break;
	case LITENN_T_ATTN_V: target = &L->wv; want_n = kvw; want_k = d; break;
	case LITENN_T_ATTN_OUTPUT: target = &L->wo; want_n = d; want_k = qw; break;
	case LITENN_T_FFN_GATE: target = &L->gate; want_n = ff; want_k = d; break;
	case LITENN_T_FFN_UP: target = &L->up; want_n = ff; want_k = d; break;
	case LITENN_T_FFN_DOWN: target = &L->down; want_n = d; want_k = ff; break;
	case LITENN_T_OUTPUT_NORM:
	case LITENN_T_ATTN_NORM:
	case LITENN_T_FFN_NORM:
		if (fmt != LITENN_FMT_F32 || n * k != d)
		{
			return fail(kAction, "norm weight must be Float32 with shape [embedding_length] or [1, embedding_length]");
		}
		if (which == LITENN_T_OUTPUT_NORM)
		{
			m->output_norm = static_cast<const float*>(data);
		}
		else if (which == LITENN_T_ATTN_NORM)
		{
			L->attn_norm = static_cast<const float*>(data);
		}
		else
		{
			L->ffn_norm = static_cast<const float*>(data);
		}
		drop_graph(m);
		return 0;
	default:
		return fail(kAction, "unknown tensor id");
	}
	if (n != want_n || k != want_k)
	{
		return fail(kAction, "tensor shape does not match the hyper-parameters");
	}
	if (row_bytes(fmt, k) == 0)
	{
		return fail(kAction, "unsupported block format or row width");
	}
	target->fmt = fmt;
	target->data = data;
	target->n = n;
	target->k = k;
	drop_graph(m);
	m->block_fused = 0; // decided again with the new tensor
	return 0;
}

extern "C" int litenn_hip_llama_reset(litenn_hip_llama* m)
{
	if (!m)
	{
		return fail(kAction, "null argument");
	}
	m->past = 0;
	return 0;
}

extern "C" int litenn_hip_llama_past(const litenn_hip_llama* m)
{
	return m ? m->past : -1;
}

extern "C" int litenn_hip_llama_block_form(const litenn_hip_llama* m)
{
	return m ? m->block_fused : 0;
}

extern "C" int litenn_hip_llama_eval(litenn_hip_llama* m, const int32_t* tokens, size_t rows, float* logits,
                                     float* last_logits, unsigned flags)
{
	if (!m || !tokens)
	{
		return fail(kAction, "null argument");
	}
	if (rows == 0)
	{
		return fail(kAction, "sequence length must be positive");
	}
	if (static_cast<size_t>(m->past) + rows > static_cast<size_t>(m->p.context_length))
	{
		return fail(kAction, "context length exceeded");
	}
	if (check_complete(m) != 0)
	{
		return 1;
	}
	for (size_t i = 0; i < rows; ++i)
	{
		if (tokens[i] < 0 || tokens[i] >= m->p.vocab_size)
		{
			return fail(kAction, "GetRows index out of range"); // Device.h:868-871
		}
	}
	DeviceGuard guard(m->dev);
	if (!guard.ok())
	{
		return fail_hip(kAction, guard.error());
	}
	const size_t logit_rows = logits ? rows : 1;
	if (ensure_rows(m, rows, logit_rows) != 0)
	{
		return 1;
	}
	(void)block_fused_ready(m);
	hipStream_t s = m->stream;
	for (int attempt = 0;; ++attempt)
	{
		LITENN_HIP_TRY(kAction, hipMemcpyAsync(m->d_tokens, tokens, sizeof(int32_t) * rows, hipMemcpyHostToDevice, s));
		set_counters_kernel<<<1, 1, 0, s>>>(m->d_counters, m->past, 0);
		forward(m, m->d_tokens, rows, logit_rows, flags);
		LITENN_HIP_TRY(kAction, hipGetLastError());
		const size_t vocab = m->p.vocab_size;
		if (logits)
		{
			LITENN_HIP_TRY(kAction, hipMemcpyAsync(logits, m->logits, sizeof(float) * rows * vocab, hipMemcpyDeviceToHost, s));
		}
		if (last_logits)
		{
			LITENN_HIP_TRY(kAction, hipMemcpyAsync(last_logits, m->logits + (logit_rows - 1) * vocab, sizeof(float) * vocab,
			                                       hipMemcpyDeviceToHost, s));
		}
		const int rc = check_error_flag(m);
		if (rc == kBlockWaitRanOut && attempt == 0)
		{
			give_up_block_launch(m); // and once more through the separate launches
			continue;
		}
		if (rc != 0)
		{
			return rc == kBlockWaitRanOut ? fail(kAction, "a wait inside the decoder step ran out") : 1;
		}
		break;
	}
	m->past += static_cast<int>(rows);
	return 0;
}

extern "C" int litenn_hip_llama_generate(litenn_hip_llama* m, const int32_t* prompt, size_t n_prompt, size_t n_new,
                                         int32_t* out_tokens, unsigned flags, double* prefill_ms, double* decode_ms)
{
	if (!m || !prompt || !out_tokens)
	{
		return fail(kAction, "null argument");
	}
	if (n_prompt == 0 || n_new == 0)
	{
		return fail(kAction, "prompt and generation lengths must be positive");
	}
	if (static_cast<size_t>(m->past) + n_prompt + n_new - 1 > static_cast<size_t>(m->p.context_length))
	{
		return fail(kAction, "context length exceeded");
	}
	if (check_complete(m) != 0)
	{
		return 1;
	}
	for (size_t i = 0; i < n_prompt; ++i)
	{
		if (prompt[i] < 0 || prompt[i] >= m->p.vocab_size)
		{
			return fail(kAction, "GetRows index out of range");
		}
	}
	DeviceGuard guard(m->dev);
	if (!guard.ok())
	{
		return fail_hip(kAction, guard.error());
	}
	if (ensure_rows(m, n_prompt, 1) != 0)
	{
		return 1;
	}
	(void)block_fused_ready(m);
	if (n_new > m->cap_out)
	{
		drop_graph(m);
		if (m->d_out)
		{
			(void)hipFree(m->d_out);
			m->d_out = nullptr;
		}
		LITENN_HIP_TRY(kAction, hipMalloc(reinterpret_cast<void**>(&m->d_out), sizeof(int32_t) * n_new));
		m->cap_out = n_new;
	}
	hipStream_t s = m->stream;
	// the events exist before any work is queued and are destroyed on every way out
	hipEvent_t ev[3] = { nullptr, nullptr, nullptr };
	auto cleanup = [&]() {
		for (hipEvent_t& e : ev)
		{
			if (e)
			{
				(void)hipEventDestroy(e);
				e = nullptr;
			}
		}
	};
	for (hipEvent_t& e : ev)
	{
		const hipError_t ce = hipEventCreate(&e);
		if (ce != hipSuccess)
		{
			e = nullptr;
			cleanup();
			return fail_hip(kAction, ce);
		}
	}
	int rc = 0;
	// A failure part-way leaves `past` as it was: the rows a failed run appended lie beyond it, are
	// never read (every pass takes its position from `past`) and are overwritten by the next call.
	// The stream is drained first so that nothing of the failed run is still in flight afterwards.
#define GEN_TRY(expr)                                                                                                  \
	do                                                                                                                 \
	{                                                                                                                  \
		const hipError_t e_ = (expr);                                                                                  \
		if (e_ != hipSuccess)                                                                                          \
		{                                                                                                              \
			(void)hipStreamSynchronize(s);                                                                             \
			cleanup();                                                                                                 \
			return fail_hip(kAction, e_);                                                                              \
		}                                                                                                              \
	} while (0)

	// prompt: one pass over n_prompt rows, logits of the last row only, first token from its arg-max
	GEN_TRY(hipMemcpyAsync(m->d_tokens, prompt, sizeof(int32_t) * n_prompt, hipMemcpyHostToDevice, s));
	set_counters_kernel<<<1, 1, 0, s>>>(m->d_counters, m->past, 0);
	GEN_TRY(hipEventRecord(ev[0], s));
	forward(m, m->d_tokens, n_prompt, 1, flags);
	launch_argmax_step(m->logits, m->p.vocab_size, m->argmax_scratch, m->d_next, m->d_counters,
	                   static_cast<int>(n_prompt), m->d_out, s);
	GEN_TRY(hipEventRecord(ev[1], s));
	GEN_TRY(hipGetLastError());

	// single-token steps: embed d_next at position counters[0], arg-max, append.  The step is
	// captured once; every replay reads its position from device memory.
	const char* graph_env = getenv("LITENN_HIP_GRAPH");
	const bool use_graph = !(graph_env && graph_env[0] == '0');
	if (n_new > 1)
	{
		if (use_graph && !m->step_exec)
		{
			GEN_TRY(hipStreamSynchronize(s));
			hipError_t ce = hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal);
			if (ce == hipSuccess)
			{
				forward(m, m->d_next, 1, 1, flags);
				launch_argmax_step(m->logits, m->p.vocab_size, m->argmax_scratch, m->d_next, m->d_counters, 1, m->d_out, s);
				ce = hipStreamEndCapture(s, &m->step_graph);
			}
			if (ce == hipSuccess)
			{
				ce = hipGraphInstantiate(&m->step_exec, m->step_graph, nullptr, nullptr, 0);
			}
			if (ce != hipSuccess)
			{
				drop_graph(m);
				cleanup();
				return fail_hip(kAction, ce);
			}
		}
		for (size_t i = 1; i < n_new; ++i)
		{
			if (use_graph)
			{
				GEN_TRY(hipGraphLaunch(m->step_exec, s));
			}
			else
			{
				forward(m, m->d_next, 1, 1, flags);
				launch_argmax_step(m->logits, m->p.vocab_size, m->argmax_scratch, m->d_next, m->d_counters, 1, m->d_out, s);
			}
		}
	}
	GEN_TRY(hipEventRecord(ev[2], s));
	GEN_TRY(hipGetLastError());
	GEN_TRY(hipMemcpyAsync(out_tokens, m->d_out, sizeof(int32_t) * n_new, hipMemcpyDeviceToHost, s));
	int step_flag = 0;
	GEN_TRY(hipMemcpyAsync(&step_flag, m->d_err, sizeof(int), hipMemcpyDeviceToHost, s));
	GEN_TRY(hipStreamSynchronize(s));
	if ((step_flag & 2) && m->block_fused > 0)
	{
		// a wait inside the one-launch attention half ran out: the tokens are void; once more, from
		// the prompt, through the separate launches (`past` has not moved)
		const int zero = 0;
		GEN_TRY(hipMemcpy(m->d_err, &zero, sizeof(int), hipMemcpyHostToDevice));
		cleanup();
		give_up_block_launch(m);
		return litenn_hip_llama_generate(m, prompt, n_prompt, n_new, out_tokens, flags, prefill_ms, decode_ms);
	}
	float ms = 0.0f;
	if (prefill_ms)
	{
		GEN_TRY(hipEventElapsedTime(&ms, ev[0], ev[1]));
		*prefill_ms = ms;
	}
	if (decode_ms)
	{
		GEN_TRY(hipEventElapsedTime(&ms, ev[1], ev[2]));
		*decode_ms = ms;
	}
	cleanup();
#undef GEN_TRY
	// the last emitted token has not been fed back: the cache holds prompt + (n_new - 1) rows
	m->past += static_cast<int>(n_prompt + n_new - 1);
	return rc;
}

extern "C" int litenn_hip_llama_get_kv(litenn_hip_llama* m, int layer, float* k, float* v)
{
	if (!m || layer < 0 || layer >= m->p.block_count)
	{
		return fail(kAction, "layer index out of range");
	}
	DeviceGuard guard(m->dev);
	if (!guard.ok())
	{
		return fail_hip(kAction, guard.error());
	}
	const size_t count = static_cast<size_t>(m->past) * m->p.head_count_kv * m->head_dim;
	if (count == 0)
	{
		return 0;
	}
	LITENN_HIP_TRY(kAction, hipStreamSynchronize(m->stream));
	float* tmp = nullptr;
	LITENN_HIP_TRY(kAction, hipMalloc(reinterpret_cast<void**>(&tmp), sizeof(float) * count));
	int rc = 0;
	const Layer& L = m->layers[static_cast<size_t>(layer)];
	const void* caches[2] = { L.kcache, L.vcache };
	float* outs[2] = { k, v };
	for (int i = 0; i < 2 && rc == 0; ++i)
	{
		if (!launch_convert(m->p.kv_dtype, caches[i], count, LITENN_F32, tmp, m->stream))
		{
			rc = fail(kAction, "cache conversion failed");
			break;
		}
		const void* src = tmp;
		hipError_t e = hipMemcpyAsync(outs[i], src, sizeof(float) * count, hipMemcpyDeviceToHost, m->stream);
		if (e == hipSuccess)
		{
			e = hipStreamSynchronize(m->stream);
		}
		if (e != hipSuccess)
		{
			rc = fail_hip(kAction, e);
		}
	}
	(void)hipFree(tmp);
	return rc;
}
