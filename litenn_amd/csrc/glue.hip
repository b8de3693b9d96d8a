// The small kernels that surround the quantised matmuls in the LLaMA decoder:
// RMSNorm, interleaved RoPE, KV-cache append, causal single-row attention over an
// fp16/f32 cache, SiLU*up, arg-max.  All of them are bandwidth-trivial next to the
// weight stream; they are written to keep f32 (f64 for the norm) semantics of the
// reference chains and to read every operand once.
#include "common.hpp"
#include "attn_math.hpp"

#include <algorithm>

// Scratch of the allocation-free attention entry point (litenn_hip_attn_decode_noalloc): the
// chunk triples {running maximum, sum, head_dim outputs} of one query row cut into key chunks,
// followed by one arrival counter per head.  1 MiB of triples: a row is cut into
// min(16, ceil(1024 / heads)) chunks at most, so heads * chunks < 2048 and every launch with heads
// of up to 128 features fits; wider heads fit up to heads * chunks * (head_dim + 2) <= 262144
// (e.g. 48 heads of 256 features, not 64).  Only rows that are cut (m == 1, heads <= 1024) use the
// array at all.  Every GPU the library runs on holds its own copy (1 MiB + 4 KiB) until the
// process ends.  Host code never uses the
// array's name as an address: static_attn_scratch() asks the runtime for the device address once
// per device and hands that pointer to the launches.
constexpr size_t kStaticAttnPartialFloats = size_t{ 256 } * 1024;
constexpr size_t kStaticAttnCounters = 1024;
static __device__ __align__(256) float scratch[kStaticAttnPartialFloats + kStaticAttnCounters];

namespace litenn_hip
{
	namespace
	{
		__global__ void zero_ints_kernel(int* p, int n)
		{
			const int i = blockIdx.x * blockDim.x + threadIdx.x;
			if (i < n)
			{
				p[i] = 0;
			}
		}

		// ---------------- RMSNorm (f64 accumulate, ComputePrimitives.h:792-817) -------------
		__global__ __launch_bounds__(1024) void rmsnorm_kernel(const float* __restrict__ x,
		                                                        const float* __restrict__ w, double eps, int d,
		                                                        float* __restrict__ y)
		{
			__shared__ double red[16];
			const float* xr = x + static_cast<size_t>(blockIdx.x) * d;
			float* yr = y + static_cast<size_t>(blockIdx.x) * d;
			double acc = 0.0;
			for (int i = threadIdx.x; i < d; i += blockDim.x)
			{
				const double v = static_cast<double>(xr[i]);
				acc += v * v;
			}
			for (int off = 32; off > 0; off >>= 1)
			{
				acc += __shfl_xor(acc, off, 64);
			}
			if ((threadIdx.x & 63) == 0)
			{
				red[threadIdx.x >> 6] = acc;
			}
			__syncthreads();
			double total = 0.0;
			for (int i = 0; i < static_cast<int>(blockDim.x >> 6); ++i)
			{
				total += red[i];
			}
			// x / denom as a multiplication by the f64 reciprocal: one f64 ulp from the quotient,
			// invisible after the final rounding to f32
			const double inv = 1.0 / sqrt(total / static_cast<double>(d) + eps);
			for (int i = threadIdx.x; i < d; i += blockDim.x)
			{
				double v = static_cast<double>(xr[i]) * inv;
				if (w)
				{
					v *= static_cast<double>(w[i]);
				}
				yr[i] = static_cast<float>(v);
			}
		}

		// ---------------- RoPE -------------------------------------------------------------
		// Angle tables exactly as MakeRoPEAngleTable builds them (RoPE.h:24-41): f64 maths,
		// stored as f32.  table[pos * half + dim] for pos in [0, positions).
		__global__ void rope_table_kernel(float* __restrict__ cos_t, float* __restrict__ sin_t, int positions, int half,
		                                  double base, double freq_scale, int pos_offset)
		{
			const int idx = blockIdx.x * blockDim.x + threadIdx.x;
			if (idx >= positions * half)
			{
				return;
			}
			const int pos = idx / half, dim = idx % half;
			const double exponent = -2.0 * static_cast<double>(dim) / static_cast<double>(half * 2);
			const double inv_freq = pow(base, exponent);
			const double angle = static_cast<double>(pos_offset + pos) * inv_freq * freq_scale;
			cos_t[idx] = static_cast<float>(cos(angle));
			sin_t[idx] = static_cast<float>(sin(angle));
		}

		// x,y [m, n_heads, head_dim]; tables indexed by row (positions start at the table's origin)
		__global__ void rope_kernel(const float* __restrict__ x, float* __restrict__ y, int m, int n_heads, int head_dim,
		                            int rope_dims, const float* __restrict__ cos_t, const float* __restrict__ sin_t)
		{
			const int half_all = head_dim / 2;
			const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
			const size_t total = static_cast<size_t>(m) * n_heads * half_all;
			if (idx >= total)
			{
				return;
			}
			const int p = idx % half_all;
			const size_t rh = idx / half_all; // row * n_heads + head
			const int row = rh / n_heads;
			const size_t base = rh * head_dim + 2 * p;
			const float a = x[base], b = x[base + 1];
			if (2 * p < rope_dims)
			{
				const int half = rope_dims / 2;
				float o0, o1;
				rotate(a, b, cos_t[row * half + p], sin_t[row * half + p], o0, o1);
				y[base] = o0;
				y[base + 1] = o1;
			}
			else
			{
				y[base] = a;
				y[base + 1] = b;
			}
		}

		template <typename KV>
		__device__ __forceinline__ void store_kv(KV* dst, float v);
		template <>
		__device__ __forceinline__ void store_kv<float>(float* dst, float v) { *dst = v; }
		template <>
		__device__ __forceinline__ void store_kv<uint16_t>(uint16_t* dst, float v) { *dst = f32_to_f16_bits_litenn(v); }

		template <typename KV>
		__device__ __forceinline__ float load_kv(const KV* src);
		template <>
		__device__ __forceinline__ float load_kv<float>(const float* src) { return *src; }
		template <>
		__device__ __forceinline__ float load_kv<uint16_t>(const uint16_t* src) { return f16_bits_to_f32(*src); }

		template <typename KV>
		__global__ void kv_append_kernel(KV* __restrict__ cache, size_t past, const float* __restrict__ cur, size_t count)
		{
			const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
			if (idx < count)
			{
				store_kv<KV>(cache + past + idx, cur[idx]);
			}
		}

		// Decoder step glue: rotate q in place, rotate k and append it and v to the caches
		// (tools/gguf/LLaMABuilder.cpp:596-622,640-645).  Position of row i is *past + i.
		// tables are [ctx, rope_dims/2].
		template <typename KV>
		__global__ void rope_qkv_append_kernel(float* __restrict__ q, const float* __restrict__ k,
		                                       const float* __restrict__ v, KV* __restrict__ kcache,
		                                       KV* __restrict__ vcache, const int* __restrict__ past_dev, int m,
		                                       int n_head, int n_kv_head, int head_dim, int rope_dims,
		                                       const float* __restrict__ cos_t, const float* __restrict__ sin_t)
		{
			const int half_all = head_dim / 2;
			const int half = rope_dims / 2;
			const int past = *past_dev;
			const int heads = n_head + 2 * n_kv_head; // q heads, k heads, v heads
			const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
			const size_t total = static_cast<size_t>(m) * heads * half_all;
			if (idx >= total)
			{
				return;
			}
			const int p = idx % half_all;
			const size_t rh = idx / half_all;
			const int row = rh / heads;
			const int h = rh % heads;
			const int pos = past + row;
			const size_t kvw = static_cast<size_t>(n_kv_head) * head_dim;
			if (h < n_head)
			{
				float* base = q + (static_cast<size_t>(row) * n_head + h) * head_dim + 2 * p;
				if (2 * p < rope_dims)
				{
					float o0, o1;
					rotate(base[0], base[1], cos_t[static_cast<size_t>(pos) * half + p],
					       sin_t[static_cast<size_t>(pos) * half + p], o0, o1);
					base[0] = o0;
					base[1] = o1;
				}
			}
			else if (h < n_head + n_kv_head)
			{
				const int kh = h - n_head;
				const float* src = k + static_cast<size_t>(row) * kvw + kh * head_dim + 2 * p;
				KV* dst = kcache + static_cast<size_t>(pos) * kvw + kh * head_dim + 2 * p;
				float o0 = src[0], o1 = src[1];
				if (2 * p < rope_dims)
				{
					rotate(src[0], src[1], cos_t[static_cast<size_t>(pos) * half + p],
					       sin_t[static_cast<size_t>(pos) * half + p], o0, o1);
				}
				store_kv<KV>(dst, o0);
				store_kv<KV>(dst + 1, o1);
			}
			else
			{
				const int vh = h - n_head - n_kv_head;
				const float* src = v + static_cast<size_t>(row) * kvw + vh * head_dim + 2 * p;
				KV* dst = vcache + static_cast<size_t>(pos) * kvw + vh * head_dim + 2 * p;
				store_kv<KV>(dst, src[0]);
				store_kv<KV>(dst + 1, src[1]);
			}
		}

		// ---------------- attention of one query row against the cache -----------------------
		// grid (n_head, splits, m); block 256.  Query row i sits at position past + i and sees
		// keys 0 .. past + i (the additive -1e9 causal constant of CausalMask.h:16-34 turns every
		// later key into an exact zero after exp in f32, so those keys are simply not visited).
		//
		// The keys of a row are cut into `splits` contiguous chunks, one workgroup each.  Inside a
		// workgroup a key is handled by 16 lanes (each lane owns a contiguous run of the head
		// dimension), so a wave covers 4 keys and the workgroup 16 keys per step, kUnroll steps in
		// flight.  Every 16-lane group keeps a running (max, sum, weighted V) triple; the 16 triples
		// are merged through LDS.  With splits > 1 the workgroup's triple goes to `partial` and the
		// last workgroup of the row/head to arrive (device-scope counter) merges the splits.
		// The merged result equals softmax(q.K^T * scale) . V of Attention.h:57-80 up to f32
		// summation order.  head_dim <= 256.
		// AttnLoad: the run of the head dimension a lane owns, fetched as raw words (so several
		// rows can be in flight before any is converted) and unpacked to f32 afterwards.
		template <typename KV, bool FAST>
		struct AttnLoad;

		// generic: up to 16 elements per lane, bounds-checked scalar loads
		template <typename KV>
		struct AttnLoad<KV, false>
		{
			static constexpr int E = 16;
			struct Raw
			{
				KV v[E];
			};
			__device__ static Raw load(const KV* p, int first, int per, int head_dim)
			{
				Raw r;
#pragma unroll
				for (int e = 0; e < E; ++e)
				{
					r.v[e] = (e < per && first + e < head_dim) ? p[first + e] : KV{};
				}
				return r;
			}
			__device__ static void unpack(const Raw& r, float (&out)[E])
			{
#pragma unroll
				for (int e = 0; e < E; ++e)
				{
					out[e] = load_kv<KV>(&r.v[e]);
				}
			}
		};

		// head_dim 128, 16-byte aligned rows: 8 elements per lane in one or two 16-byte loads
		template <>
		struct AttnLoad<uint16_t, true>
		{
			static constexpr int E = 8;
			using Raw = uint4;
			// non-temporal like the weight rows of the GEMV: a cached key or value is read once per launch
			// by the query heads of its group (7B-shape decode 728.7 -> 737.1 tok/s, 8B shape 635.7 -> 641.3)
			__device__ static Raw load(const uint16_t* p, int first, int, int)
			{
				typedef unsigned u32x4_t __attribute__((ext_vector_type(4)));
				const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p + first));
				return make_uint4(v.x, v.y, v.z, v.w);
			}
			__device__ static void unpack(const Raw& raw, float (&out)[E])
			{
				const uint32_t w[4] = { raw.x, raw.y, raw.z, raw.w };
#pragma unroll
				for (int i = 0; i < 4; ++i)
				{
					out[2 * i] = f16_bits_to_f32(static_cast<uint16_t>(w[i] & 0xffffu));
					out[2 * i + 1] = f16_bits_to_f32(static_cast<uint16_t>(w[i] >> 16));
				}
			}
		};

		template <>
		struct AttnLoad<float, true>
		{
			static constexpr int E = 8;
			struct Raw
			{
				float4 a, b;
			};
			__device__ static Raw load(const float* p, int first, int, int)
			{
				return Raw{ *reinterpret_cast<const float4*>(p + first), *reinterpret_cast<const float4*>(p + first + 4) };
			}
			__device__ static void unpack(const Raw& r, float (&out)[E])
			{
				out[0] = r.a.x, out[1] = r.a.y, out[2] = r.a.z, out[3] = r.a.w;
				out[4] = r.b.x, out[5] = r.b.y, out[6] = r.b.z, out[7] = r.b.w;
			}
		};

		constexpr int kMaxAttnSplits = 16;

		// Key chunks a single row's attention over `len` cached keys is cut into: the nearest integer
		// to 2.2 sqrt(len / 64), within 1 .. 16 (3 at 128 keys, 6 at 512, 9 at 1024, 16 from 3400 on).
		// More chunks shorten a chunk's key loop and lengthen nothing but the merge, whose cost hardly
		// depends on their number; measured in the decoder, 8B shape at 512 .. 1024 keys: 2 chunks
		// 574, 4: 602, 6: 608, 8: 606, 12: 602, 16: 600 tok/s; 7B shape at 128 .. 384 keys flat within
		// 2 % from 3 to 8.  Integer arithmetic, so the host (which sizes the grid) and the kernel
		// (which reads the length on the device) agree: c + 1 chunks from (2c + 1)^2 * 400 <= 121 len.
		__host__ __device__ inline int attn_live_chunks(long long len)
		{
			int c = 1;
			while (c < kMaxAttnSplits && static_cast<long long>(2 * c + 1) * (2 * c + 1) * 400 <= 121 * len)
			{
				++c;
			}
			return c;
		}

		// What the single-token step adds when the rotation and the cache append ride inside the
		// attention launch (tools/gguf/LLaMABuilder.cpp:596-622,640-645): q, k_new and v_new are the
		// un-rotated projections of the one new row; the tables are [ctx, rope_dims / 2].
		struct AttnStep
		{
			const float* k_new;
			const float* v_new;
			const float* cos_t;
			const float* sin_t;
			int rope_dims;
		};

		// FUSED (single new row, head_dim 128): q arrives un-rotated and is rotated in registers;
		// the cache holds positions 0 .. past - 1 and the new position's key/value come from
		// step.k_new / step.v_new, rounded through the cache's type exactly as an append followed
		// by a read would round them.  The first query head of every KV head also writes them to
		// the cache, which no workgroup of this launch reads at that position.
		//
		// Every global load that does not depend on another is issued before the first wait (the
		// row's operands, the first batch of cached keys), so a launch costs about two memory
		// latencies however it is configured.
		template <typename KV, bool FAST, bool FUSED>
		__global__ __launch_bounds__(256) void attn_decode_kernel(const float* __restrict__ q, KV* __restrict__ kcache,
		                                                           KV* __restrict__ vcache, float* __restrict__ out,
		                                                           const int* __restrict__ past_dev, int past_host,
		                                                           int n_head, int n_kv_head, int head_dim,
		                                                           float scale, float* __restrict__ partial,
		                                                           int* __restrict__ counters, AttnStep step)
		{
			static_assert(!FUSED || FAST, "the fused step exists for 128-wide heads only");
			using Load = AttnLoad<KV, FAST>;
			using LoadF = AttnLoad<float, FAST>;
			constexpr int E = Load::E;
			constexpr int kUnroll = 4;
			__shared__ float s_m[16], s_l[16];
			__shared__ float s_o[16][256 + 4];
			__shared__ int s_last;
			// Workgroups go to the eight XCDs (each with its own L2) round-robin in the order of
			// blockIdx.x: with a head count that is a multiple of 8, XCD x is given the heads
			// [x n_head / 8, (x + 1) n_head / 8), so that the query heads that share a KV head read
			// its keys and values through one L2 (8B shape, 32 heads over 8 KV heads: 8.4 MB fetched
			// per launch for 2.1 MB of cache otherwise).
			const int h = (n_head & 7) == 0 ? static_cast<int>(blockIdx.x & 7) * (n_head >> 3) + static_cast<int>(blockIdx.x >> 3)
			                                : static_cast<int>(blockIdx.x);
			const int split = blockIdx.y;
			const int row = blockIdx.z;
			const int tid = threadIdx.x;
			const int past = past_dev ? *past_dev : past_host;
			const int pos = past + row;
			const int len = FUSED ? pos : pos + 1; // keys read from the cache
			// The grid holds the chunks of the longest cache the launch may meet (a captured launch is
			// replayed while the cache fills); the chunks this length does not need leave at once.
			const int splits = min(static_cast<int>(gridDim.y), attn_live_chunks(len));
			if (split >= splits)
			{
				return;
			}
			const int kvh = h / (n_head / n_kv_head);
			const size_t kvw = static_cast<size_t>(n_kv_head) * head_dim;
			const float* qr = q + (static_cast<size_t>(row) * n_head + h) * head_dim;
			const KV* kbase = kcache + static_cast<size_t>(kvh) * head_dim;
			const KV* vbase = vcache + static_cast<size_t>(kvh) * head_dim;

			const int sub = tid & 15; // lane within the key's group
			const int grp = tid >> 4; // key slot of the workgroup
			const int per = FAST ? 8 : (head_dim + 15) >> 4;
			const int first = sub * per;

			const int chunk = (len + splits - 1) / splits;
			const int t_begin = split * chunk;
			const int t_end = min(len, t_begin + chunk);

			// ---- issue: the row's operands, then the first batch of keys and values
			const typename LoadF::Raw q_raw = LoadF::load(qr, first, per, head_dim);
			const bool new_key_here = FUSED && split == splits - 1 && grp == 0;
			float4 cos4 = {}, sin4 = {};
			typename LoadF::Raw kn_raw = {}, vn_raw = {};
			const bool rotates = FUSED && first < step.rope_dims;
			if constexpr (FUSED)
			{
				// lanes outside the rotary width fetch (and ignore) the first angles of the row
				const size_t at = static_cast<size_t>(pos) * (step.rope_dims >> 1) + (rotates ? first >> 1 : 0);
				cos4 = *reinterpret_cast<const float4*>(step.cos_t + at);
				sin4 = *reinterpret_cast<const float4*>(step.sin_t + at);
				kn_raw = LoadF::load(step.k_new + static_cast<size_t>(kvh) * head_dim, first, per, head_dim);
				vn_raw = LoadF::load(step.v_new + static_cast<size_t>(kvh) * head_dim, first, per, head_dim);
			}
			typename Load::Raw k_raw[kUnroll], v_raw[kUnroll];
			int t0 = t_begin + grp;
			const auto issue = [&](int from) {
#pragma unroll
				for (int u = 0; u < kUnroll; ++u)
				{
					// keys past the chunk re-read a valid one and get weight zero below
					const int t = min(from + 16 * u, t_end - 1);
					k_raw[u] = Load::load(kbase + static_cast<size_t>(t) * kvw, first, per, head_dim);
					v_raw[u] = Load::load(vbase + static_cast<size_t>(t) * kvw, first, per, head_dim);
				}
			};
			if (t0 < t_end)
			{
				issue(t0);
			}

			float qv[E];
			LoadF::unpack(q_raw, qv);
			float kn[E], vn[E];
			if constexpr (FUSED)
			{
				LoadF::unpack(kn_raw, kn);
				LoadF::unpack(vn_raw, vn);
				if (rotates)
				{
					rotate8(qv, cos4, sin4);
					rotate8(kn, cos4, sin4);
				}
				if (new_key_here)
				{
					round_through_cache<KV>(kn);
					round_through_cache<KV>(vn);
					if (h % (n_head / n_kv_head) == 0)
					{
						store8_exact(kcache + static_cast<size_t>(pos) * kvw + kvh * head_dim + first, kn);
						store8_exact(vcache + static_cast<size_t>(pos) * kvw + kvh * head_dim + first, vn);
					}
				}
			}

			float run_m = -INFINITY, run_l = 0.0f;
			float o[E];
#pragma unroll
			for (int e = 0; e < E; ++e)
			{
				o[e] = 0.0f;
			}
			while (t0 < t_end)
			{
				float kf[kUnroll][E], vf[kUnroll][E];
				float s[kUnroll];
#pragma unroll
				for (int u = 0; u < kUnroll; ++u)
				{
					Load::unpack(k_raw[u], kf[u]);
					Load::unpack(v_raw[u], vf[u]);
				}
				const int t_next = t0 + 16 * kUnroll;
				if (t_next < t_end)
				{
					issue(t_next);
				}
				float step_m = run_m;
#pragma unroll
				for (int u = 0; u < kUnroll; ++u)
				{
					float acc = 0.0f;
#pragma unroll
					for (int e = 0; e < E; ++e)
					{
						acc = fmaf(qv[e], kf[u][e], acc);
					}
					acc = row16_sum(acc) * scale;
					s[u] = (t0 + 16 * u < t_end) ? acc : -INFINITY;
					step_m = fmaxf(step_m, s[u]);
				}
				// step_m is finite: the first key of the step is always inside the chunk
				const float corr = expf(run_m - step_m);
				run_l *= corr;
#pragma unroll
				for (int e = 0; e < E; ++e)
				{
					o[e] *= corr;
				}
#pragma unroll
				for (int u = 0; u < kUnroll; ++u)
				{
					const float p = expf(s[u] - step_m);
					run_l += p;
#pragma unroll
					for (int e = 0; e < E; ++e)
					{
						o[e] = fmaf(p, vf[u][e], o[e]);
					}
				}
				run_m = step_m;
				t0 = t_next;
			}

			if constexpr (FUSED)
			{
				if (new_key_here)
				{
					float acc = 0.0f;
#pragma unroll
					for (int e = 0; e < E; ++e)
					{
						acc = fmaf(qv[e], kn[e], acc);
					}
					const float sc = row16_sum(acc) * scale;
					const float step_m = fmaxf(run_m, sc);
					const float corr = expf(run_m - step_m);
					const float pw = expf(sc - step_m);
					run_l = fmaf(run_l, corr, pw);
#pragma unroll
					for (int e = 0; e < E; ++e)
					{
						o[e] = fmaf(pw, vn[e], o[e] * corr);
					}
					run_m = step_m;
				}
			}

			if (sub == 0)
			{
				s_m[grp] = run_m;
				s_l[grp] = run_l;
			}
#pragma unroll
			for (int e = 0; e < E; ++e)
			{
				if (e < per && first + e < head_dim)
				{
					s_o[grp][first + e] = o[e];
				}
			}
			__syncthreads();
			float m_all = -INFINITY, l_all = 0.0f, o_all = 0.0f;
			if (tid < head_dim)
			{
#pragma unroll
				for (int g = 0; g < 16; ++g)
				{
					m_all = fmaxf(m_all, s_m[g]);
				}
#pragma unroll
				for (int g = 0; g < 16; ++g)
				{
					const float w = softmax_weight(s_m[g], m_all);
					l_all = fmaf(s_l[g], w, l_all);
					o_all = fmaf(s_o[g][tid], w, o_all);
				}
			}
			float* dst = out + (static_cast<size_t>(row) * n_head + h) * head_dim;
			if (splits == 1)
			{
				if (tid < head_dim)
				{
					dst[tid] = o_all / l_all;
				}
				return;
			}

			// several splits: publish this chunk's triple, the last arrival merges them
			const size_t slot = static_cast<size_t>(row) * n_head + h;
			const int stride = head_dim + 2;
			float* mine = partial + (slot * splits + split) * stride;
			// The triples cross between workgroups (and between the chip's L2 slices) through
			// device-scope relaxed atomics, which write through and read around the non-coherent
			// cache levels; a full device fence would instead flush the whole L2 in every workgroup.
			// Order: triple stores complete (vmcnt 0) -> barrier -> counter increment; the merging
			// workgroup reads the triples only after it has seen the last increment.
			if (tid < head_dim)
			{
				device_store(mine + 2 + tid, o_all);
				if (tid == 0)
				{
					device_store(mine, m_all);
					device_store(mine + 1, l_all);
				}
			}
			asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
			__syncthreads();
			if (tid == 0)
			{
				const int arrived = __hip_atomic_fetch_add(&counters[slot], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
				s_last = arrived == splits - 1;
				if (s_last)
				{
					// ready for the next launch on this stream
					__hip_atomic_store(&counters[slot], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
				}
			}
			__syncthreads();
			if (!s_last)
			{
				return;
			}
			if (tid < head_dim)
			{
				// every split's triple is fetched before the first is used: one memory latency
				const float* all = partial + slot * splits * stride;
				float pm[kMaxAttnSplits], pl[kMaxAttnSplits], po[kMaxAttnSplits];
#pragma unroll
				for (int sidx = 0; sidx < kMaxAttnSplits; ++sidx)
				{
					const float* src = all + min(sidx, splits - 1) * stride;
					pm[sidx] = device_load(src);
					pl[sidx] = device_load(src + 1);
					po[sidx] = device_load(src + 2 + tid);
				}
				float mm = -INFINITY;
#pragma unroll
				for (int sidx = 0; sidx < kMaxAttnSplits; ++sidx)
				{
					mm = fmaxf(mm, pm[sidx]);
				}
				float ll = 0.0f, oo = 0.0f;
#pragma unroll
				for (int sidx = 0; sidx < kMaxAttnSplits; ++sidx)
				{
					const float w = sidx < splits ? softmax_weight(pm[sidx], mm) : 0.0f;
					ll = fmaf(pl[sidx], w, ll);
					oo = fmaf(po[sidx], w, oo);
				}
				dst[tid] = oo / ll;
			}
		}

		// ---------------- attention with the reference layer's options -----------------------
		// AddFlashAttnExt with mask, ALiBi slope, logit softcap, sinks and an offset causal mask
		// (src/LiteNN/Layer/FlashAttnExt.h:17-29,100-228), every head of a call at once.  The
		// LLaMA lowering uses none of these options, so this kernel is plain: grid (n_head, m), 256
		// threads, sixteen lanes per key as in the row kernel above, one pass with an online softmax.
		struct AttnExt
		{
			const float* mask;  // additive [m, keys], or null
			const float* sinks; // [n_head], or null
			float score_scale;  // scale, or scale / softcap
			float softcap;      // 0: none
			int apply_scale;    // the reference emits no multiply by exactly 1 (FlashAttnExt.h:57-67)
			int apply_cap;      // softcap != 1
			double max_bias;    // > 0: the mask is multiplied by the head's ALiBi slope
			int causal;
			long long key_offset, query_offset;
			int keys;
		};

		// Detail::ComputeALiBiSlope (FlashAttnExt.h:69-96), in double like the reference
		__device__ inline double alibi_slope(int head, int heads, double max_bias)
		{
			int head_log2 = 1;
			while ((head_log2 << 1) <= heads)
			{
				head_log2 <<= 1;
			}
			const double m0 = pow(2.0, -max_bias / static_cast<double>(head_log2));
			const double m1 = pow(2.0, -(max_bias / 2.0) / static_cast<double>(head_log2));
			return head < head_log2 ? pow(m0, static_cast<double>(head + 1))
			                        : pow(m1, static_cast<double>(2 * (head - head_log2) + 1));
		}

		template <typename KV>
		__global__ __launch_bounds__(256) void attn_ext_kernel(const float* __restrict__ q, const KV* __restrict__ kcache,
		                                                       const KV* __restrict__ vcache, float* __restrict__ out,
		                                                       int n_head, int n_kv_head, int head_dim, AttnExt x)
		{
			using Load = AttnLoad<KV, false>;
			using LoadF = AttnLoad<float, false>;
			constexpr int E = Load::E;
			__shared__ float s_m[16], s_l[16];
			__shared__ float s_o[16][256 + 4];
			const int h = blockIdx.x, row = blockIdx.y, tid = threadIdx.x;
			const int sub = tid & 15, grp = tid >> 4;
			const int per = (head_dim + 15) >> 4;
			const int first = sub * per;
			const int kvh = h / (n_head / n_kv_head);
			const size_t kvw = static_cast<size_t>(n_kv_head) * head_dim;
			const KV* kbase = kcache + static_cast<size_t>(kvh) * head_dim;
			const KV* vbase = vcache + static_cast<size_t>(kvh) * head_dim;
			float qv[E];
			LoadF::unpack(LoadF::load(q + (static_cast<size_t>(row) * n_head + h) * head_dim, first, per, head_dim), qv);
			float slope = 1.0f;
			bool apply_slope = false;
			if (x.mask && x.max_bias > 0.0)
			{
				const double sl = alibi_slope(h, n_head, x.max_bias);
				slope = static_cast<float>(sl);
				apply_slope = sl != 1.0;
			}
			// keys the causal mask leaves visible; a masked key's weight is exp(-1e9 - max) = 0 exactly
			// in the reference, so it is not visited (the host has checked that every row sees one)
			int len = x.keys;
			if (x.causal)
			{
				const long long visible = x.query_offset + row - x.key_offset + 1;
				len = static_cast<int>(visible < len ? visible : len);
			}
			float run_m = -INFINITY, run_l = 0.0f;
			float o[E];
#pragma unroll
			for (int e = 0; e < E; ++e)
			{
				o[e] = 0.0f;
			}
			for (int t = grp; t < len; t += 16)
			{
				float kf[E], vf[E];
				Load::unpack(Load::load(kbase + static_cast<size_t>(t) * kvw, first, per, head_dim), kf);
				Load::unpack(Load::load(vbase + static_cast<size_t>(t) * kvw, first, per, head_dim), vf);
				float acc = 0.0f;
#pragma unroll
				for (int e = 0; e < E; ++e)
				{
					acc = fmaf(qv[e], kf[e], acc);
				}
				float sc = row16_sum(acc);
				if (x.apply_scale)
				{
					sc = __fmul_rn(sc, x.score_scale);
				}
				if (x.softcap != 0.0f)
				{
					// AddTanh as the layer lowers it (Activation.h:34-50): (exp(2x) - 1) / (exp(2x) + 1)
					const float ex = expf(__fmul_rn(sc, 2.0f));
					sc = __fdiv_rn(__fsub_rn(ex, 1.0f), __fadd_rn(ex, 1.0f));
					if (x.apply_cap)
					{
						sc = __fmul_rn(sc, x.softcap);
					}
				}
				if (x.mask)
				{
					float mv = x.mask[static_cast<size_t>(row) * x.keys + t];
					if (apply_slope)
					{
						mv = __fmul_rn(mv, slope);
					}
					sc = __fadd_rn(sc, mv);
				}
				const float new_m = fmaxf(run_m, sc);
				const float corr = softmax_weight(run_m, new_m);
				const float pw = expf(sc - new_m);
				run_l = fmaf(run_l, corr, pw);
#pragma unroll
				for (int e = 0; e < E; ++e)
				{
					o[e] = fmaf(pw, vf[e], o[e] * corr);
				}
				run_m = new_m;
			}
			if (sub == 0)
			{
				s_m[grp] = run_m;
				s_l[grp] = run_l;
			}
#pragma unroll
			for (int e = 0; e < E; ++e)
			{
				if (e < per && first + e < head_dim)
				{
					s_o[grp][first + e] = o[e];
				}
			}
			__syncthreads();
			if (tid < head_dim)
			{
				float m_all = -INFINITY;
#pragma unroll
				for (int g = 0; g < 16; ++g)
				{
					m_all = fmaxf(m_all, s_m[g]);
				}
				float l_all = 0.0f, o_all = 0.0f;
				if (x.sinks)
				{
					// the sink joins the row maximum and the denominator, not the values (FlashAttnExt.h:184-212)
					const float sink = x.sinks[h];
					m_all = fmaxf(m_all, sink);
					l_all = expf(sink - m_all);
				}
#pragma unroll
				for (int g = 0; g < 16; ++g)
				{
					const float w = softmax_weight(s_m[g], m_all);
					l_all = fmaf(s_l[g], w, l_all);
					o_all = fmaf(s_o[g][tid], w, o_all);
				}
				out[(static_cast<size_t>(row) * n_head + h) * head_dim + tid] = o_all / l_all;
			}
		}

		// ---------------- SiLU(gate) * up (Activation.h:22-35,56-63; SwiGLU.h:63-66) ---------
		__global__ void silu_mul_kernel(const float* __restrict__ gate, const float* __restrict__ up,
		                                float* __restrict__ y, size_t n)
		{
			const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
			if (i < n)
			{
				const float g = gate[i];
				const float sig = __fdiv_rn(1.0f, __fadd_rn(1.0f, expf(-g)));
				y[i] = __fmul_rn(__fmul_rn(g, sig), up[i]);
			}
		}

		// ---------------- arg-max: first maximal index ---------------------------------------
		__global__ __launch_bounds__(1024) void argmax_kernel(const float* __restrict__ x, int n,
		                                                       int32_t* __restrict__ out)
		{
			__shared__ float bv[16];
			__shared__ int bi[16];
			const float* xr = x + static_cast<size_t>(blockIdx.x) * n;
			float best = -INFINITY;
			int best_i = 0x7fffffff;
			for (int i = threadIdx.x; i < n; i += blockDim.x)
			{
				const float v = xr[i];
				if (v > best || best_i == 0x7fffffff)
				{
					best = v;
					best_i = i;
				}
			}
			for (int off = 32; off > 0; off >>= 1)
			{
				const float ov = __shfl_xor(best, off, 64);
				const int oi = __shfl_xor(best_i, off, 64);
				if (ov > best || (ov == best && oi < best_i))
				{
					best = ov;
					best_i = oi;
				}
			}
			if ((threadIdx.x & 63) == 0)
			{
				bv[threadIdx.x >> 6] = best;
				bi[threadIdx.x >> 6] = best_i;
			}
			__syncthreads();
			if (threadIdx.x == 0)
			{
				for (int wv = 1; wv < static_cast<int>(blockDim.x >> 6); ++wv)
				{
					if (bv[wv] > best || (bv[wv] == best && bi[wv] < best_i))
					{
						best = bv[wv];
						best_i = bi[wv];
					}
				}
				out[blockIdx.x] = best_i == 0x7fffffff ? 0 : best_i;
			}
		}

		// ---- arg-max of one long row in two launches (the decoder's vocabulary) -------------------
		// Many workgroups scan a chunk each; one wavefront merges their (value, index) pairs, stores
		// the token and advances the decoder's device-side counters {past length, tokens emitted}.
		constexpr int kArgmaxChunk = 2048;

		__device__ __forceinline__ void argmax_take(float ov, int oi, float& best, int& best_i)
		{
			if (ov > best || (ov == best && oi < best_i))
			{
				best = ov;
				best_i = oi;
			}
		}

		__global__ __launch_bounds__(256) void argmax_partial_kernel(const float* __restrict__ x, int n,
		                                                              float* __restrict__ pv, int* __restrict__ pi)
		{
			__shared__ float bv[4];
			__shared__ int bi[4];
			const int begin = blockIdx.x * kArgmaxChunk, end = min(n, begin + kArgmaxChunk);
			float best = -INFINITY;
			int best_i = 0x7fffffff;
			for (int i = begin + threadIdx.x; i < end; i += 256)
			{
				const float v = x[i];
				if (v > best || best_i == 0x7fffffff)
				{
					best = v;
					best_i = i;
				}
			}
			for (int off = 32; off > 0; off >>= 1)
			{
				argmax_take(__shfl_xor(best, off, 64), __shfl_xor(best_i, off, 64), best, best_i);
			}
			if ((threadIdx.x & 63) == 0)
			{
				bv[threadIdx.x >> 6] = best;
				bi[threadIdx.x >> 6] = best_i;
			}
			__syncthreads();
			if (threadIdx.x == 0)
			{
				for (int wv = 1; wv < 4; ++wv)
				{
					argmax_take(bv[wv], bi[wv], best, best_i);
				}
				pv[blockIdx.x] = best;
				pi[blockIdx.x] = best_i;
			}
		}

		// one wavefront; counters = {past length, tokens emitted, steps run}, out may be null
		__global__ __launch_bounds__(64) void argmax_merge_step_kernel(const float* __restrict__ pv,
		                                                                const int* __restrict__ pi, int blocks,
		                                                                int32_t* __restrict__ next, int* counters,
		                                                                int past_inc, int32_t* __restrict__ out)
		{
			float best = -INFINITY;
			int best_i = 0x7fffffff;
			for (int b = threadIdx.x; b < blocks; b += 64)
			{
				argmax_take(pv[b], pi[b], best, best_i);
			}
			for (int off = 32; off > 0; off >>= 1)
			{
				argmax_take(__shfl_xor(best, off, 64), __shfl_xor(best_i, off, 64), best, best_i);
			}
			if (threadIdx.x == 0)
			{
				const int32_t token = best_i == 0x7fffffff ? 0 : best_i;
				*next = token;
				if (out)
				{
					out[counters[1]] = token;
					counters[1] += 1;
				}
				counters[0] += past_inc;
				counters[2] += 1;
			}
		}

		__global__ void add_int_kernel(int* p, int v) { *p += v; }
		__global__ void set_int_kernel(int* p, int v) { *p = v; }
	} // namespace

	// ---- launchers used by the C ABI and by the decoder runtime ---------------------------
	// clears n ints with a small kernel (a fill that a captured graph replays correctly)
	void launch_zero_ints(int* p, size_t n, hipStream_t s)
	{
		if (n)
		{
			zero_ints_kernel<<<dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0, s>>>(p, static_cast<int>(n));
		}
	}

	void launch_rmsnorm(const float* x, const float* w, double eps, size_t m, size_t d, float* y, hipStream_t s)
	{
		rmsnorm_kernel<<<dim3(m), dim3(d >= 4096 ? 1024 : 256), 0, s>>>(x, w, eps, static_cast<int>(d), y);
	}

	void launch_rope_table(float* cos_t, float* sin_t, size_t positions, size_t half, double base, double freq_scale,
	                       size_t pos_offset, hipStream_t s)
	{
		const size_t total = positions * half;
		rope_table_kernel<<<dim3((total + 255) / 256), dim3(256), 0, s>>>(cos_t, sin_t, static_cast<int>(positions),
		                                                                   static_cast<int>(half), base, freq_scale,
		                                                                   static_cast<int>(pos_offset));
	}

	void launch_rope(const float* x, float* y, size_t m, size_t n_heads, size_t head_dim, size_t rope_dims,
	                 const float* cos_t, const float* sin_t, hipStream_t s)
	{
		const size_t total = m * n_heads * (head_dim / 2);
		rope_kernel<<<dim3((total + 255) / 256), dim3(256), 0, s>>>(x, y, static_cast<int>(m),
		                                                             static_cast<int>(n_heads),
		                                                             static_cast<int>(head_dim),
		                                                             static_cast<int>(rope_dims), cos_t, sin_t);
	}

	void launch_kv_append(void* cache, int cache_dtype, size_t past_elems, const float* cur, size_t count, hipStream_t s)
	{
		const dim3 grid((count + 255) / 256), block(256);
		if (cache_dtype == LITENN_F16)
		{
			kv_append_kernel<uint16_t><<<grid, block, 0, s>>>(static_cast<uint16_t*>(cache), past_elems, cur, count);
		}
		else
		{
			kv_append_kernel<float><<<grid, block, 0, s>>>(static_cast<float*>(cache), past_elems, cur, count);
		}
	}

	void launch_rope_qkv_append(float* q, const float* k, const float* v, void* kcache, void* vcache, int cache_dtype,
	                            const int* past_dev, size_t m, size_t n_head, size_t n_kv_head, size_t head_dim,
	                            size_t rope_dims, const float* cos_t, const float* sin_t, hipStream_t s)
	{
		const size_t total = m * (n_head + 2 * n_kv_head) * (head_dim / 2);
		const dim3 grid((total + 255) / 256), block(256);
		if (cache_dtype == LITENN_F16)
		{
			rope_qkv_append_kernel<uint16_t><<<grid, block, 0, s>>>(
			    q, k, v, static_cast<uint16_t*>(kcache), static_cast<uint16_t*>(vcache), past_dev, static_cast<int>(m),
			    static_cast<int>(n_head), static_cast<int>(n_kv_head), static_cast<int>(head_dim),
			    static_cast<int>(rope_dims), cos_t, sin_t);
		}
		else
		{
			rope_qkv_append_kernel<float><<<grid, block, 0, s>>>(
			    q, k, v, static_cast<float*>(kcache), static_cast<float*>(vcache), past_dev, static_cast<int>(m),
			    static_cast<int>(n_head), static_cast<int>(n_kv_head), static_cast<int>(head_dim),
			    static_cast<int>(rope_dims), cos_t, sin_t);
		}
	}

	// Upper bound of the key chunks one query row is cut into, which is the grid's second extent and
	// sizes the scratch.  Only a single row is ever split (several rows already give the machine
	// enough workgroups).  It depends on the upper bound of the key length alone, so a captured
	// launch stays valid while the cache fills; the kernel itself uses as many of the grid's chunks
	// as the length it finds on the device asks for.
	size_t attn_splits(size_t m, size_t max_len, size_t n_head)
	{
		if (m != 1)
		{
			return 1;
		}
		// the kernel cuts a row into min(grid, attn_live_chunks(keys)) chunks; the grid is capped so that
		// a launch stays near a thousand workgroups, and by LITENN_HIP_ATTN_SPLITS for experiments
		static const int forced = env_int("LITENN_HIP_ATTN_SPLITS", 0);
		const size_t cap = forced > 0 ? std::min<size_t>(kMaxAttnSplits, static_cast<size_t>(forced)) : kMaxAttnSplits;
		const size_t by_len = static_cast<size_t>(attn_live_chunks(static_cast<long long>(max_len)));
		const size_t by_heads = (1024 + n_head - 1) / n_head;
		return std::max<size_t>(1, std::min<size_t>({ cap, by_len, by_heads }));
	}

	// floats of `partial` a launch with that many splits needs (and m * n_head zeroed ints of counters)
	size_t attn_partial_floats(size_t m, size_t n_head, size_t head_dim, size_t splits)
	{
		return splits > 1 ? m * n_head * splits * (head_dim + 2) : 0;
	}

	template <typename KV>
	static void launch_attn_typed(const float* q, KV* kcache, KV* vcache, size_t m, const int* past_dev,
	                              size_t past_host, size_t n_head, size_t n_kv_head, size_t head_dim, float* out,
	                              size_t splits, float* partial, int* counters, const AttnStep* step, hipStream_t s)
	{
		const dim3 grid(n_head, splits, m), block(256);
		const float scale = static_cast<float>(1.0 / sqrt(static_cast<double>(head_dim)));
		const auto aligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
		const bool fast = head_dim == 128 && aligned(q) && aligned(kcache) && aligned(vcache);
		auto kernel = step ? attn_decode_kernel<KV, true, true>
		                   : fast ? attn_decode_kernel<KV, true, false> : attn_decode_kernel<KV, false, false>;
		kernel<<<grid, block, 0, s>>>(q, kcache, vcache, out, past_dev, static_cast<int>(past_host),
		                              static_cast<int>(n_head), static_cast<int>(n_kv_head),
		                              static_cast<int>(head_dim), scale, partial, counters,
		                              step ? *step : AttnStep{});
	}

	static void launch_attn_any(const float* q, void* kcache, void* vcache, int cache_dtype, size_t m,
	                            const int* past_dev, size_t past_host, size_t n_head, size_t n_kv_head,
	                            size_t head_dim, float* out, size_t splits, float* partial, int* counters,
	                            const AttnStep* step, hipStream_t s)
	{
		if (cache_dtype == LITENN_F16)
		{
			launch_attn_typed<uint16_t>(q, static_cast<uint16_t*>(kcache), static_cast<uint16_t*>(vcache), m, past_dev,
			                            past_host, n_head, n_kv_head, head_dim, out, splits, partial, counters, step, s);
		}
		else
		{
			launch_attn_typed<float>(q, static_cast<float*>(kcache), static_cast<float*>(vcache), m, past_dev, past_host,
			                         n_head, n_kv_head, head_dim, out, splits, partial, counters, step, s);
		}
	}

	// splits > 1 needs `partial` (attn_partial_floats) and `counters` (m * n_head ints, zero before
	// the first launch; every launch leaves them zero again)
	void launch_attn_decode(const float* q, const void* kcache, const void* vcache, int cache_dtype, size_t m,
	                        const int* past_dev, size_t past_host, size_t n_head, size_t n_kv_head, size_t head_dim,
	                        float* out, size_t splits, float* partial, int* counters, hipStream_t s)
	{
		launch_attn_any(q, const_cast<void*>(kcache), const_cast<void*>(vcache), cache_dtype, m, past_dev, past_host,
		                n_head, n_kv_head, head_dim, out, splits, partial, counters, nullptr, s);
	}

	// Device address of this file's `scratch` array on the CURRENT device, looked up once per device
	// (each GPU holds its own copy at its own address).  No allocation: the array is part of the
	// code object.
	static hipError_t static_attn_scratch(float** base)
	{
		constexpr int kMaxDevices = 64;
		static std::mutex mutex;
		static float* per_device[kMaxDevices] = {};
		int dev = 0;
		hipError_t e = hipGetDevice(&dev);
		if (e != hipSuccess)
		{
			return e;
		}
		if (dev < 0 || dev >= kMaxDevices)
		{
			return hipErrorInvalidDevice;
		}
		std::lock_guard<std::mutex> lock(mutex);
		if (!per_device[dev])
		{
			void* ptr = nullptr;
			e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
			if (e != hipSuccess)
			{
				return e;
			}
			if (!ptr)
			{
				return hipErrorInvalidSymbol;
			}
			per_device[dev] = static_cast<float*>(ptr);
		}
		*base = per_device[dev];
		return hipSuccess;
	}

	// Whether a launch of that geometry fits the static scratch (always true without chunks).
	bool attn_static_fits(size_t m, size_t n_head, size_t head_dim, size_t splits)
	{
		return splits <= 1 || (attn_partial_floats(m, n_head, head_dim, splits) <= kStaticAttnPartialFloats &&
		                       m * n_head <= kStaticAttnCounters);
	}

	size_t attn_static_scratch_bytes() { return sizeof(float) * (kStaticAttnPartialFloats + kStaticAttnCounters); }

	// launch_attn_decode with the chunk triples and counters in the static scratch of the current
	// device.  The counters are cleared by a small kernel first (not a memset node: a caller may be
	// capturing), so a launch that was cut short earlier cannot leave a stale count behind.  Calls
	// that overlap on one GPU share the array and race.
	hipError_t launch_attn_decode_static(const float* q, const void* kcache, const void* vcache, int cache_dtype,
	                                     size_t m, size_t past_host, size_t n_head, size_t n_kv_head, size_t head_dim,
	                                     float* out, size_t splits, hipStream_t s)
	{
		float* partial = nullptr;
		int* counters = nullptr;
		if (splits > 1)
		{
			float* base = nullptr;
			const hipError_t e = static_attn_scratch(&base);
			if (e != hipSuccess)
			{
				return e;
			}
			partial = base;
			counters = reinterpret_cast<int*>(base + kStaticAttnPartialFloats);
			const int n = static_cast<int>(m * n_head);
			zero_ints_kernel<<<dim3((n + 255) / 256), dim3(256), 0, s>>>(counters, n);
		}
		launch_attn_decode(q, kcache, vcache, cache_dtype, m, nullptr, past_host, n_head, n_kv_head, head_dim, out,
		                   splits, partial, counters, s);
		return hipSuccess;
	}

	// Whether one new row's rotation, cache append and attention can run as a single launch.
	bool attn_step_fusable(const float* q, const float* k, const float* v, const void* kcache, const void* vcache,
	                       size_t head_dim, size_t rope_dims, const float* cos_t, const float* sin_t)
	{
		const auto aligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
		return head_dim == 128 && rope_dims % 8 == 0 && rope_dims <= head_dim && aligned(q) && aligned(k) &&
		       aligned(v) && aligned(kcache) && aligned(vcache) && aligned(cos_t) && aligned(sin_t);
	}

	// rope(q), rope(k) -> cache, v -> cache, attention of the new row: one launch.  Position = *past_dev.
	void launch_attn_step(const float* q, const float* k, const float* v, void* kcache, void* vcache, int cache_dtype,
	                      const int* past_dev, size_t n_head, size_t n_kv_head, size_t head_dim, size_t rope_dims,
	                      const float* cos_t, const float* sin_t, float* out, size_t splits, float* partial,
	                      int* counters, hipStream_t s)
	{
		const AttnStep step{ k, v, cos_t, sin_t, static_cast<int>(rope_dims) };
		launch_attn_any(q, kcache, vcache, cache_dtype, 1, past_dev, 0, n_head, n_kv_head, head_dim, out, splits,
		                partial, counters, &step, s);
	}

	// Attention of m rows over `keys` cached rows with the reference layer's options; operands as in
	// launch_attn_decode, mask [m, keys] and sinks [n_head] in f32 on the device or null.
	void launch_attn_ext(const float* q, const void* kcache, const void* vcache, int cache_dtype, size_t m, size_t keys,
	                     size_t n_head, size_t n_kv_head, size_t head_dim, double scale, double max_bias,
	                     double logit_softcap, const float* mask, const float* sinks, bool causal, size_t key_offset,
	                     size_t query_offset, float* out, hipStream_t s)
	{
		AttnExt x;
		const double score_scale = logit_softcap != 0.0 ? scale / logit_softcap : scale;
		x.mask = mask;
		x.sinks = sinks;
		x.score_scale = static_cast<float>(score_scale);
		x.softcap = static_cast<float>(logit_softcap);
		x.apply_scale = (scale != 1.0 || logit_softcap != 0.0) && score_scale != 1.0;
		x.apply_cap = logit_softcap != 1.0;
		x.max_bias = max_bias;
		x.causal = causal;
		x.key_offset = static_cast<long long>(key_offset);
		x.query_offset = static_cast<long long>(query_offset);
		x.keys = static_cast<int>(keys);
		const dim3 grid(n_head, m), block(256);
		if (cache_dtype == LITENN_F16)
		{
			attn_ext_kernel<uint16_t><<<grid, block, 0, s>>>(q, static_cast<const uint16_t*>(kcache),
			                                                 static_cast<const uint16_t*>(vcache), out,
			                                                 static_cast<int>(n_head), static_cast<int>(n_kv_head),
			                                                 static_cast<int>(head_dim), x);
		}
		else
		{
			attn_ext_kernel<float><<<grid, block, 0, s>>>(q, static_cast<const float*>(kcache),
			                                              static_cast<const float*>(vcache), out,
			                                              static_cast<int>(n_head), static_cast<int>(n_kv_head),
			                                              static_cast<int>(head_dim), x);
		}
	}

	void launch_silu_mul(const float* gate, const float* up, float* y, size_t n, hipStream_t s)
	{
		silu_mul_kernel<<<dim3((n + 255) / 256), dim3(256), 0, s>>>(gate, up, y, n);
	}

	void launch_argmax(const float* x, size_t rows, size_t n, int32_t* out, hipStream_t s)
	{
		argmax_kernel<<<dim3(rows), dim3(1024), 0, s>>>(x, static_cast<int>(n), out);
	}

	// bytes of scratch launch_argmax_step needs for a row of n values
	size_t argmax_step_scratch_bytes(size_t n)
	{
		return ((n + kArgmaxChunk - 1) / kArgmaxChunk) * (sizeof(float) + sizeof(int));
	}

	// next = arg-max of x[0 .. n) (first maximal index); out[counters[1]++] = next (when out is given);
	// counters[0] += past_inc
	void launch_argmax_step(const float* x, size_t n, void* scratch, int32_t* next, int* counters, int past_inc,
	                        int32_t* out, hipStream_t s)
	{
		const int blocks = static_cast<int>((n + kArgmaxChunk - 1) / kArgmaxChunk);
		float* pv = static_cast<float*>(scratch);
		int* pi = reinterpret_cast<int*>(pv + blocks);
		argmax_partial_kernel<<<dim3(blocks), dim3(256), 0, s>>>(x, static_cast<int>(n), pv, pi);
		argmax_merge_step_kernel<<<dim3(1), dim3(64), 0, s>>>(pv, pi, blocks, next, counters, past_inc, out);
	}

	void launch_add_int(int* p, int v, hipStream_t s) { add_int_kernel<<<1, 1, 0, s>>>(p, v); }
	void launch_set_int(int* p, int v, hipStream_t s) { set_int_kernel<<<1, 1, 0, s>>>(p, v); }
} // namespace litenn_hip
