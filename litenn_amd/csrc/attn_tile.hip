// litenn-hip: causal attention of many query rows on the matrix cores (prompt pass).
//
// The reference lowers attention to MatMul -> scale -> mask -> softmax -> MatMul per head
// (tools/gguf/LLaMABuilder.cpp:350-404, src/LiteNN/Layer/FlashAttnExt.h:100-228,
// src/LiteNN/Layer/CausalMask.h:16-56).  For one new row that is a bandwidth problem and the
// row kernel in glue.hip streams the cache once.  For a prompt of M rows the same row kernel
// re-reads every key once per row; here a workgroup owns 64 consecutive query rows of one
// head, walks the keys in tiles of 64 staged through LDS and does both contractions with
// v_mfma_f32_16x16x32_f16, softmax kept online in f32.  The workgroup is two halves of four
// wavefronts: one takes the even key tiles, the other the odd ones, each with its own LDS
// buffers, so every SIMD holds two wavefronts in different phases; the halves' (max, sum,
// output) triples are merged once at the end.
//
//   S^T[key, q]  = K[key, :] . Q[q, :]        A = key tile (row-major in LDS), B = Q (registers)
//   O^T[d, q]   += V^T[d, key] . P^T[key, q]  A = value tile staged dimension-major, B = P
//
// Computing the transposed products keeps the query in the lane index of every result, so
// the softmax weights leave the first contraction in exactly the register layout the second
// one wants as its B operand (the order in which keys enter the second contraction is chosen
// to match), and the running maximum / sum / rescale of a query live in the lanes that hold
// its outputs.  Operands are fp16 (the cache already is; q * 1/sqrt(d) and the softmax
// weights are rounded once), accumulation is f32.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>

#include "common.hpp"
#include "fetch_model.hpp"

namespace litenn_hip
{
	namespace
	{
		typedef _Float16 half8 __attribute__((ext_vector_type(8)));
		typedef _Float16 half4 __attribute__((ext_vector_type(4)));
		typedef _Float16 half2v __attribute__((ext_vector_type(2)));
		typedef float float2v __attribute__((ext_vector_type(2)));
		typedef float floatx4 __attribute__((ext_vector_type(4)));
		typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

		constexpr int kQTile = 64;     // query rows of a workgroup (16 per wavefront)
		constexpr int kKeyTile = 64;   // keys staged per step
		constexpr int kDim = 128;      // head width this kernel is written for
		constexpr int kKStride = 136;  // halves between staged key rows: 16 rows x 16 bytes fall on 64 distinct banks
		constexpr int kVtStride = 72;  // halves between staged value columns (dimension-major)

		__device__ __forceinline__ half2v pack2(float a, float b)
		{
			const float2v f = { a, b };
			return __builtin_convertvector(f, half2v); // v_cvt_pk_f16_f32
		}

		constexpr int kTileHalves = kKeyTile * kKStride + kDim * kVtStride; // one half's key + value buffers
		constexpr size_t kAttnTileLds = 2 * kTileHalves * sizeof(_Float16);

		__global__ __launch_bounds__(512) void attn_tile_kernel(const float* __restrict__ q,
		                                                         const uint16_t* __restrict__ kcache,
		                                                         const uint16_t* __restrict__ vcache,
		                                                         float* __restrict__ out,
		                                                         const int* __restrict__ past_dev, int past_host, int m,
		                                                         int n_head, int n_kv_head, float scale)
		{
			extern __shared__ __attribute__((aligned(16))) _Float16 attn_lds[];
			const int part = threadIdx.x >> 8; // which half of the workgroup: key tiles part, part + 2, ...
			_Float16* const k_lds = attn_lds + part * kTileHalves;
			_Float16* const vt_lds = k_lds + kKeyTile * kKStride;
			const int tid = threadIdx.x & 255;
			const int lane = tid & 63;
			const int wave = tid >> 6;
			const int j = lane & 15; // query (B operand / result column), key or dimension row (A operand)
			const int g = lane >> 4;
			// heads are dealt to the XCDs in runs (XCD x: heads [x n_head / 8, (x + 1) n_head / 8)), so that
			// the query heads of one KV head read its keys and values through one L2
			const int h = (n_head & 7) == 0 ? static_cast<int>(blockIdx.x & 7) * (n_head >> 3) + static_cast<int>(blockIdx.x >> 3)
			                                : static_cast<int>(blockIdx.x);
			const int q_tiles = gridDim.y;
			const int tile = q_tiles - 1 - static_cast<int>(blockIdx.y); // the longest key runs start first
			const int past = past_dev ? *past_dev : past_host;
			const int kvh = h / (n_head / n_kv_head);
			const size_t kvw = static_cast<size_t>(n_kv_head) * kDim;
			const uint16_t* kbase = kcache + static_cast<size_t>(kvh) * kDim;
			const uint16_t* vbase = vcache + static_cast<size_t>(kvh) * kDim;

			const int q_first = tile * kQTile;
			const int kv_len = fetch::attn_tile_kv_len(past, q_first, kQTile, m); // keys any row of this tile may see
			const int n_key_tiles = (kv_len + kKeyTile - 1) / kKeyTile;
			const int n_steps = (n_key_tiles + 1) >> 1; // both halves make the same number of steps

			// the wavefront's 16 queries as the B operand of the first contraction, scaled and rounded once
			const int my_q = q_first + 16 * wave + j;
			const int my_q_clamped = min(my_q, m - 1);
			const float* q_row = q + (static_cast<size_t>(my_q_clamped) * n_head + h) * kDim;
			half8 q_frag[4];
#pragma unroll
			for (int st = 0; st < 4; ++st)
			{
				const float4 a = *reinterpret_cast<const float4*>(q_row + 32 * st + 8 * g);
				const float4 b = *reinterpret_cast<const float4*>(q_row + 32 * st + 8 * g + 4);
				const half2v p0 = pack2(a.x * scale, a.y * scale), p1 = pack2(a.z * scale, a.w * scale);
				const half2v p2 = pack2(b.x * scale, b.y * scale), p3 = pack2(b.z * scale, b.w * scale);
				q_frag[st] = half8{ p0.x, p0.y, p1.x, p1.y, p2.x, p2.y, p3.x, p3.y };
			}
			const int my_limit = past + my_q_clamped; // last key position this query sees

			// staging: keys row-major (thread = 16-byte piece of a key row, consecutive lanes consecutive
			// pieces), values dimension-major (thread = one key, 64 consecutive bytes of its row)
			u32x4 k_reg[4], v_reg[4];
			const int v_key = tid & 63;
			const int v_part0 = (tid >> 6) * 4;
			const auto fetch = [&](int kt) {
#pragma unroll
				for (int i = 0; i < 4; ++i)
				{
					const int c = tid + 256 * i;
					const int key = fetch::attn_tile_key(kt, kKeyTile, c >> 4, kv_len);
					k_reg[i] = *reinterpret_cast<const u32x4*>(kbase + static_cast<size_t>(key) * kvw + (c & 15) * 8);
				}
				const int key = fetch::attn_tile_key(kt, kKeyTile, v_key, kv_len);
				const uint16_t* vr = vbase + static_cast<size_t>(key) * kvw + v_part0 * 8;
#pragma unroll
				for (int i = 0; i < 4; ++i)
				{
					v_reg[i] = *reinterpret_cast<const u32x4*>(vr + 8 * i);
				}
			};
			const auto stage = [&]() {
#pragma unroll
				for (int i = 0; i < 4; ++i)
				{
					const int c = tid + 256 * i;
					*reinterpret_cast<u32x4*>(&k_lds[(c >> 4) * kKStride + (c & 15) * 8]) = k_reg[i];
				}
				uint16_t* vt = reinterpret_cast<uint16_t*>(vt_lds);
#pragma unroll
				for (int i = 0; i < 4; ++i)
				{
					const uint32_t w[4] = { v_reg[i].x, v_reg[i].y, v_reg[i].z, v_reg[i].w };
#pragma unroll
					for (int e = 0; e < 4; ++e)
					{
						const int d = (v_part0 + i) * 8 + 2 * e;
						vt[d * kVtStride + v_key] = static_cast<uint16_t>(w[e] & 0xffffu);
						vt[(d + 1) * kVtStride + v_key] = static_cast<uint16_t>(w[e] >> 16);
					}
				}
			};

			floatx4 o[8];
#pragma unroll
			for (int db = 0; db < 8; ++db)
			{
				o[db] = floatx4{ 0.0f, 0.0f, 0.0f, 0.0f };
			}
			float run_m = -INFINITY, run_l = 0.0f; // run_l: this lane's share of the sum

			fetch(min(part, n_key_tiles - 1));
			for (int step = 0; step < n_steps; ++step)
			{
				const int kt = 2 * step + part;
				// a half whose last step has no tile left stages a valid one again and masks all of it
				const int limit = kt < n_key_tiles ? my_limit : -1;
				__syncthreads(); // the previous tile has been consumed
				stage();
				fetch(min(kt + 2, n_key_tiles - 1)); // no branch around the loads: past the end a tile is re-read
				__syncthreads();

				// S^T: four blocks of 16 keys; lane (j, g) gets keys 16 b + 4 g + 0..3 of query j
				floatx4 s[4];
#pragma unroll
				for (int b = 0; b < 4; ++b)
				{
					s[b] = floatx4{ 0.0f, 0.0f, 0.0f, 0.0f };
#pragma unroll
					for (int st = 0; st < 4; ++st)
					{
						const half8 a = *reinterpret_cast<const half8*>(&k_lds[(16 * b + j) * kKStride + 32 * st + 8 * g]);
						s[b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, q_frag[st], s[b], 0, 0, 0);
					}
				}
				// causal mask, tile maximum of the query (its keys are spread over four lanes)
				const int key0 = kt * kKeyTile + 4 * g;
				float tile_m = -INFINITY;
				float sv[4][4];
#pragma unroll
				for (int b = 0; b < 4; ++b)
				{
					const float v4[4] = { s[b].x, s[b].y, s[b].z, s[b].w };
#pragma unroll
					for (int r = 0; r < 4; ++r)
					{
						sv[b][r] = (key0 + 16 * b + r <= limit) ? v4[r] : -INFINITY;
						tile_m = fmaxf(tile_m, sv[b][r]);
					}
				}
				tile_m = fmaxf(tile_m, __shfl_xor(tile_m, 16, 64));
				tile_m = fmaxf(tile_m, __shfl_xor(tile_m, 32, 64));
				// the odd half may not have seen a visible key yet: exponents then take 0 as the maximum
				const float new_m = fmaxf(run_m, tile_m);
				const float ref_m = new_m == -INFINITY ? 0.0f : new_m;
				const float corr = __expf(run_m - ref_m);
				run_m = new_m;
				float sum = 0.0f;
				half8 p_frag[2];
#pragma unroll
				for (int ks = 0; ks < 2; ++ks)
				{
					float p[8];
#pragma unroll
					for (int r = 0; r < 4; ++r)
					{
						p[r] = __expf(sv[2 * ks][r] - ref_m);
						p[4 + r] = __expf(sv[2 * ks + 1][r] - ref_m);
					}
#pragma unroll
					for (int e = 0; e < 8; ++e)
					{
						sum += p[e];
					}
					const half2v p0 = pack2(p[0], p[1]), p1 = pack2(p[2], p[3]);
					const half2v p2 = pack2(p[4], p[5]), p3 = pack2(p[6], p[7]);
					p_frag[ks] = half8{ p0.x, p0.y, p1.x, p1.y, p2.x, p2.y, p3.x, p3.y };
				}
				run_l = fmaf(run_l, corr, sum);
				// O^T: eight blocks of 16 dimensions; contraction index 8 g + e of step ks stands for
				// key 16 (2 ks) + 4 g + e (e < 4) and key 16 (2 ks + 1) + 4 g + e - 4 (e >= 4)
#pragma unroll
				for (int db = 0; db < 8; ++db)
				{
					o[db] *= corr;
#pragma unroll
					for (int ks = 0; ks < 2; ++ks)
					{
						const _Float16* col = &vt_lds[(16 * db + j) * kVtStride + 32 * ks + 4 * g];
						const half4 lo = *reinterpret_cast<const half4*>(col);
						const half4 hi = *reinterpret_cast<const half4*>(col + 16);
						const half8 a = half8{ lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w };
						o[db] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, p_frag[ks], o[db], 0, 0, 0);
					}
				}
			}

			run_l += __shfl_xor(run_l, 16, 64);
			run_l += __shfl_xor(run_l, 32, 64);
			// the odd half hands its triple to the even half through its own (now idle) buffers
			__syncthreads();
			float* const xch = reinterpret_cast<float*>(attn_lds + kTileHalves);
			if (part == 1)
			{
#pragma unroll
				for (int db = 0; db < 8; ++db)
				{
					*reinterpret_cast<floatx4*>(xch + (db * 256 + tid) * 4) = o[db];
				}
				xch[8 * 1024 + tid] = run_m;
				xch[8 * 1024 + 256 + tid] = run_l;
			}
			__syncthreads();
			if (part == 1)
			{
				return;
			}
			{
				const float other_m = xch[8 * 1024 + tid], other_l = xch[8 * 1024 + 256 + tid];
				const float all_m = fmaxf(run_m, other_m); // finite: the even half has seen key 0
				const float w0 = __expf(run_m - all_m), w1 = other_m == -INFINITY ? 0.0f : __expf(other_m - all_m);
				run_l = run_l * w0 + other_l * w1;
#pragma unroll
				for (int db = 0; db < 8; ++db)
				{
					const floatx4 t = *reinterpret_cast<const floatx4*>(xch + (db * 256 + tid) * 4);
					o[db] = o[db] * w0 + t * w1;
				}
			}
			if (my_q < m)
			{
				const float inv = 1.0f / run_l;
				float* dst = out + (static_cast<size_t>(my_q) * n_head + h) * kDim + 4 * g;
#pragma unroll
				for (int db = 0; db < 8; ++db)
				{
					*reinterpret_cast<float4*>(dst + 16 * db) =
					    make_float4(o[db].x * inv, o[db].y * inv, o[db].z * inv, o[db].w * inv);
				}
			}
		}
	} // namespace

	// Causal attention of m rows (positions past .. past + m - 1) with fp16 operands on the matrix
	// cores.  Returns false, launching nothing, when the shape is not the one the kernel is written
	// for (128-wide heads, fp16 cache, 16-byte aligned buffers); the caller then uses the row kernel.
	bool launch_attn_tile(const float* q, const void* kcache, const void* vcache, int cache_dtype, size_t m,
	                      const int* past_dev, size_t past_host, size_t n_head, size_t n_kv_head, size_t head_dim,
	                      float* out, hipStream_t s)
	{
		const auto aligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
		if (cache_dtype != LITENN_F16 || head_dim != kDim || m == 0 || m > 0x3fffffffu || n_kv_head == 0 ||
		    n_head % n_kv_head != 0 || n_head > 65535 || !aligned(q) || !aligned(kcache) || !aligned(vcache) ||
		    !aligned(out))
		{
			return false;
		}
		const size_t q_tiles = (m + kQTile - 1) / kQTile;
		if (q_tiles > 65535)
		{
			return false;
		}
		const float scale = static_cast<float>(1.0 / sqrt(static_cast<double>(head_dim)));
		allow_dynamic_lds(reinterpret_cast<const void*>(&attn_tile_kernel), kAttnTileLds);
		attn_tile_kernel<<<dim3(n_head, q_tiles), dim3(512), kAttnTileLds, s>>>(
		    q, static_cast<const uint16_t*>(kcache), static_cast<const uint16_t*>(vcache), out, past_dev,
		    static_cast<int>(past_host), static_cast<int>(m), static_cast<int>(n_head), static_cast<int>(n_kv_head),
		    scale);
		return true;
	}
} // namespace litenn_hip
