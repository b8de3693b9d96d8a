// Batched quantised matmul for prefill (M >= 16 activation rows):
//   Y[M, N] = X[M, K] . deq(W)[N, K]^T  (+ residual)
// the value AddLinear produces for a sequence after the lowering's dequantise + transpose
// (tools/gguf/LLaMABuilder.cpp:144-150,225-230; src/LiteNN/Layer/Linear.h:67-95), computed on
// the matrix cores: weights are decoded from their GGUF blocks straight into MFMA operand
// registers as fp16 (one rounding of the f32 value d*q [- dmin*m]), activations are rounded to
// fp16 once by a small pre-pass, products accumulate in f32 (v_mfma_f32_16x16x32_f16).
// Error against the f32 reference: two independent fp16 roundings per product, about 4e-4
// relative L2 on the output.  Each activation row is scaled by a power of two into the fp16
// range first (and its results scaled back), so the range of the activations does not matter;
// LITENN_HIP_MATMUL_PRECISE selects the f32 GEMV path instead.
//
// Work split: a workgroup (4 wavefronts) owns 64 * NG weight rows and BM activation rows; a
// wavefront owns NG groups of 16 weight rows and walks K in chunks of 256 (one K-quant
// super-block, eight 32-element blocks).  Lane (r, g) = (lane % 16, lane / 16) decodes 64 of
// the 256 elements of row r of each of its groups per chunk, eight per MFMA step, in whatever
// order is cheapest for the format; the activation operand is read from LDS in the same order,
// so the contraction is complete and no weight byte is decoded twice or staged in LDS.
// The weights of chunk c + 1 are loaded while chunk c is multiplied; the fp16 activation tile
// of the next chunk is staged into the second half of a double-buffered LDS tile.
#include "common.hpp"

#include <algorithm>

namespace litenn_hip
{
	namespace
	{
		typedef _Float16 half8 __attribute__((ext_vector_type(8)));
		typedef _Float16 half2v __attribute__((ext_vector_type(2)));
		typedef float float2v __attribute__((ext_vector_type(2)));
		typedef float floatx4 __attribute__((ext_vector_type(4)));
		typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
		typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

		constexpr int kChunk = 256;          // K elements per step of the outer loop
		constexpr int kTileStride = 256 + 8; // halves per activation row in LDS (pad: 4 banks per row)

		__device__ __forceinline__ uint32_t pack_f16(float a, float b)
		{
			const float2v f = { a, b };
			const half2v h = __builtin_convertvector(f, half2v); // v_cvt_pk_f16_f32, round to nearest even
			return __builtin_bit_cast(uint32_t, h);
		}

		// unaligned little-endian reads from global memory (blocks are only 2-byte aligned)
		__device__ __forceinline__ uint32_t ld_u32(const uint8_t* p)
		{
			typedef uint32_t u32_a2 __attribute__((aligned(2)));
			return *reinterpret_cast<const u32_a2*>(p);
		}
		__device__ __forceinline__ uint32_t ld_u16(const uint8_t* p)
		{
			return *reinterpret_cast<const uint16_t*>(p);
		}

		// ---- per-format decoders -----------------------------------------------------------
		// Raw   : the bytes lane (r, g) needs from one 256-element chunk of its row
		// Scale : per-chunk factors derived once from Raw
		// frag  : the 8 fp16 values of MFMA step s (0..7) as 4 packed dwords
		// koff  : offsets (in elements, within the chunk) of the two runs of 4 activations
		//         that pair with frag(s): elements 0..3 <-> k0 .. k0+3, 4..7 <-> k1 .. k1+3

		struct Q4_0Frag
		{
			static constexpr int kChunkBytes = 8 * 18;
			struct Raw { uint32_t w[9]; }; // blocks 2g and 2g+1: 36 bytes
			struct Scale { float d0, d1; };
			static __device__ __forceinline__ Raw load(const uint8_t* chunk, int g)
			{
				Raw r;
				const uint8_t* p = chunk + 36 * g; // 4-byte aligned: rows are 16-byte aligned
#pragma unroll
				for (int i = 0; i < 9; ++i)
				{
					r.w[i] = ld_u32(p + 4 * i);
				}
				return r;
			}
			static __device__ __forceinline__ Scale prep(const Raw& r, int)
			{
				return { f16_bits_to_f32(r.w[0]), f16_bits_to_f32(r.w[4] >> 16) };
			}
			// dword t (0..3) of the nibble bytes of block b (0/1)
			static __device__ __forceinline__ uint32_t qs(const Raw& r, int b, int t)
			{
				if (b == 0)
				{
					return (r.w[t] >> 16) | (r.w[t + 1] << 16); // bytes 2 + 4t ..
				}
				return r.w[5 + t]; // bytes 20 + 4t ..
			}
			static __device__ __forceinline__ void frag(const Raw& r, const Scale& sc, int s, uint32_t (&out)[4])
			{
				const int b = s >> 2, t = s & 3;
				const uint32_t v = qs(r, b, t);
				const float d = b == 0 ? sc.d0 : sc.d1;
				float f[8];
#pragma unroll
				for (int e = 0; e < 4; ++e)
				{
					f[e] = (static_cast<float>((v >> (8 * e)) & 0xFu) - 8.0f) * d;         // element 4t + e
					f[4 + e] = (static_cast<float>((v >> (8 * e + 4)) & 0xFu) - 8.0f) * d; // element 16 + 4t + e
				}
#pragma unroll
				for (int i = 0; i < 4; ++i)
				{
					out[i] = pack_f16(f[2 * i], f[2 * i + 1]);
				}
			}
			static __device__ __forceinline__ void koff(int g, int s, int& k0, int& k1)
			{
				const int base = 32 * (2 * g + (s >> 2)) + 4 * (s & 3);
				k0 = base;
				k1 = base + 16;
			}
		};

		struct Q8_0Frag
		{
			static constexpr int kChunkBytes = 8 * 34;
			struct Raw { uint32_t w[17]; }; // blocks 2g and 2g+1: 68 bytes
			struct Scale { float d0, d1; };
			static __device__ __forceinline__ Raw load(const uint8_t* chunk, int g)
			{
				Raw r;
				const uint8_t* p = chunk + 68 * g;
#pragma unroll
				for (int i = 0; i < 17; ++i)
				{
					r.w[i] = ld_u32(p + 4 * i);
				}
				return r;
			}
			static __device__ __forceinline__ Scale prep(const Raw& r, int)
			{
				return { f16_bits_to_f32(r.w[0]), f16_bits_to_f32(r.w[8] >> 16) };
			}
			static __device__ __forceinline__ void frag(const Raw& r, const Scale& sc, int s, uint32_t (&out)[4])
			{
				const int b = s >> 2, t = s & 3; // elements 8t .. 8t+7 of block b
				uint32_t lo, hi;
				if (b == 0)
				{
					// quants start at byte 2
					lo = (r.w[2 * t] >> 16) | (r.w[2 * t + 1] << 16);
					hi = (r.w[2 * t + 1] >> 16) | (r.w[2 * t + 2] << 16);
				}
				else
				{
					// block 1 starts at byte 34, its quants at byte 36 = dword 9
					lo = r.w[9 + 2 * t];
					hi = r.w[10 + 2 * t];
				}
				const float d = b == 0 ? sc.d0 : sc.d1;
				float f[8];
#pragma unroll
				for (int e = 0; e < 4; ++e)
				{
					f[e] = static_cast<float>(static_cast<int8_t>(lo >> (8 * e))) * d;
					f[4 + e] = static_cast<float>(static_cast<int8_t>(hi >> (8 * e))) * d;
				}
#pragma unroll
				for (int i = 0; i < 4; ++i)
				{
					out[i] = pack_f16(f[2 * i], f[2 * i + 1]);
				}
			}
			static __device__ __forceinline__ void koff(int g, int s, int& k0, int& k1)
			{
				k0 = 32 * (2 * g + (s >> 2)) + 8 * (s & 3);
				k1 = k0 + 4;
			}
		};

		struct Q4_KFrag
		{
			static constexpr int kChunkBytes = 144;
			struct Raw { u32x4 h; uint32_t q[8]; }; // header (d, dmin, 12 scale bytes) + the 32 nibble bytes of group g
			struct Scale { float s0, m0, s1, m1; }; // d*sc and dmin*m of sub-blocks 2g and 2g+1
			static __device__ __forceinline__ Raw load(const uint8_t* chunk, int g)
			{
				Raw r;
				r.h = *reinterpret_cast<const u32x4*>(chunk);
				const u32x4 a = *reinterpret_cast<const u32x4*>(chunk + 16 + 32 * g);
				const u32x4 b = *reinterpret_cast<const u32x4*>(chunk + 32 + 32 * g);
				r.q[0] = a.x, r.q[1] = a.y, r.q[2] = a.z, r.q[3] = a.w;
				r.q[4] = b.x, r.q[5] = b.y, r.q[6] = b.z, r.q[7] = b.w;
				return r;
			}
			static __device__ __forceinline__ uint32_t scale_byte(const u32x4& h, int i) // byte i of scales[12]
			{
				const uint32_t w = i < 4 ? h.y : (i < 8 ? h.z : h.w);
				return (w >> (8 * (i & 3))) & 0xffu;
			}
			static __device__ __forceinline__ void scale_min(const u32x4& h, int j, float& sc, float& mn)
			{
				uint32_t s, m;
				if (j < 4)
				{
					s = scale_byte(h, j) & 63u;
					m = scale_byte(h, j + 4) & 63u;
				}
				else
				{
					s = (scale_byte(h, j + 4) & 0xFu) | ((scale_byte(h, j - 4) >> 6) << 4);
					m = (scale_byte(h, j + 4) >> 4) | ((scale_byte(h, j) >> 6) << 4);
				}
				sc = static_cast<float>(s);
				mn = static_cast<float>(m);
			}
			static __device__ __forceinline__ Scale prep(const Raw& r, int g)
			{
				const float d = f16_bits_to_f32(r.h.x), dmin = f16_bits_to_f32(r.h.x >> 16);
				float s0, m0, s1, m1;
				scale_min(r.h, 2 * g, s0, m0);
				scale_min(r.h, 2 * g + 1, s1, m1);
				return { d * s0, dmin * m0, d * s1, dmin * m1 };
			}
			static __device__ __forceinline__ void frag(const Raw& r, const Scale& sc, int s, uint32_t (&out)[4])
			{
				const uint32_t v = r.q[s];
				float f[8];
#pragma unroll
				for (int e = 0; e < 4; ++e)
				{
					f[e] = static_cast<float>((v >> (8 * e)) & 0xFu) * sc.s0 - sc.m0;         // sub-block 2g, element 4s + e
					f[4 + e] = static_cast<float>((v >> (8 * e + 4)) & 0xFu) * sc.s1 - sc.m1; // sub-block 2g+1
				}
#pragma unroll
				for (int i = 0; i < 4; ++i)
				{
					out[i] = pack_f16(f[2 * i], f[2 * i + 1]);
				}
			}
			static __device__ __forceinline__ void koff(int g, int s, int& k0, int& k1)
			{
				k0 = 64 * g + 4 * s;
				k1 = k0 + 32;
			}
		};

		struct Q6_KFrag
		{
			static constexpr int kChunkBytes = 210;
			// lane g = 2h + j covers l in [16j, 16j + 16) of half h: 16 bytes of each ql half-row,
			// 16 bytes of qh, the four scales 8h + j + 2i and d
			struct Raw { uint32_t la[4], lb[4], qh[4]; uint32_t sc[4]; uint32_t d; };
			struct Scale { float s[4]; };
			static __device__ __forceinline__ Raw load(const uint8_t* chunk, int g)
			{
				const int h = g >> 1, j = g & 1;
				Raw r;
				const uint8_t* ql = chunk + 64 * h + 16 * j;
				const uint8_t* qh = chunk + 128 + 32 * h + 16 * j;
#pragma unroll
				for (int i = 0; i < 4; ++i)
				{
					r.la[i] = ld_u32(ql + 4 * i);
					r.lb[i] = ld_u32(ql + 32 + 4 * i);
					r.qh[i] = ld_u32(qh + 4 * i);
				}
				const uint8_t* sc = chunk + 192 + 8 * h + j;
#pragma unroll
				for (int i = 0; i < 4; ++i)
				{
					r.sc[i] = sc[2 * i];
				}
				r.d = ld_u16(chunk + 208);
				return r;
			}
			static __device__ __forceinline__ Scale prep(const Raw& r, int)
			{
				const float d = f16_bits_to_f32(r.d);
				Scale s;
#pragma unroll
				for (int i = 0; i < 4; ++i)
				{
					s.s[i] = d * static_cast<float>(static_cast<int8_t>(r.sc[i]));
				}
				return s;
			}
			// step s: quarter i = s / 2 (q1..q4 of the reference decoder), elements 8 (s % 2) .. + 7 of the
			// lane's 16
			static __device__ __forceinline__ void frag(const Raw& r, const Scale& sc, int s, uint32_t (&out)[4])
			{
				const int i = s >> 1, u = s & 1;
				float f[8];
#pragma unroll
				for (int w = 0; w < 2; ++w)
				{
					const uint32_t lw = (i & 1) ? r.lb[2 * u + w] : r.la[2 * u + w];
					const uint32_t hw = r.qh[2 * u + w];
#pragma unroll
					for (int e = 0; e < 4; ++e)
					{
						const uint32_t lo = (lw >> (8 * e + (i >= 2 ? 4 : 0))) & 0xFu;
						const uint32_t hi = (hw >> (8 * e + 2 * i)) & 3u;
						const int q = static_cast<int>(lo | (hi << 4)) - 32;
						f[4 * w + e] = static_cast<float>(q) * sc.s[i];
					}
				}
#pragma unroll
				for (int k = 0; k < 4; ++k)
				{
					out[k] = pack_f16(f[2 * k], f[2 * k + 1]);
				}
			}
			static __device__ __forceinline__ void koff(int g, int s, int& k0, int& k1)
			{
				const int h = g >> 1, j = g & 1;
				k0 = 128 * h + 32 * (s >> 1) + 16 * j + 8 * (s & 1);
				k1 = k0 + 4;
			}
		};

		// ---- activations to fp16 -------------------------------------------------------------------
		// One workgroup per row.  Every row is scaled by a power of two so that its largest magnitude
		// lands in [2^14, 2^15): nothing overflows fp16 whatever the activations' range, small rows keep
		// full fp16 precision, and the scaling itself is exact; the GEMM multiplies the row's results by
		// the inverse factor.  Rows m .. m_pad - 1 are zero padding.
		__global__ __launch_bounds__(256) void to_half_kernel(const float* __restrict__ x, _Float16* __restrict__ xh,
		                                                       float* __restrict__ unscale, int m, int k)
		{
			__shared__ float red[4];
			const int row = blockIdx.x;
			_Float16* dst = xh + static_cast<size_t>(row) * k;
			if (row >= m)
			{
				for (int i = threadIdx.x * 8; i < k; i += 256 * 8)
				{
					*reinterpret_cast<u32x4*>(dst + i) = u32x4{ 0u, 0u, 0u, 0u };
				}
				if (threadIdx.x == 0)
				{
					unscale[row] = 0.0f;
				}
				return;
			}
			const float* src = x + static_cast<size_t>(row) * k;
			float mx = 0.0f;
			for (int i = threadIdx.x * 4; i < k; i += 256 * 4)
			{
				const float4 v = *reinterpret_cast<const float4*>(src + i);
				mx = fmaxf(fmaxf(mx, fmaxf(fabsf(v.x), fabsf(v.y))), fmaxf(fabsf(v.z), fabsf(v.w)));
			}
			mx = wave_max(mx);
			if ((threadIdx.x & 63) == 0)
			{
				red[threadIdx.x >> 6] = mx;
			}
			__syncthreads();
			mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
			int shift = 0; // xh = x * 2^shift
			if (mx > 0.0f && mx <= 3.0e38f)
			{
				shift = 14 - ilogbf(mx);
			}
			for (int i = threadIdx.x * 4; i < k; i += 256 * 4)
			{
				const float4 v = *reinterpret_cast<const float4*>(src + i);
				u32x2 out;
				out.x = pack_f16(ldexpf(v.x, shift), ldexpf(v.y, shift));
				out.y = pack_f16(ldexpf(v.z, shift), ldexpf(v.w, shift));
				*reinterpret_cast<u32x2*>(dst + i) = out;
			}
			if (threadIdx.x == 0)
			{
				unscale[row] = ldexpf(1.0f, -shift);
			}
		}

		// ---- the GEMM ---------------------------------------------------------------------------
		// grid (ceil(N / (64 NG)), ceil(M_pad / BM)); block 256.
		template <typename F, int BM, int NG>
		__global__ __launch_bounds__(256) void gemm_q_kernel(const uint8_t* __restrict__ w, const _Float16* __restrict__ xh,
		                                                      const float* __restrict__ unscale, float* __restrict__ y,
		                                                      const float* __restrict__ residual, int n, int k, int m,
		                                                      int m_pad, size_t row_bytes)
		{
			constexpr int MT = BM / 16;                      // 16-row activation tiles
			constexpr int kTileHalves = BM * kTileStride;    // one buffer of the LDS tile
			constexpr int kStageLoads = (BM * 32) / 256;     // 16-byte loads per thread per chunk (BM rows x 512 B)
			extern __shared__ __attribute__((aligned(16))) _Float16 tile[]; // [2][BM][kTileStride]
			const int lane = threadIdx.x & 63;
			const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
			const int r = lane & 15, g = lane >> 4;
			const int n_base = (blockIdx.x * 4 + wave) * 16 * NG;
			const int m_base = blockIdx.y * BM;
			const int chunks = k / kChunk;

			const uint8_t* rows[NG];
#pragma unroll
			for (int q = 0; q < NG; ++q)
			{
				// rows past the end re-read the last row; their results are never stored
				rows[q] = w + static_cast<size_t>(min(n_base + 16 * q + r, n - 1)) * row_bytes;
			}

			// activation staging: thread t moves 16-byte pieces p = t, t + 256, ... of the BM x 512 B tile
			u32x4 stage[kStageLoads];
			const auto stage_load = [&](int c) {
#pragma unroll
				for (int i = 0; i < kStageLoads; ++i)
				{
					const int p = threadIdx.x + 256 * i;
					const int row = p >> 5, piece = p & 31;
					const int mm = min(m_base + row, m_pad - 1);
					stage[i] = *reinterpret_cast<const u32x4*>(xh + static_cast<size_t>(mm) * k + c * kChunk + piece * 8);
				}
			};
			const auto stage_store = [&](int buf) {
#pragma unroll
				for (int i = 0; i < kStageLoads; ++i)
				{
					const int p = threadIdx.x + 256 * i;
					const int row = p >> 5, piece = p & 31;
					*reinterpret_cast<u32x4*>(tile + buf * kTileHalves + row * kTileStride + piece * 8) = stage[i];
				}
			};

			floatx4 acc[NG][MT];
#pragma unroll
			for (int q = 0; q < NG; ++q)
			{
#pragma unroll
				for (int t = 0; t < MT; ++t)
				{
					acc[q][t] = floatx4{ 0.0f, 0.0f, 0.0f, 0.0f };
				}
			}

			typename F::Raw raw[NG], raw_next[NG];
#pragma unroll
			for (int q = 0; q < NG; ++q)
			{
				raw[q] = F::load(rows[q], g);
			}
			stage_load(0);
			stage_store(0);
			__syncthreads();

			for (int c = 0; c < chunks; ++c)
			{
				const int buf = c & 1;
				const bool more = c + 1 < chunks;
				if (more)
				{
#pragma unroll
					for (int q = 0; q < NG; ++q)
					{
						raw_next[q] = F::load(rows[q] + static_cast<size_t>(c + 1) * F::kChunkBytes, g);
					}
					stage_load(c + 1);
				}
				typename F::Scale sc[NG];
#pragma unroll
				for (int q = 0; q < NG; ++q)
				{
					sc[q] = F::prep(raw[q], g);
				}
				const _Float16* xt = tile + buf * kTileHalves + r * kTileStride;
#pragma unroll
				for (int s = 0; s < 8; ++s)
				{
					half8 a[NG];
#pragma unroll
					for (int q = 0; q < NG; ++q)
					{
						uint32_t pk[4];
						F::frag(raw[q], sc[q], s, pk);
						const u32x4 v = { pk[0], pk[1], pk[2], pk[3] };
						a[q] = __builtin_bit_cast(half8, v);
					}
					int k0, k1;
					F::koff(g, s, k0, k1);
#pragma unroll
					for (int t = 0; t < MT; ++t)
					{
						const _Float16* xr = xt + t * 16 * kTileStride;
						const u32x2 b0 = *reinterpret_cast<const u32x2*>(xr + k0);
						const u32x2 b1 = *reinterpret_cast<const u32x2*>(xr + k1);
						const u32x4 bv = { b0.x, b0.y, b1.x, b1.y };
						const half8 b = __builtin_bit_cast(half8, bv);
#pragma unroll
						for (int q = 0; q < NG; ++q)
						{
							// D[i = weight row][j = activation row] += A[i][k] * B[k][j]
							acc[q][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[q], b, acc[q][t], 0, 0, 0);
						}
					}
				}
				if (more)
				{
					stage_store(buf ^ 1);
#pragma unroll
					for (int q = 0; q < NG; ++q)
					{
						raw[q] = raw_next[q];
					}
				}
				__syncthreads();
			}

			// D layout: lane holds activation row j = lane % 16 and weight rows 4 (lane / 16) + 0..3
#pragma unroll
			for (int q = 0; q < NG; ++q)
			{
				const int n0 = n_base + 16 * q + 4 * g;
#pragma unroll
				for (int t = 0; t < MT; ++t)
				{
					const int mm = m_base + 16 * t + r;
					if (mm < m)
					{
						float* dst = y + static_cast<size_t>(mm) * n + n0;
						const float* res = residual ? residual + static_cast<size_t>(mm) * n + n0 : nullptr;
						const float us = unscale[mm];
						const float vals[4] = { acc[q][t].x * us, acc[q][t].y * us, acc[q][t].z * us, acc[q][t].w * us };
#pragma unroll
						for (int e = 0; e < 4; ++e)
						{
							if (n0 + e < n)
							{
								dst[e] = res ? res[e] + vals[e] : vals[e];
							}
						}
					}
				}
			}
		}

		template <typename F, int BM, int NG>
		void launch_variant(const uint8_t* w, const _Float16* xh, const float* unscale, float* y, const float* residual,
		                    int n, int k, int m, int m_pad, size_t row_bytes, hipStream_t stream)
		{
			constexpr size_t lds = sizeof(_Float16) * 2 * BM * kTileStride;
			static const hipError_t attr =
			    hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_q_kernel<F, BM, NG>),
			                        hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
			(void)attr;
			const dim3 grid((n + 64 * NG - 1) / (64 * NG), (m_pad + BM - 1) / BM);
			gemm_q_kernel<F, BM, NG><<<grid, dim3(256), lds, stream>>>(w, xh, unscale, y, residual, n, k, m, m_pad,
			                                                         row_bytes);
		}

		// Tile choice: the activation tile as tall as the batch allows (each weight byte is
		// decoded once per activation tile), then as many row groups per wavefront as still
		// leave at least one workgroup per CU.
		template <typename F>
		void launch_format(const uint8_t* w, const _Float16* xh, const float* unscale, float* y, const float* residual,
		                   int n, int k, int m, int m_pad, size_t row_bytes, int cus, hipStream_t stream)
		{
			const auto blocks = [&](int bm, int ng) {
				return static_cast<long>((n + 64 * ng - 1) / (64 * ng)) * ((m_pad + bm - 1) / bm);
			};
			if (m_pad >= 128)
			{
				if (blocks(128, 4) >= cus)
				{
					launch_variant<F, 128, 4>(w, xh, unscale, y, residual, n, k, m, m_pad, row_bytes, stream);
				}
				else if (blocks(128, 2) >= cus)
				{
					launch_variant<F, 128, 2>(w, xh, unscale, y, residual, n, k, m, m_pad, row_bytes, stream);
				}
				else
				{
					launch_variant<F, 128, 1>(w, xh, unscale, y, residual, n, k, m, m_pad, row_bytes, stream);
				}
			}
			else if (m_pad >= 64)
			{
				if (blocks(64, 2) >= cus)
				{
					launch_variant<F, 64, 2>(w, xh, unscale, y, residual, n, k, m, m_pad, row_bytes, stream);
				}
				else
				{
					launch_variant<F, 64, 1>(w, xh, unscale, y, residual, n, k, m, m_pad, row_bytes, stream);
				}
			}
			else if (m_pad >= 32)
			{
				launch_variant<F, 32, 1>(w, xh, unscale, y, residual, n, k, m, m_pad, row_bytes, stream);
			}
			else
			{
				launch_variant<F, 16, 1>(w, xh, unscale, y, residual, n, k, m, m_pad, row_bytes, stream);
			}
		}
	} // namespace

	// halves of scratch launch_gemm needs for an m-row batch of width k
	size_t gemm_scratch_halves(size_t m, size_t k)
	{
		const size_t m_pad = (m + 15) / 16 * 16;
		return m_pad * k + 2 * m_pad; // fp16 rows, then one f32 factor per row
	}

	// Returns false when the shape is not one this kernel takes (the caller then uses the GEMV):
	// K must be a whole number of 256-element chunks and the rows 16-byte aligned.
	bool launch_gemm(int fmt, const void* wq, size_t n, size_t k, const float* x, size_t m, float* y,
	                 const float* residual, void* scratch_halves, hipStream_t stream)
	{
		const size_t rb = row_bytes(fmt, k);
		if (fmt != LITENN_FMT_Q4_0 && fmt != LITENN_FMT_Q8_0 && fmt != LITENN_FMT_Q4_K && fmt != LITENN_FMT_Q6_K)
		{
			return false;
		}
		// Q6_K blocks (210 bytes) are read with 2-byte aligned accesses; the other decoders use
		// 4- and 16-byte loads, which rows of whole 256-element chunks always allow
		const uintptr_t w_align = fmt == LITENN_FMT_Q6_K ? 2 : 16;
		if (k % kChunk != 0 || rb == 0 || reinterpret_cast<uintptr_t>(wq) % w_align != 0 ||
		    reinterpret_cast<uintptr_t>(x) % 16 != 0 || reinterpret_cast<uintptr_t>(scratch_halves) % 16 != 0 ||
		    !scratch_halves)
		{
			return false;
		}
		static const int cus = [] {
			int dev = 0;
			hipDeviceProp_t prop;
			if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess)
			{
				return 256;
			}
			return prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
		}();
		const size_t m_pad = (m + 15) / 16 * 16;
		_Float16* xh = static_cast<_Float16*>(scratch_halves);
		float* unscale = reinterpret_cast<float*>(xh + m_pad * k); // 4-byte aligned: m_pad * k is even
		to_half_kernel<<<dim3(static_cast<unsigned>(m_pad)), dim3(256), 0, stream>>>(x, xh, unscale, static_cast<int>(m),
		                                                                            static_cast<int>(k));
		const uint8_t* w = static_cast<const uint8_t*>(wq);
		const int ni = static_cast<int>(n), ki = static_cast<int>(k), mi = static_cast<int>(m),
		          mp = static_cast<int>(m_pad);
		switch (fmt)
		{
		case LITENN_FMT_Q4_0: launch_format<Q4_0Frag>(w, xh, unscale, y, residual, ni, ki, mi, mp, rb, cus, stream); break;
		case LITENN_FMT_Q8_0: launch_format<Q8_0Frag>(w, xh, unscale, y, residual, ni, ki, mi, mp, rb, cus, stream); break;
		case LITENN_FMT_Q4_K: launch_format<Q4_KFrag>(w, xh, unscale, y, residual, ni, ki, mi, mp, rb, cus, stream); break;
		default: launch_format<Q6_KFrag>(w, xh, unscale, y, residual, ni, ki, mi, mp, rb, cus, stream); break;
		}
		return true;
	}
} // namespace litenn_hip
