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
// Work split: a workgroup (WAVES wavefronts) owns 16 * WAVES * NG weight rows and 16 * MT
// activation rows; a wavefront owns NG groups of 16 weight rows and walks K in chunks of 256 (one
// K-quant super-block, eight 32-element blocks).  Lane (r, g) = (lane % 16, lane / 16) decodes 64
// of the 256 elements of row r of each of its groups per chunk, eight per MFMA step, in whatever
// order is cheapest for the format.  The activations are stored by the pre-pass in exactly that
// order, as ready-made 1 KB MFMA fragments, so the contraction is complete, no weight byte is
// decoded twice or staged in LDS, and an activation fragment is one lane-linear 128-bit access
// everywhere.  Chunk c + 1 (activation tile by direct-to-LDS loads, weights into a second
// register set) is fetched while chunk c is multiplied.
#include "common.hpp"

#include <algorithm>
#include <type_traits>

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

// Timing instrumentation, never set in a product build: -DLITENN_GEMM_KNOCKOUT=<bits> compiles a
// kernel with parts switched off (its results are then wrong) so that what the remaining parts
// cost can be measured: 1 activation staging, 2 weight loads, 4 the per-chunk barrier, 8 the
// decode arithmetic, 16 the LDS fragment reads.
#ifndef LITENN_GEMM_KNOCKOUT
#define LITENN_GEMM_KNOCKOUT 0
#endif
		constexpr int kChunk = 256; // K elements per step of the outer loop

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
		//
		// Small unsigned integers enter the arithmetic as binary16 SUBNORMALS: a 16-bit lane
		// holding 0..1023 read as a half is exactly value * 2^-24, so a masked nibble or byte is a
		// ready-made operand of v_fma_mix_f32 (half widened to f32 inside the multiply-add) and no
		// integer -> float conversion is issued; the 2^24 rides in the f32 scale.

		typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
		constexpr float kTwo24 = 16777216.0f, kTwo20 = 1048576.0f;

		// lo16(pair) * scale + bias and hi16(pair) * scale + bias, halves taken as subnormal binary16
		__device__ __forceinline__ void scale_pair(uint32_t pair, float scale, float bias, float& a, float& b)
		{
			const half2_t h = __builtin_bit_cast(half2_t, pair);
			a = __builtin_fmaf(static_cast<float>(h.x), scale, bias);
			b = __builtin_fmaf(static_cast<float>(h.y), scale, bias);
		}

		// One dword of packed nibbles -> 8 values: out[0..3] = low nibbles of bytes 0..3 (scale/bias
		// lo), out[4..7] = high nibbles (scale/bias hi; the nibble sits 4 bits up, scale_hi carries
		// 2^20 instead of 2^24)
		__device__ __forceinline__ void nibbles8(uint32_t v, float s_lo, float b_lo, float s_hi, float b_hi,
		                                          uint32_t (&out)[4])
		{
			const uint32_t t = v >> 8;
			float f0, f1, f2, f3;
			scale_pair(v & 0x000f000fu, s_lo, b_lo, f0, f2); // bytes 0, 2
			scale_pair(t & 0x000f000fu, s_lo, b_lo, f1, f3); // bytes 1, 3
			out[0] = pack_f16(f0, f1);
			out[1] = pack_f16(f2, f3);
			scale_pair(v & 0x00f000f0u, s_hi, b_hi, f0, f2);
			scale_pair(t & 0x00f000f0u, s_hi, b_hi, f1, f3);
			out[2] = pack_f16(f0, f1);
			out[3] = pack_f16(f2, f3);
		}

		// One dword of unsigned bytes -> 4 values u * scale + bias as two packed dwords
		__device__ __forceinline__ void bytes4(uint32_t v, float scale, float bias, uint32_t& p01, uint32_t& p23)
		{
			const uint32_t even = __builtin_amdgcn_perm(0u, v, 0x0c020c00u); // {b0, b2} as 16-bit lanes
			const uint32_t odd = __builtin_amdgcn_perm(0u, v, 0x0c030c01u);  // {b1, b3}
			float f0, f1, f2, f3;
			scale_pair(even, scale, bias, f0, f2);
			scale_pair(odd, scale, bias, f1, f3);
			p01 = pack_f16(f0, f1);
			p23 = pack_f16(f2, f3);
		}

		struct Q4_0Frag
		{
			static constexpr int kChunkBytes = 8 * 18;
			static constexpr int kFragValu = 19; // VALU instructions of one frag(), roughly
			static constexpr bool kWideTile = true; // two row groups x eight activation tiles fit the registers
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
			// (q - 8) * d: elements 4t .. 4t+3 (low nibbles) and 16 + 4t .. (high nibbles) of block b
			static __device__ __forceinline__ void frag(const Raw& r, const Scale& sc, int s, uint32_t (&out)[4])
			{
				const int b = s >> 2, t = s & 3;
				const float d = b == 0 ? sc.d0 : sc.d1;
				nibbles8(qs(r, b, t), d * kTwo24, -8.0f * d, d * kTwo20, -8.0f * d, out);
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
			static constexpr int kFragValu = 24;
			static constexpr bool kWideTile = false;
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
				// int8 q -> unsigned byte q + 128; the bias leaves through the -128 d term
				const float d = b == 0 ? sc.d0 : sc.d1;
				bytes4(lo ^ 0x80808080u, d * kTwo24, -128.0f * d, out[0], out[1]);
				bytes4(hi ^ 0x80808080u, d * kTwo24, -128.0f * d, out[2], out[3]);
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
			static constexpr int kFragValu = 17;
			static constexpr bool kWideTile = true;
			struct Raw { u32x4 h; uint32_t q[8]; }; // header (d, dmin, 12 scale bytes) + the 32 nibble bytes of group g
			struct Scale { float s0, m0, s1, m1; }; // d*sc*2^24, -dmin*m of sub-block 2g; d*sc*2^20, -dmin*m of 2g+1
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
			// 6-bit (scale, min) of sub-blocks 2g and 2g+1 (get_scale_min_k4 of the ggml block
			// definition): for g < 2 bytes 2g, 2g+1 (scales) and 2g+4, 2g+5 (mins) masked to 6 bits;
			// for g >= 2 low/high nibbles of bytes 2g+4, 2g+5 with bits 6..7 of bytes 2g-4, 2g-3
			// (scales) and 2g, 2g+1 (mins) on top.
			static __device__ __forceinline__ Scale prep(const Raw& r, int g)
			{
				const float d = f16_bits_to_f32(r.h.x), dmin = f16_bits_to_f32(r.h.x >> 16);
				const int sh = (g & 1) * 16;
				const uint32_t w0 = (r.h.y >> sh) & 0xffffu; // scale bytes 2g', 2g'+1 with g' = g & 1
				const uint32_t w1 = (r.h.z >> sh) & 0xffffu; // bytes 4 + 2g', 5 + 2g'
				const uint32_t w2 = (r.h.w >> sh) & 0xffffu; // bytes 8 + 2g', 9 + 2g'
				uint32_t sc, mn; // two values each, in 16-bit... byte lanes 0 and 1
				if (g < 2)
				{
					sc = w0 & 0x3f3fu;
					mn = w1 & 0x3f3fu;
				}
				else
				{
					sc = (w2 & 0x0f0fu) | ((w0 >> 2) & 0x3030u);
					mn = ((w2 >> 4) & 0x0f0fu) | ((w1 >> 2) & 0x3030u);
				}
				const float s0 = static_cast<float>(sc & 0xffu), s1 = static_cast<float>(sc >> 8);
				const float m0 = static_cast<float>(mn & 0xffu), m1 = static_cast<float>(mn >> 8);
				return { d * s0 * kTwo24, -(dmin * m0), d * s1 * kTwo20, -(dmin * m1) };
			}
			static __device__ __forceinline__ void frag(const Raw& r, const Scale& sc, int s, uint32_t (&out)[4])
			{
				// low nibbles: sub-block 2g, elements 4s ..; high nibbles: sub-block 2g+1
				nibbles8(r.q[s], sc.s0, sc.m0, sc.s1, sc.m1, out);
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
			static constexpr int kFragValu = 28;
			static constexpr bool kWideTile = false;
			// lane g = 2h + j covers l in [16j, 16j + 16) of half h: 16 bytes of each ql half-row,
			// 16 bytes of qh, the four scales 8h + j + 2i and d
			struct Raw { uint32_t la[4], lb[4], qh[4]; uint32_t sc[4]; uint32_t d; };
			struct Scale { float s[4], b[4]; }; // d*scale*2^24 and -32*d*scale per quarter
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
					const float ds = d * static_cast<float>(static_cast<int8_t>(r.sc[i]));
					s.s[i] = ds * kTwo24;
					s.b[i] = -32.0f * ds;
				}
				return s;
			}
			// step s: quarter i = s / 2 (q1..q4 of the ggml block definition), elements 8 (s % 2) .. + 7
			// of the lane's 16; 6-bit value = nibble | two bits of qh << 4, minus 32
			static __device__ __forceinline__ void frag(const Raw& r, const Scale& sc, int s, uint32_t (&out)[4])
			{
				const int i = s >> 1, u = s & 1;
#pragma unroll
				for (int w = 0; w < 2; ++w)
				{
					const uint32_t lw = (i & 1) ? r.lb[2 * u + w] : r.la[2 * u + w];
					const uint32_t nib = (i >= 2 ? lw >> 4 : lw) & 0x0f0f0f0fu;
					const uint32_t top = ((r.qh[2 * u + w] >> (2 * i)) & 0x03030303u) << 4;
					bytes4(nib | top, sc.s[i], sc.b[i], out[2 * w], out[2 * w + 1]);
				}
			}
			static __device__ __forceinline__ void koff(int g, int s, int& k0, int& k1)
			{
				const int h = g >> 1, j = g & 1;
				k0 = 128 * h + 32 * (s >> 1) + 16 * j + 8 * (s & 1);
				k1 = k0 + 4;
			}
		};

		// ---- activations to fp16, in fragment order ----------------------------------------------------
		// One workgroup per row.  Every row is scaled by a power of two so that its largest magnitude
		// lands in [2^14, 2^15): nothing overflows fp16 whatever the activations' range, small rows keep
		// full fp16 precision, and the scaling itself is exact; the GEMM multiplies the row's results by
		// the inverse factor.  Rows m .. m_pad - 1 are zero padding.
		//
		// The fp16 rows are not stored row-major but as the GEMM consumes them: for every 16-row tile
		// mt and 256-element chunk c, eight 1 KB fragments (one per MFMA step s), each holding for lane
		// (r, g) the 8 halves of row 16 mt + r that pair with the format's weight fragment of that step
		// (F::koff).  A fragment is then one lane-linear 128-bit read, in global memory and in LDS.
		constexpr int kFragBytes = 1024;                // 64 lanes x 8 halves
		constexpr int kChunkTileBytes = 8 * kFragBytes; // one 16-row tile of one chunk

		template <typename F>
		__global__ __launch_bounds__(256) void to_half_kernel(const float* __restrict__ x, uint8_t* __restrict__ xf,
		                                                       float* __restrict__ unscale, int m, int k)
		{
			__shared__ float red[4];
			const int row = blockIdx.x;
			const int chunks = k / kChunk;
			const int mt = row >> 4, r = row & 15;
			uint8_t* tile_row = xf + static_cast<size_t>(mt) * chunks * kChunkTileBytes + r * 16;
			const int items = chunks * 32; // (chunk, step, lane group) triples of this row
			if (row >= m)
			{
				for (int it = threadIdx.x; it < items; it += 256)
				{
					const int c = it >> 5, st = (it >> 2) & 7, g = it & 3;
					*reinterpret_cast<u32x4*>(tile_row + (c * 8 + st) * kFragBytes + g * 256) = u32x4{ 0u, 0u, 0u, 0u };
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
			for (int it = threadIdx.x; it < items; it += 256)
			{
				const int c = it >> 5, st = (it >> 2) & 7, g = it & 3;
				int k0, k1;
				F::koff(g, st, k0, k1);
				const float4 v0 = *reinterpret_cast<const float4*>(src + c * kChunk + k0);
				const float4 v1 = *reinterpret_cast<const float4*>(src + c * kChunk + k1);
				u32x4 out;
				out.x = pack_f16(ldexpf(v0.x, shift), ldexpf(v0.y, shift));
				out.y = pack_f16(ldexpf(v0.z, shift), ldexpf(v0.w, shift));
				out.z = pack_f16(ldexpf(v1.x, shift), ldexpf(v1.y, shift));
				out.w = pack_f16(ldexpf(v1.z, shift), ldexpf(v1.w, shift));
				*reinterpret_cast<u32x4*>(tile_row + (c * 8 + st) * kFragBytes + g * 256) = out;
			}
			if (threadIdx.x == 0)
			{
				unscale[row] = ldexpf(1.0f, -shift);
			}
		}

		// ---- the GEMM ---------------------------------------------------------------------------
		// grid (ceil(N / (16 WAVES NG)), ceil(M_tiles / MT)); block 64 WAVES; MT 16-row activation
		// tiles and NG 16-row weight groups per wavefront.
		//
		// Per 256-element chunk the workgroup's MT activation tiles (MT x 8 KB, already in fragment
		// order) are copied global -> LDS by direct loads, into the half of a double buffer the
		// previous chunk is not using; the wavefront's weights of the next chunk are loaded into the
		// idle one of two register sets at the same time.  Inside a chunk the eight MFMA steps are
		// software-pipelined: while the NG x MT MFMAs of step s run, the activation fragments of step
		// s + 1 are read from LDS and the weight fragments of step s + 1 are decoded, the three
		// instruction streams interleaved by scheduling directives.  One barrier per chunk, before
		// the last step reads the first fragments of the next chunk.
		typedef __attribute__((address_space(3))) void* gemm_lds_ptr_t;
		typedef const __attribute__((address_space(1))) void* gemm_global_ptr_t;

		template <typename F, int MT, int NG, int WAVES>
		__global__ __launch_bounds__(64 * WAVES) void gemm_q_kernel(const uint8_t* __restrict__ w,
		                                                             const uint8_t* __restrict__ xf,
		                                                             const float* __restrict__ unscale,
		                                                             float* __restrict__ y,
		                                                             const float* __restrict__ residual, int n, int k,
		                                                             int m, int m_tiles, size_t row_bytes)
		{
			constexpr int kThreads = 64 * WAVES;
			constexpr int kTileBytes = MT * kChunkTileBytes; // one chunk of the workgroup's activations
			constexpr int kStageLoads = kTileBytes / (kThreads * 16);
			static_assert(kStageLoads >= 1 && kStageLoads * kThreads * 16 == kTileBytes, "tile / thread split");
			extern __shared__ __attribute__((aligned(16))) uint8_t tile[]; // [2][kTileBytes]
			const int lane = threadIdx.x & 63;
			const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
			const int r = lane & 15, g = lane >> 4;
			const int n_base = (blockIdx.x * WAVES + wave) * 16 * NG;
			const int mt_base = blockIdx.y * MT;
			const int chunks = k / kChunk;

			const uint8_t* rows[NG];
#pragma unroll
			for (int q = 0; q < NG; ++q)
			{
				// rows past the end re-read the last row; their results are never stored
				rows[q] = w + static_cast<size_t>(min(n_base + 16 * q + r, n - 1)) * row_bytes;
			}

			// activation staging: load i of wavefront `wave` moves the 1 KB piece i * WAVES + wave of
			// the tile, lane l its bytes 16 l ..; tiles past the end re-read the last one.  The piece
			// offsets are wavefront-uniform (scalar registers), only the lane offset is per lane.
			uint32_t stage_off[kStageLoads];
#pragma unroll
			for (int i = 0; i < kStageLoads; ++i)
			{
				const int piece = i * WAVES + wave; // 1 KB pieces, 8 per 16-row tile
				const int t = min(mt_base + (piece >> 3), m_tiles - 1);
				stage_off[i] = static_cast<uint32_t>(t * chunks) * kChunkTileBytes + (piece & 7) * kFragBytes;
			}
			// Issued outside the compiler's view: it would otherwise treat the pending direct-to-LDS
			// loads as possibly out-of-order returns and turn every later LDS wait of the chunk into a
			// wait for everything.  The explicit vmcnt(0) before the chunk's barrier covers them.
			const uint32_t lane_off = lane * 16;
			const uint32_t tile_lds = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
			    (__attribute__((address_space(3))) const uint8_t*)(tile)));
			const auto stage_issue = [&](int c, int buf) {
#pragma unroll
				for (int i = 0; i < kStageLoads; ++i)
				{
					const int piece = i * WAVES + wave;
					const uint8_t* src = xf + (stage_off[i] + static_cast<uint32_t>(c) * kChunkTileBytes);
					const uint32_t dst = tile_lds + buf * kTileBytes + piece * kFragBytes;
					asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
					             :
					             : "s"(dst), "v"(lane_off), "s"(src)
					             : "memory", "m0");
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

			half8 a_cur[NG], a_nxt[NG];
			u32x4 b[MT]; // fragment t of the current step until its MFMAs are issued, then of the next
			const uint8_t* lane_tile = tile + lane * 16;
			const auto read_b = [&](int t, int buf, int s) {
				b[t] = *reinterpret_cast<const u32x4*>(lane_tile + buf * kTileBytes + t * kChunkTileBytes + s * kFragBytes);
			};
			const auto decode = [&](half8 (&a)[NG], const typename F::Raw (&raw)[NG], const typename F::Scale (&sc)[NG],
			                        int s) {
#pragma unroll
				for (int q = 0; q < NG; ++q)
				{
					uint32_t pk[4];
					F::frag(raw[q], sc[q], s, pk);
					const u32x4 v = { pk[0], pk[1], pk[2], pk[3] };
					a[q] = __builtin_bit_cast(half8, v);
				}
			};
			// the MFMAs of the current step; fragment t is refilled for step (buf, s) right after its
			// last use (refill = false on the very last step)
			const auto mfma_step = [&](bool refill, int buf, int s) {
#pragma unroll
				for (int t = 0; t < MT; ++t)
				{
					const half8 bt = __builtin_bit_cast(half8, b[t]);
#pragma unroll
					for (int q = 0; q < NG; ++q)
					{
						// D[i = weight row][j = activation row] += A[i][k] * B[k][j]
						acc[q][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_cur[q], bt, acc[q][t], 0, 0, 0);
					}
					if (refill)
					{
						read_b(t, buf, s);
					}
				}
			};
			const auto rotate = [&]() {
#pragma unroll
				for (int q = 0; q < NG; ++q)
				{
					a_cur[q] = a_nxt[q];
				}
			};
			// spread the LDS reads and the decode arithmetic of a step between its MFMAs
			const auto interleave = [&]() {
				constexpr int kMfma = NG * MT;
				constexpr int kValuPerTile = (F::kFragValu * NG + MT - 1) / MT;
#pragma unroll
				for (int t = 0; t < MT; ++t)
				{
					__builtin_amdgcn_sched_group_barrier(0x008, NG, 0);           // the MFMAs of one activation fragment
					__builtin_amdgcn_sched_group_barrier(0x100, 1, 0);            // its refill from LDS
					__builtin_amdgcn_sched_group_barrier(0x002, kValuPerTile, 0); // a share of the decode arithmetic
				}
				(void)kMfma;
			};
			const auto load_raw = [&](typename F::Raw (&raw)[NG], int c) {
#pragma unroll
				for (int q = 0; q < NG; ++q)
				{
					raw[q] = F::load(rows[q] + static_cast<size_t>(c) * F::kChunkBytes, g);
				}
			};
			const auto prep_all = [&](typename F::Scale (&sc)[NG], const typename F::Raw (&raw)[NG]) {
#pragma unroll
				for (int q = 0; q < NG; ++q)
				{
					sc[q] = F::prep(raw[q], g);
				}
			};
			constexpr int kWaitAllLoads = 0x0F70; // s_waitcnt vmcnt(0), the other counters at their maxima

			// one chunk out of `cur`, fetching the next into `nxt`
			const auto chunk = [&](auto has_next_tag, const typename F::Raw (&raw_cur)[NG],
			                       const typename F::Scale (&sc_cur)[NG], typename F::Raw (&raw_nxt)[NG],
			                       typename F::Scale (&sc_nxt)[NG], int c, int buf) {
				constexpr bool has_next = decltype(has_next_tag)::value;
				if (has_next)
				{
#if !(LITENN_GEMM_KNOCKOUT & 1)
					stage_issue(c + 1, buf ^ 1);
#endif
#if !(LITENN_GEMM_KNOCKOUT & 2)
					load_raw(raw_nxt, c + 1);
#endif
				}
#pragma unroll
				for (int s = 0; s < 7; ++s)
				{
#if !(LITENN_GEMM_KNOCKOUT & 8)
					decode(a_nxt, raw_cur, sc_cur, s + 1);
#endif
					mfma_step(!(LITENN_GEMM_KNOCKOUT & 16), buf, s + 1);
					interleave();
					__builtin_amdgcn_sched_barrier(0);
					rotate();
				}
				// Everything this wavefront requested at the top of the chunk has landed, every
				// wavefront's LDS reads of this chunk have returned: after the barrier the next tile is
				// complete and this one may be overwritten.
				__builtin_amdgcn_s_waitcnt(kWaitAllLoads);
#if !(LITENN_GEMM_KNOCKOUT & 4)
				__syncthreads();
#endif
				if (has_next)
				{
#if !(LITENN_GEMM_KNOCKOUT & 2)
					prep_all(sc_nxt, raw_nxt);
#endif
#if !(LITENN_GEMM_KNOCKOUT & 8)
					decode(a_nxt, raw_nxt, sc_nxt, 0);
#endif
				}
				mfma_step(has_next && !(LITENN_GEMM_KNOCKOUT & 16), buf ^ 1, 0);
				if (has_next)
				{
					interleave();
				}
				__builtin_amdgcn_sched_barrier(0);
				rotate();
			};

			typename F::Raw raw_a[NG], raw_b[NG];
			typename F::Scale sc_a[NG], sc_b[NG];
			stage_issue(0, 0);
			load_raw(raw_a, 0);
			__builtin_amdgcn_s_waitcnt(kWaitAllLoads);
			__syncthreads();
			prep_all(sc_a, raw_a);
#pragma unroll
			for (int t = 0; t < MT; ++t)
			{
				read_b(t, 0, 0);
			}
			decode(a_cur, raw_a, sc_a, 0);
#if LITENN_GEMM_KNOCKOUT
			load_raw(raw_b, 0);
			prep_all(sc_b, raw_b);
			decode(a_nxt, raw_a, sc_a, 1);
#endif
			// chunks come in pairs (one per register set and LDS half); the last one fetches nothing
			using std::false_type;
			using std::true_type;
			int c = 0;
			for (; c + 2 < chunks; c += 2)
			{
				chunk(true_type{}, raw_a, sc_a, raw_b, sc_b, c, 0);
				chunk(true_type{}, raw_b, sc_b, raw_a, sc_a, c + 1, 1);
			}
			if (c + 2 == chunks)
			{
				chunk(true_type{}, raw_a, sc_a, raw_b, sc_b, c, 0);
				chunk(false_type{}, raw_b, sc_b, raw_a, sc_a, c + 1, 1);
			}
			else
			{
				chunk(false_type{}, raw_a, sc_a, raw_b, sc_b, c, 0);
			}

			// D layout: lane holds activation row j = lane % 16 and weight rows 4 (lane / 16) + 0..3
			const bool vec_ok = (n & 3) == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0 &&
			                    (!residual || (reinterpret_cast<uintptr_t>(residual) & 15) == 0);
#pragma unroll
			for (int q = 0; q < NG; ++q)
			{
				const int n0 = n_base + 16 * q + 4 * g;
#pragma unroll
				for (int t = 0; t < MT; ++t)
				{
					const int mm = (mt_base + t) * 16 + r;
					if (mm < m)
					{
						float* dst = y + static_cast<size_t>(mm) * n + n0;
						const float* res = residual ? residual + static_cast<size_t>(mm) * n + n0 : nullptr;
						const float us = unscale[mm];
						const float vals[4] = { acc[q][t].x * us, acc[q][t].y * us, acc[q][t].z * us, acc[q][t].w * us };
						if (vec_ok && n0 + 3 < n)
						{
							float4 out = { vals[0], vals[1], vals[2], vals[3] };
							if (res)
							{
								const float4 rv = *reinterpret_cast<const float4*>(res);
								out.x += rv.x, out.y += rv.y, out.z += rv.z, out.w += rv.w;
							}
							*reinterpret_cast<float4*>(dst) = out;
						}
						else
						{
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
		}

		template <typename F, int MT, int NG, int WAVES>
		void launch_variant(const uint8_t* w, const uint8_t* xf, const float* unscale, float* y, const float* residual,
		                    int n, int k, int m, int m_tiles, size_t row_bytes, hipStream_t stream)
		{
			constexpr size_t lds = 2 * MT * kChunkTileBytes;
			static const hipError_t attr =
			    hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_q_kernel<F, MT, NG, WAVES>),
			                        hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
			(void)attr;
			constexpr int bn = 16 * WAVES * NG;
			const dim3 grid((n + bn - 1) / bn, (m_tiles + MT - 1) / MT);
			gemm_q_kernel<F, MT, NG, WAVES><<<grid, dim3(64 * WAVES), lds, stream>>>(w, xf, unscale, y, residual, n, k, m,
			                                                                        m_tiles, row_bytes);
		}

		// Tile choice: MT activation tiles per workgroup so that a weight is decoded as few times as
		// possible (MT = 8 takes 128 KB of LDS, so eight wavefronts share it); two weight groups per
		// wavefront (each activation fragment read from LDS feeds two MFMAs) when that still leaves
		// every CU a workgroup.
		template <typename F>
		void launch_format(const uint8_t* w, const uint8_t* xf, const float* unscale, float* y, const float* residual,
		                   int n, int k, int m, int m_tiles, size_t row_bytes, int cus, hipStream_t stream)
		{
			const auto blocks = [&](int mt, int bn) {
				return static_cast<long>((n + bn - 1) / bn) * ((m_tiles + mt - 1) / mt);
			};
			static const int forced = env_int("LITENN_HIP_GEMM_TILE", 0); // MT * 100 + NG * 10 + WAVES
#define LITENN_GEMM_ARGS w, xf, unscale, y, residual, n, k, m, m_tiles, row_bytes, stream
#define LITENN_GEMM_CASE(MT_, NG_, WV_)                                                                              \
	if (pick == MT_ * 100 + NG_ * 10 + WV_)                                                                        \
	{                                                                                                              \
		launch_variant<F, MT_, NG_, WV_>(LITENN_GEMM_ARGS);                                                        \
		return;                                                                                                    \
	}
			int pick = forced;
			if (pick == 0)
			{
				// measured on the MI355X (K = 4096, N = 4096 and 14336, M = 16 .. 512): the widest tile
				// wins once it nearly fills the card, otherwise the tallest single-group tile that
				// still gives every CU a workgroup
				if (m_tiles >= 8 && F::kWideTile && 5 * blocks(8, 256) >= 4 * cus)
				{
					pick = 828;
				}
				else if (m_tiles >= 8 && blocks(8, 128) >= cus)
				{
					pick = 818;
				}
				else if (m_tiles >= 4 && blocks(4, 64) >= cus)
				{
					pick = 414;
				}
				else if (m_tiles >= 2 && blocks(2, 64) >= cus)
				{
					pick = 214;
				}
				else
				{
					pick = 114;
				}
			}
			LITENN_GEMM_CASE(8, 2, 8)
			LITENN_GEMM_CASE(8, 1, 8)
			LITENN_GEMM_CASE(4, 1, 4)
			LITENN_GEMM_CASE(2, 1, 4)
			LITENN_GEMM_CASE(1, 1, 4)
			launch_variant<F, 1, 1, 4>(LITENN_GEMM_ARGS);
#undef LITENN_GEMM_CASE
#undef LITENN_GEMM_ARGS
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
		    !scratch_halves || 2 * ((m + 15) / 16 * 16) * k >= (size_t{ 1 } << 32)) // 32-bit tile offsets
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
		uint8_t* xf = static_cast<uint8_t*>(scratch_halves);
		float* unscale = reinterpret_cast<float*>(xf + 2 * m_pad * k); // after the fp16 tiles
		const uint8_t* w = static_cast<const uint8_t*>(wq);
		const int ni = static_cast<int>(n), ki = static_cast<int>(k), mi = static_cast<int>(m),
		          mt = static_cast<int>(m_pad / 16);
		const dim3 rows_grid(static_cast<unsigned>(m_pad));
		switch (fmt)
		{
		case LITENN_FMT_Q4_0:
			to_half_kernel<Q4_0Frag><<<rows_grid, dim3(256), 0, stream>>>(x, xf, unscale, mi, ki);
			launch_format<Q4_0Frag>(w, xf, unscale, y, residual, ni, ki, mi, mt, rb, cus, stream);
			break;
		case LITENN_FMT_Q8_0:
			to_half_kernel<Q8_0Frag><<<rows_grid, dim3(256), 0, stream>>>(x, xf, unscale, mi, ki);
			launch_format<Q8_0Frag>(w, xf, unscale, y, residual, ni, ki, mi, mt, rb, cus, stream);
			break;
		case LITENN_FMT_Q4_K:
			to_half_kernel<Q4_KFrag><<<rows_grid, dim3(256), 0, stream>>>(x, xf, unscale, mi, ki);
			launch_format<Q4_KFrag>(w, xf, unscale, y, residual, ni, ki, mi, mt, rb, cus, stream);
			break;
		default:
			to_half_kernel<Q6_KFrag><<<rows_grid, dim3(256), 0, stream>>>(x, xf, unscale, mi, ki);
			launch_format<Q6_KFrag>(w, xf, unscale, y, residual, ni, ki, mi, mt, rb, cus, stream);
			break;
		}
		return true;
	}
} // namespace litenn_hip
