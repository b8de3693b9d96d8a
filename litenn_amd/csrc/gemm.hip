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
#include "fetch_model.hpp"

#include <algorithm>
#include <cstdio>
#include <cstring>
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

		constexpr int kChunk = 256; // K elements per step of the outer loop

		__device__ __forceinline__ uint32_t pack_f16(float a, float b)
		{
			const float2v f = { a, b };
			const half2v h = __builtin_convertvector(f, half2v); // v_cvt_pk_f16_f32, round to nearest even
			return __builtin_bit_cast(uint32_t, h);
		}

		// the weight bytes reach the decoders through LDS
		typedef const __attribute__((address_space(3))) uint8_t* lds_bytes_t;
		typedef const __attribute__((address_space(3))) u32x4* lds_u32x4_t;

		// little-endian reads at 2-byte alignment (K-quant blocks are only that aligned)
		__device__ __forceinline__ uint32_t ld_u32(lds_bytes_t p)
		{
			typedef uint32_t u32_a2 __attribute__((aligned(2)));
			return *(const __attribute__((address_space(3))) u32_a2*)(p);
		}
		__device__ __forceinline__ uint32_t ld_u32_aligned(lds_bytes_t p)
		{
			return *(const __attribute__((address_space(3))) uint32_t*)(p);
		}
		__device__ __forceinline__ uint32_t ld_u16(lds_bytes_t p)
		{
			return *(const __attribute__((address_space(3))) uint16_t*)(p);
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
			static constexpr bool kAligned16 = true; // chunks start on 16-byte boundaries
			static constexpr bool kWideTile = true;  // two row groups x eight activation tiles fit the registers
			struct Raw { uint32_t w[9]; }; // blocks 2g and 2g+1: 36 bytes
			struct Scale { float d0, d1; };
			static __device__ __forceinline__ Raw load(lds_bytes_t chunk, int g)
			{
				Raw r;
				lds_bytes_t p = chunk + 36 * g; // 4-byte aligned: rows are 16-byte aligned
#pragma unroll
				for (int i = 0; i < 9; ++i)
				{
					r.w[i] = ld_u32_aligned(p + 4 * i);
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

		// One dword of packed nibbles plus their fifth bits -> 8 values: `lo4` / `hi4` hold the fifth
		// bits of the four low-nibble / high-nibble elements (bit j for byte j).  The bit joins its
		// nibble inside the 16-bit lane (16 units of the nibble's own scale); the multipliers copy
		// bits 0 and 2 (bytes 0, 2) or 1 and 3 (bytes 1, 3) to the lanes' positions.
		__device__ __forceinline__ void nibbles8_fifth(uint32_t v, uint32_t lo4, uint32_t hi4, float s_lo, float b_lo,
		                                                float s_hi, float b_hi, uint32_t (&out)[4])
		{
			const uint32_t t = v >> 8;
			float f0, f1, f2, f3;
			scale_pair((v & 0x000f000fu) | ((lo4 * 0x00040010u) & 0x00100010u), s_lo, b_lo, f0, f2); // bytes 0, 2
			scale_pair((t & 0x000f000fu) | ((lo4 * 0x00020008u) & 0x00100010u), s_lo, b_lo, f1, f3); // bytes 1, 3
			out[0] = pack_f16(f0, f1);
			out[1] = pack_f16(f2, f3);
			scale_pair((v & 0x00f000f0u) | ((hi4 * 0x00400100u) & 0x01000100u), s_hi, b_hi, f0, f2);
			scale_pair((t & 0x00f000f0u) | ((hi4 * 0x00200080u) & 0x01000100u), s_hi, b_hi, f1, f3);
			out[2] = pack_f16(f0, f1);
			out[3] = pack_f16(f2, f3);
		}

		struct Q4_1Frag // block { fp16 d; fp16 m; u8 qs[16]; }: q d + m
		{
			static constexpr int kChunkBytes = 8 * 20;
			static constexpr int kFragValu = 19;
			static constexpr bool kAligned16 = true;
			static constexpr bool kWideTile = false;
			struct Raw { uint32_t w[10]; }; // blocks 2g and 2g+1: {d m} q q q q {d m} q q q q
			struct Scale { float d0, m0, d1, m1; };
			static __device__ __forceinline__ Raw load(lds_bytes_t chunk, int g)
			{
				Raw r;
				lds_bytes_t p = chunk + 40 * g;
#pragma unroll
				for (int i = 0; i < 10; ++i)
				{
					r.w[i] = ld_u32_aligned(p + 4 * i);
				}
				return r;
			}
			static __device__ __forceinline__ Scale prep(const Raw& r, int)
			{
				return { f16_bits_to_f32(r.w[0]), f16_bits_to_f32(r.w[0] >> 16), f16_bits_to_f32(r.w[5]),
					     f16_bits_to_f32(r.w[5] >> 16) };
			}
			static __device__ __forceinline__ void frag(const Raw& r, const Scale& sc, int s, uint32_t (&out)[4])
			{
				const int b = s >> 2, t = s & 3;
				const float d = b == 0 ? sc.d0 : sc.d1, m = b == 0 ? sc.m0 : sc.m1;
				nibbles8(r.w[5 * b + 1 + t], d * kTwo24, m, d * kTwo20, m, out);
			}
			static __device__ __forceinline__ void koff(int g, int s, int& k0, int& k1) { Q4_0Frag::koff(g, s, k0, k1); }
		};

		struct Q5_0Frag // block { fp16 d; u8 qh[4]; u8 qs[16]; }: ((nibble | bit << 4) - 16) d
		{
			static constexpr int kChunkBytes = 8 * 22;
			static constexpr int kFragValu = 33;
			static constexpr bool kAligned16 = true;
			static constexpr bool kWideTile = true;  // (182 VGPRs with two row groups: no spill)
			struct Raw { uint32_t w[11]; }; // blocks 2g and 2g+1: bytes 0..21 and 22..43
			struct Scale { float d0, d1; };
			static __device__ __forceinline__ Raw load(lds_bytes_t chunk, int g)
			{
				Raw r;
				lds_bytes_t p = chunk + 44 * g;
#pragma unroll
				for (int i = 0; i < 11; ++i)
				{
					r.w[i] = ld_u32_aligned(p + 4 * i);
				}
				return r;
			}
			static __device__ __forceinline__ Scale prep(const Raw& r, int)
			{
				return { f16_bits_to_f32(r.w[0]), f16_bits_to_f32(r.w[5] >> 16) };
			}
			static __device__ __forceinline__ void frag(const Raw& r, const Scale& sc, int s, uint32_t (&out)[4])
			{
				const int b = s >> 2, t = s & 3;
				// block 0: qh at byte 2, qs at byte 6; block 1: qh at byte 24, qs at byte 28
				const uint32_t qh = b == 0 ? ((r.w[0] >> 16) | (r.w[1] << 16)) : r.w[6];
				const uint32_t qs = b == 0 ? ((r.w[1 + t] >> 16) | (r.w[2 + t] << 16)) : r.w[7 + t];
				const float d = b == 0 ? sc.d0 : sc.d1;
				nibbles8_fifth(qs, (qh >> (4 * t)) & 0xFu, (qh >> (16 + 4 * t)) & 0xFu, d * kTwo24, -16.0f * d, d * kTwo20,
				               -16.0f * d, out);
			}
			static __device__ __forceinline__ void koff(int g, int s, int& k0, int& k1) { Q4_0Frag::koff(g, s, k0, k1); }
		};

		struct Q5_1Frag // block { fp16 d; fp16 m; u8 qh[4]; u8 qs[16]; }: (nibble | bit << 4) d + m
		{
			static constexpr int kChunkBytes = 8 * 24;
			static constexpr int kFragValu = 33;
			static constexpr bool kAligned16 = true;
			static constexpr bool kWideTile = false;
			struct Raw { uint32_t w[12]; }; // {d m} qh q q q q, twice
			struct Scale { float d0, m0, d1, m1; };
			static __device__ __forceinline__ Raw load(lds_bytes_t chunk, int g)
			{
				Raw r;
				lds_bytes_t p = chunk + 48 * g;
#pragma unroll
				for (int i = 0; i < 12; ++i)
				{
					r.w[i] = ld_u32_aligned(p + 4 * i);
				}
				return r;
			}
			static __device__ __forceinline__ Scale prep(const Raw& r, int)
			{
				return { f16_bits_to_f32(r.w[0]), f16_bits_to_f32(r.w[0] >> 16), f16_bits_to_f32(r.w[6]),
					     f16_bits_to_f32(r.w[6] >> 16) };
			}
			static __device__ __forceinline__ void frag(const Raw& r, const Scale& sc, int s, uint32_t (&out)[4])
			{
				const int b = s >> 2, t = s & 3;
				const uint32_t qh = r.w[6 * b + 1];
				const float d = b == 0 ? sc.d0 : sc.d1, m = b == 0 ? sc.m0 : sc.m1;
				nibbles8_fifth(r.w[6 * b + 2 + t], (qh >> (4 * t)) & 0xFu, (qh >> (16 + 4 * t)) & 0xFu, d * kTwo24, m,
				               d * kTwo20, m, out);
			}
			static __device__ __forceinline__ void koff(int g, int s, int& k0, int& k1) { Q4_0Frag::koff(g, s, k0, k1); }
		};

		// Q2_K and Q3_K: lane g owns the 64 consecutive elements 64 g .. of the super-block: planes
		// 2 (g % 2) and 2 (g % 2) + 1 of the 32 quant bytes of half g / 2.  Step s covers elements
		// 16 (s / 2) + 8 (s % 2) .. + 7 of the lane's 64: group s / 2 (one scale), plane (s / 2) / 2,
		// bytes 16 ((s / 2) % 2) + 8 (s % 2) .. + 7.
		struct Q2_KFrag // { u8 scales[16]; u8 qs[64]; fp16 d; fp16 dmin; }: d (sc & 15) q - dmin (sc >> 4)
		{
			static constexpr int kChunkBytes = 84;
			static constexpr int kFragValu = 24;
			static constexpr bool kAligned16 = false; // 84-byte blocks: 4-byte aligned
			static constexpr bool kWideTile = true;  // (206 VGPRs with two row groups: no spill)
			struct Raw { uint32_t q[8]; uint32_t sc, dd; };
			struct Scale { float s[4], b[4]; int shift; };
			static __device__ __forceinline__ Raw load(lds_bytes_t chunk, int g)
			{
				Raw r;
				lds_bytes_t q = chunk + 16 + 32 * (g >> 1);
#pragma unroll
				for (int i = 0; i < 8; ++i)
				{
					r.q[i] = ld_u32_aligned(q + 4 * i);
				}
				r.sc = ld_u32_aligned(chunk + 4 * g);
				r.dd = ld_u32_aligned(chunk + 80);
				return r;
			}
			static __device__ __forceinline__ Scale prep(const Raw& r, int g)
			{
				const float d = f16_bits_to_f32(r.dd), dmin = f16_bits_to_f32(r.dd >> 16);
				Scale s;
#pragma unroll
				for (int i = 0; i < 4; ++i)
				{
					const uint32_t sc = (r.sc >> (8 * i)) & 0xffu;
					s.s[i] = d * static_cast<float>(sc & 0xFu) * kTwo24;
					s.b[i] = -(dmin * static_cast<float>(sc >> 4));
				}
				s.shift = 4 * (g & 1);
				return s;
			}
			static __device__ __forceinline__ void frag(const Raw& r, const Scale& sc, int s, uint32_t (&out)[4])
			{
				const int grp = s >> 1, w0 = 4 * (grp & 1) + 2 * (s & 1);
				const int shift = sc.shift + 2 * (grp >> 1);
				bytes4((r.q[w0] >> shift) & 0x03030303u, sc.s[grp], sc.b[grp], out[0], out[1]);
				bytes4((r.q[w0 + 1] >> shift) & 0x03030303u, sc.s[grp], sc.b[grp], out[2], out[3]);
			}
			static __device__ __forceinline__ void koff(int g, int s, int& k0, int& k1)
			{
				k0 = 64 * g + 8 * s;
				k1 = k0 + 4;
			}
		};

		struct Q3_KFrag // { u8 hmask[32]; u8 qs[64]; u8 scales[12]; fp16 d; }: d (sc - 32) (q - (bit ? 0 : 4))
		{
			static constexpr int kChunkBytes = 110;
			static constexpr int kFragValu = 34;
			static constexpr bool kAligned16 = false; // 110-byte blocks: 2-byte aligned
			static constexpr bool kWideTile = false;
			struct Raw { uint32_t hm[8], q[8], s[3], d; };
			struct Scale { float s[4], b[4]; int shift, hshift; };
			static __device__ __forceinline__ Raw load(lds_bytes_t chunk, int g)
			{
				Raw r;
				lds_bytes_t q = chunk + 32 + 32 * (g >> 1);
#pragma unroll
				for (int i = 0; i < 8; ++i)
				{
					r.hm[i] = ld_u32(chunk + 4 * i);
					r.q[i] = ld_u32(q + 4 * i);
				}
#pragma unroll
				for (int i = 0; i < 3; ++i)
				{
					r.s[i] = ld_u32(chunk + 96 + 4 * i);
				}
				r.d = ld_u16(chunk + 108);
				return r;
			}
			// the lane's four six-bit scales 4 g .. 4 g + 3, biased by 32: low four bits are the low
			// (g < 2) or high nibbles of scale bytes 4 (g % 2) .. + 3, the top two are bits 2 g, 2 g + 1
			// of bytes 8 .. 11
			static __device__ __forceinline__ Scale prep(const Raw& r, int g)
			{
				const float d = f16_bits_to_f32(r.d);
				const uint32_t low4 = (((g & 1) ? r.s[1] : r.s[0]) >> (4 * (g >> 1))) & 0x0f0f0f0fu;
				const uint32_t top2 = ((r.s[2] >> (2 * g)) & 0x03030303u) << 4;
				const uint32_t six = low4 | top2;
				Scale s;
#pragma unroll
				for (int i = 0; i < 4; ++i)
				{
					const float ds = d * static_cast<float>(static_cast<int>((six >> (8 * i)) & 0xffu) - 32);
					s.s[i] = ds * kTwo24;
					s.b[i] = -4.0f * ds;
				}
				s.shift = 4 * (g & 1);
				s.hshift = 2 * g;
				return s;
			}
			static __device__ __forceinline__ void frag(const Raw& r, const Scale& sc, int s, uint32_t (&out)[4])
			{
				const int grp = s >> 1, w0 = 4 * (grp & 1) + 2 * (s & 1);
				const int shift = sc.shift + 2 * (grp >> 1), hshift = sc.hshift + (grp >> 1);
#pragma unroll
				for (int w = 0; w < 2; ++w)
				{
					const uint32_t two = (r.q[w0 + w] >> shift) & 0x03030303u;
					const uint32_t high = ((r.hm[w0 + w] >> hshift) & 0x01010101u) << 2;
					bytes4(two | high, sc.s[grp], sc.b[grp], out[2 * w], out[2 * w + 1]); // (q + 4 bit - 4) d (sc - 32)
				}
			}
			static __device__ __forceinline__ void koff(int g, int s, int& k0, int& k1)
			{
				k0 = 64 * g + 8 * s;
				k1 = k0 + 4;
			}
		};

		struct Q8_0Frag
		{
			static constexpr int kChunkBytes = 8 * 34;
			static constexpr int kFragValu = 24;
			static constexpr bool kAligned16 = true;
			static constexpr bool kWideTile = false;
			struct Raw { uint32_t w[17]; }; // blocks 2g and 2g+1: 68 bytes
			struct Scale { float d0, d1; };
			static __device__ __forceinline__ Raw load(lds_bytes_t chunk, int g)
			{
				Raw r;
				lds_bytes_t p = chunk + 68 * g;
#pragma unroll
				for (int i = 0; i < 17; ++i)
				{
					r.w[i] = ld_u32_aligned(p + 4 * i);
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
			static constexpr bool kAligned16 = true;
			static constexpr bool kWideTile = true;
			struct Raw { u32x4 h; uint32_t q[8]; }; // header (d, dmin, 12 scale bytes) + the 32 nibble bytes of group g
			struct Scale { float s0, m0, s1, m1; }; // d*sc*2^24, -dmin*m of sub-block 2g; d*sc*2^20, -dmin*m of 2g+1
			static __device__ __forceinline__ Raw load(lds_bytes_t chunk, int g)
			{
				Raw r;
				r.h = *(lds_u32x4_t)(chunk);
				const u32x4 a = *(lds_u32x4_t)(chunk + 16 + 32 * g);
				const u32x4 b = *(lds_u32x4_t)(chunk + 32 + 32 * g);
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

		struct Q5_KFrag
		{
			static constexpr int kChunkBytes = 176;
			static constexpr int kFragValu = 27;
			static constexpr bool kAligned16 = true;
			static constexpr bool kWideTile = true;  // (185 VGPRs with two row groups: no spill)
			// header (d, dmin, 12 scale bytes), the 32 fifth-bit bytes, the 32 nibble bytes of group g
			struct Raw { u32x4 h; uint32_t qh[8]; uint32_t q[8]; };
			struct Scale { float s0, m0, s1, m1; int shift; }; // as Q4_K; shift = 2g, the group's bit pair in qh
			static __device__ __forceinline__ Raw load(lds_bytes_t chunk, int g)
			{
				Raw r;
				r.h = *(lds_u32x4_t)(chunk);
				const u32x4 ha = *(lds_u32x4_t)(chunk + 16);
				const u32x4 hb = *(lds_u32x4_t)(chunk + 32);
				const u32x4 a = *(lds_u32x4_t)(chunk + 48 + 32 * g);
				const u32x4 b = *(lds_u32x4_t)(chunk + 64 + 32 * g);
				r.qh[0] = ha.x, r.qh[1] = ha.y, r.qh[2] = ha.z, r.qh[3] = ha.w;
				r.qh[4] = hb.x, r.qh[5] = hb.y, r.qh[6] = hb.z, r.qh[7] = hb.w;
				r.q[0] = a.x, r.q[1] = a.y, r.q[2] = a.z, r.q[3] = a.w;
				r.q[4] = b.x, r.q[5] = b.y, r.q[6] = b.z, r.q[7] = b.w;
				return r;
			}
			static __device__ __forceinline__ Scale prep(const Raw& r, int g)
			{
				Q4_KFrag::Raw head;
				head.h = r.h;
				const Q4_KFrag::Scale s = Q4_KFrag::prep(head, g);
				return { s.s0, s.m0, s.s1, s.m1, 2 * g };
			}
			// low nibbles | bit 2g of qh: sub-block 2g, elements 4s ..; high nibbles | bit 2g+1: sub-block 2g+1.
			// The fifth bit joins its nibble inside the 16-bit lane (16 units of the nibble's own scale).
			static __device__ __forceinline__ void frag(const Raw& r, const Scale& sc, int s, uint32_t (&out)[4])
			{
				const uint32_t v = r.q[s], t = v >> 8;
				const uint32_t lo_bits = r.qh[s] >> sc.shift, hi_bits = lo_bits >> 1;
				float f0, f1, f2, f3;
				scale_pair((v & 0x000f000fu) | ((lo_bits & 0x00010001u) << 4), sc.s0, sc.m0, f0, f2);        // bytes 0, 2
				scale_pair((t & 0x000f000fu) | (((lo_bits >> 8) & 0x00010001u) << 4), sc.s0, sc.m0, f1, f3); // bytes 1, 3
				out[0] = pack_f16(f0, f1);
				out[1] = pack_f16(f2, f3);
				scale_pair((v & 0x00f000f0u) | ((hi_bits & 0x00010001u) << 8), sc.s1, sc.m1, f0, f2);
				scale_pair((t & 0x00f000f0u) | (((hi_bits >> 8) & 0x00010001u) << 8), sc.s1, sc.m1, f1, f3);
				out[2] = pack_f16(f0, f1);
				out[3] = pack_f16(f2, f3);
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
			static constexpr bool kAligned16 = false; // 210-byte blocks: 2-byte aligned
			static constexpr bool kWideTile = false;
			// lane g = 2h + j covers l in [16j, 16j + 16) of half h: 16 bytes of each ql half-row,
			// 16 bytes of qh, the four scales 8h + j + 2i and d
			struct Raw { uint32_t la[4], lb[4], qh[4]; uint32_t sc[4]; uint32_t d; };
			struct Scale { float s[4], b[4]; }; // d*scale*2^24 and -32*d*scale per quarter
			static __device__ __forceinline__ Raw load(lds_bytes_t chunk, int g)
			{
				const int h = g >> 1, j = g & 1;
				Raw r;
				lds_bytes_t ql = chunk + 64 * h + 16 * j;
				lds_bytes_t qh = chunk + 128 + 32 * h + 16 * j;
#pragma unroll
				for (int i = 0; i < 4; ++i)
				{
					r.la[i] = ld_u32(ql + 4 * i);
					r.lb[i] = ld_u32(ql + 32 + 4 * i);
					r.qh[i] = ld_u32(qh + 4 * i);
				}
				lds_bytes_t sc = chunk + 192 + 8 * h + j;
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

		// Optional producers folded into the pre-pass (they would otherwise be a launch and a pass over
		// the activations each): RMSNorm with f64 accumulation and the f32 result the stand-alone kernel
		// gives (ComputePrimitives.h:792-817), or SwiGLU's silu(gate) * up with its separately rounded
		// steps (Activation.h:22-35,56-63; SwiGLU.h:63-66).  The row stays in registers throughout.
		constexpr int kHeldItems = 8; // 8-element items per thread held in registers: rows up to 16384 wide

		template <typename F>
		__device__ __forceinline__ void to_half_body(const float* __restrict__ x, uint8_t* __restrict__ xf,
		                                             float* __restrict__ unscale, int m, int k,
		                                             const float* __restrict__ norm_w, double eps,
		                                             const float* __restrict__ up, float (&red)[4], double (&red64)[4])
		{
			// Eight consecutive rows of a tile share every 128-byte line of the fragment layout (16 bytes
			// each).  Workgroups go to the eight XCDs round-robin in the order of blockIdx.x and the L2s
			// are not coherent with each other, so with one row per workgroup in that order every line
			// would be put together in memory from eight partial writes; with a row count that is a
			// multiple of 64, XCD x takes the row octets x, x + 8, ... instead, eight workgroups that
			// follow each other on that XCD per octet, and its L2 writes whole lines.
			int row = blockIdx.x;
			if ((gridDim.x & 63) == 0)
			{
				const int xcd = row & 7, nth = row >> 3;
				row = (((nth >> 3) << 3) + xcd) * 8 + (nth & 7);
			}

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
			float held[kHeldItems][8];
			// element offsets of item `it`: 0..3 at k0, 4..7 at k1
			const auto offsets = [&](int it, int& o0, int& o1) {
				const int c = it >> 5, st = (it >> 2) & 7, g = it & 3;
				int k0, k1;
				F::koff(g, st, k0, k1);
				o0 = c * kChunk + k0;
				o1 = c * kChunk + k1;
			};
			double ss = 0.0;
#pragma unroll
			for (int u = 0; u < kHeldItems; ++u)
			{
				const int it = threadIdx.x + 256 * u;
				if (it < items)
				{
					int o0, o1;
					offsets(it, o0, o1);
					const float4 a = *reinterpret_cast<const float4*>(src + o0);
					const float4 b = *reinterpret_cast<const float4*>(src + o1);
					held[u][0] = a.x, held[u][1] = a.y, held[u][2] = a.z, held[u][3] = a.w;
					held[u][4] = b.x, held[u][5] = b.y, held[u][6] = b.z, held[u][7] = b.w;
					if (up)
					{
						const float4 ua = *reinterpret_cast<const float4*>(up + static_cast<size_t>(row) * k + o0);
						const float4 ub = *reinterpret_cast<const float4*>(up + static_cast<size_t>(row) * k + o1);
						const float uu[8] = { ua.x, ua.y, ua.z, ua.w, ub.x, ub.y, ub.z, ub.w };
#pragma unroll
						for (int e = 0; e < 8; ++e)
						{
							const float gv = held[u][e];
							const float sig = __fdiv_rn(1.0f, __fadd_rn(1.0f, expf(-gv)));
							held[u][e] = __fmul_rn(__fmul_rn(gv, sig), uu[e]);
						}
					}
					if (norm_w)
					{
#pragma unroll
						for (int e = 0; e < 8; ++e)
						{
							const double v = static_cast<double>(held[u][e]);
							ss += v * v;
						}
					}
				}
			}
			if (norm_w)
			{
				for (int off = 32; off > 0; off >>= 1)
				{
					ss += __shfl_xor(ss, off, 64);
				}
				if ((threadIdx.x & 63) == 0)
				{
					red64[threadIdx.x >> 6] = ss;
				}
				__syncthreads();
				const double total = red64[0] + red64[1] + red64[2] + red64[3];
				const double inv = 1.0 / sqrt(total / static_cast<double>(k) + eps);
#pragma unroll
				for (int u = 0; u < kHeldItems; ++u)
				{
					const int it = threadIdx.x + 256 * u;
					if (it < items)
					{
						int o0, o1;
						offsets(it, o0, o1);
						const float4 wa = *reinterpret_cast<const float4*>(norm_w + o0);
						const float4 wb = *reinterpret_cast<const float4*>(norm_w + o1);
						const float ww[8] = { wa.x, wa.y, wa.z, wa.w, wb.x, wb.y, wb.z, wb.w };
#pragma unroll
						for (int e = 0; e < 8; ++e)
						{
							held[u][e] = static_cast<float>(static_cast<double>(held[u][e]) * inv * static_cast<double>(ww[e]));
						}
					}
				}
			}
			float mx = 0.0f;
#pragma unroll
			for (int u = 0; u < kHeldItems; ++u)
			{
				if (threadIdx.x + 256 * u < items)
				{
#pragma unroll
					for (int e = 0; e < 8; ++e)
					{
						mx = fmaxf(mx, fabsf(held[u][e]));
					}
				}
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
#pragma unroll
			for (int u = 0; u < kHeldItems; ++u)
			{
				const int it = threadIdx.x + 256 * u;
				if (it < items)
				{
					const int c = it >> 5, st = (it >> 2) & 7, g = it & 3;
					u32x4 out;
					out.x = pack_f16(ldexpf(held[u][0], shift), ldexpf(held[u][1], shift));
					out.y = pack_f16(ldexpf(held[u][2], shift), ldexpf(held[u][3], shift));
					out.z = pack_f16(ldexpf(held[u][4], shift), ldexpf(held[u][5], shift));
					out.w = pack_f16(ldexpf(held[u][6], shift), ldexpf(held[u][7], shift));
					*reinterpret_cast<u32x4*>(tile_row + (c * 8 + st) * kFragBytes + g * 256) = out;
				}
			}
			if (threadIdx.x == 0)
			{
				unscale[row] = ldexpf(1.0f, -shift);
			}
		}

		template <typename F>
		__global__ __launch_bounds__(256) void to_half_kernel(const float* __restrict__ x, uint8_t* __restrict__ xf,
		                                                       float* __restrict__ unscale, int m, int k,
		                                                       const float* __restrict__ norm_w, double eps,
		                                                       const float* __restrict__ up)
		{
			__shared__ float red[4];
			__shared__ double red64[4];
			to_half_body<F>(x, xf, unscale, m, k, norm_w, eps, up, red, red64);
		}

		// The same rows in the fragment orders of two formats (matrices of two formats that share their
		// activations and one GEMM launch): grid y picks the format, each with its own destination.
		template <typename F0, typename F1>
		__global__ __launch_bounds__(256) void to_half_pair_kernel(const float* __restrict__ x, uint8_t* __restrict__ xf0,
		                                                            uint8_t* __restrict__ xf1, float* __restrict__ unscale0,
		                                                            float* __restrict__ unscale1, int m, int k,
		                                                            const float* __restrict__ norm_w, double eps)
		{
			__shared__ float red[4];
			__shared__ double red64[4];
			if (blockIdx.y == 0)
			{
				to_half_body<F0>(x, xf0, unscale0, m, k, norm_w, eps, nullptr, red, red64);
			}
			else
			{
				to_half_body<F1>(x, xf1, unscale1, m, k, norm_w, eps, nullptr, red, red64);
			}
		}

		// ---- the GEMM ---------------------------------------------------------------------------
		// grid (ceil(N / (16 WAVES NG)), ceil(M_tiles / MT)); block 64 WAVES; MT 16-row activation
		// tiles and NG 16-row weight groups per wavefront.
		//
		// Everything reaches the CU by direct-to-LDS loads, issued with inline assembly and waited for
		// with explicit vmcnt counts (the compiler, seeing such loads, would turn every later LDS wait
		// into a wait for everything outstanding):
		//   * activations: half a chunk (four MFMA steps, MT x 4 KB, already in fragment order) per
		//     buffer, three buffers, so the half needed next but one is requested while the current
		//     one is multiplied;
		//   * weights: each wavefront has one private slot holding the raw blocks of its 16 NG rows for
		//     one chunk (rows back to back, as 16-byte pieces from a 16-byte aligned start), requested
		//     for chunk c + 1 as soon as chunk c's bytes have been moved to registers.
		// Inside a chunk the eight MFMA steps are software-pipelined: while the NG x MT MFMAs of step s
		// run, every activation fragment is refilled from LDS for step s + 1 right after its last use
		// and the weight fragments of step s + 1 are decoded, the three instruction streams
		// interleaved by scheduling directives.  One barrier per half chunk: it publishes the next
		// half's activations and frees the buffer of the previous one.
		// The direct-to-LDS loads below set M0 themselves and say so in their clobber lists; clang
		// warns that it does not save a reserved register around such a statement.  Nothing else in
		// this kernel lives in M0 (no other LDS-DMA, no register-indexed arrays).
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
		template <int N>
		__device__ __forceinline__ void vm_wait()
		{
			asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
		}

		template <typename F>
		constexpr int weight_pieces() // 16-byte pieces per row and chunk in the LDS slot
		{
			return fetch::gemm_weight_pieces(F::kChunkBytes, F::kAligned16);
		}

		constexpr size_t kLdsLimit = 160 * 1024;

		// KS: groups of WAVES / KS wavefronts that share a tile and split its K walk (each group has its own
		// ring of activation buffers)
		template <typename F, int MT, int NG, int WAVES, int KS = 1>
		constexpr size_t gemm_lds_bytes()
		{
			return static_cast<size_t>(KS) * 3 * MT * 4 * kFragBytes + static_cast<size_t>(WAVES) * NG * 16 * 16 * weight_pieces<F>();
		}

		// Up to three matrices of one format and width that share the activations (q/k/v, gate/up):
		// their row blocks are laid side by side along grid x.
		struct GemmMats
		{
			const uint8_t* w[3];
			float* y[3];
			int n[3];
			int first_block[3]; // grid x index of each matrix's first row block (INT_MAX when unused)
			float* partial;     // [grid z - 1][M, n[0]]: products of the later K ranges of a split walk (single matrix)
		};

		// Workgroup numbering of the tiled GEMM
		__device__ __forceinline__ void gemm_grid_position(int& grid_x, int& grid_y)
		{
			// Workgroups are dispatched in the order x + gridDim.x * y and dealt out to the eight XCDs
			// (each with its own L2) round-robin.  The workgroups that share a strip of weight rows (one
			// per block of activation rows) are therefore numbered so that they follow each other on one
			// XCD: number L takes strip 8 (L / (8 gy)) + L % 8 and row block (L / 8) % gy.  Numbered plainly
			// they sit on one XCD too when gridDim.x is a multiple of 8, but a launch of more workgroups
			// than CUs reaches a strip's later row blocks only in its second round and fetches the strip
			// again (8B-shape gate/up at 512 rows: 166 MB fetched for 66 MB of weights).
			grid_x = blockIdx.x, grid_y = blockIdx.y;
			if (gridDim.y > 1)
			{
				const int gx = gridDim.x, gy = gridDim.y;
				const int full = gx & ~7;
				const int L = grid_x + gx * grid_y;
				if (L < full * gy)
				{
					grid_x = (L / (8 * gy)) * 8 + (L & 7);
					grid_y = (L >> 3) % gy;
				}
				else
				{
					const int rem = gx - full, l2 = L - full * gy;
					grid_x = full + l2 % rem;
					grid_y = l2 / rem;
				}
			}
		}

		// The matrix strip grid_x of a launch belongs to (selects, so that the argument block stays where it is)
#define LITENN_GEMM_PICK_MATRIX(mats, grid_x)                                                                         \
	const int which = ((grid_x) >= (mats).first_block[1]) + ((grid_x) >= (mats).first_block[2]);                       \
	const uint8_t* w = which == 0 ? (mats).w[0] : (which == 1 ? (mats).w[1] : (mats).w[2]);                            \
	float* y = which == 0 ? (mats).y[0] : (which == 1 ? (mats).y[1] : (mats).y[2]);                                    \
	const int n = which == 0 ? (mats).n[0] : (which == 1 ? (mats).n[1] : (mats).n[2]);                                 \
	const int block_x = (grid_x) - (which == 0 ? 0 : (which == 1 ? (mats).first_block[1] : (mats).first_block[2]))

		// One workgroup's tile: strip block_x of the n-row matrix w against row block grid_y.
		// GATED (two weight groups per wavefront): the second group holds the same rows of a second
		// matrix w_up, and what is stored is silu(x . w^T) * (x . w_up^T), SwiGLU's product with its
		// separately rounded steps (Activation.h:22-35,56-63; SwiGLU.h:63-66), to the single output y.
		// KS = 2: the workgroup's wavefronts form two groups that work on the same tile; group 0 walks the
		// first half of the workgroup's K range and group 1 the second, each through its own three
		// activation buffers, and group 1's accumulators are added to group 0's through LDS before the
		// tile is stored.  A tile that gives a CU one wavefront per SIMD (64 x 64 outputs, four wavefronts)
		// is bound by that wavefront's in-order instruction stream; this puts a second one beside it
		// without a second product in memory.  The two groups pass the same barriers, so their ranges
		// must hold the same number of chunks (the launcher sees to it).
		template <typename F, int MT, int NG, int WAVES, bool GATED = false, int KS = 1>
		__device__ __forceinline__ void gemm_q_body(const uint8_t* w, const uint8_t* w_up, float* y, int n, int block_x,
		                                            float* partial, const uint8_t* __restrict__ xf,
		                                            const float* __restrict__ unscale,
		                                            const float* __restrict__ residual, int k, int m, int m_tiles,
		                                            size_t row_bytes, int grid_y)
		{
			constexpr int kHalfBytes = MT * 4 * kFragBytes; // one activation buffer: four steps of MT tiles
			constexpr int WG = WAVES / KS;                  // wavefronts that share one K range
			static_assert(WG * KS == WAVES && (KS == 1 || (KS == 2 && !GATED)), "K groups");
			constexpr int kXLoads = MT * 4 / WG;            // 1 KB pieces a wavefront moves per half
			static_assert(kXLoads >= 1 && kXLoads * WG == MT * 4, "activation pieces / wavefront split");
			constexpr int P = weight_pieces<F>();
			constexpr int kRowStride = 16 * P;              // bytes of one row's chunk in the slot
			constexpr int kSlotBytes = NG * 16 * kRowStride;
			constexpr int kWLoads = (NG * 16 * P + 63) / 64;
			extern __shared__ __attribute__((aligned(16))) uint8_t lds[]; // [KS][3][kHalfBytes][WAVES][kSlotBytes]
			const int lane = threadIdx.x & 63;
			const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
			const int kgroup = KS == 1 ? 0 : wave / WG; // which K range of the workgroup's
			const int wv = KS == 1 ? wave : wave % WG;  // wavefront within its group
			const int r = lane & 15, g = lane >> 4;
			static_assert(!GATED || NG == 2, "the gated form pairs the two weight groups of a wavefront");
			const int n_base = (block_x * WG + wv) * 16 * (GATED ? 1 : NG);
			const int mt_base = grid_y * MT;
			const int chunks = k / kChunk;
			// grid z (and the workgroup's K groups) split the K walk: these wavefronts multiply chunks
			// [c_begin, c_end)
			const int k_part = static_cast<int>(blockIdx.z) * KS + kgroup;
			const int k_parts = static_cast<int>(gridDim.z) * KS;
			const fetch::ChunkRange my_chunks = fetch::gemm_chunk_range(k_part, k_parts, chunks);
			const int c_begin = my_chunks.begin;
			const int c_end = my_chunks.end;
			constexpr int kXRegion = KS * 3 * kHalfBytes; // every group's three activation buffers
			const int x_group = kgroup * 3 * kHalfBytes;  // this group's
			const uint32_t lds_base =
			    static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) const uint8_t*)(lds)));
			const uint32_t slot_lds = lds_base + kXRegion + wave * kSlotBytes;
			const uint32_t lane_off = lane * 16;

			// ---- activation requests: piece i * WAVES + wave of the half (tile t = piece / 4, step
			// piece % 4); tiles past the end re-read the last one.  Offsets are wavefront-uniform.
			uint32_t x_off[kXLoads];
#pragma unroll
			for (int i = 0; i < kXLoads; ++i)
			{
				const int piece = i * WG + wv;
				const int t = min(mt_base + (piece >> 2), m_tiles - 1);
				x_off[i] = static_cast<uint32_t>(t * chunks) * kChunkTileBytes + (piece & 3) * kFragBytes;
			}
			const auto issue_x = [&](int half, int buf_off) {
#pragma unroll
				for (int i = 0; i < kXLoads; ++i)
				{
					const int piece = i * WG + wv;
					const uint8_t* src = xf + (x_off[i] + static_cast<uint32_t>(half) * (4 * kFragBytes));
					const uint32_t dst = lds_base + x_group + buf_off + piece * kFragBytes;
					asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
					             :
					             : "s"(dst), "v"(lane_off), "s"(src)
					             : "memory", "m0");
				}
			};

			// ---- weight requests: piece p = 64 i + lane of the slot is piece p % P of row p / P; a
			// row's pieces start at the 16-byte boundary at or below its chunk (an aligned piece that
			// holds a byte of the tensor lies in that byte's page, so nothing outside the tensor's
			// pages is touched).  Rows past the end re-read the last row; their results are never
			// stored.
			// The address arithmetic lives in fetch_model.hpp, where a host test runs it for every
			// thread of a launch.
			const uint8_t* w_src[kWLoads]; // the row's chunk 0
			int w_piece[kWLoads];          // 16 j
			bool w_issued[kWLoads];
#pragma unroll
			for (int i = 0; i < kWLoads; ++i)
			{
				const fetch::GemmWeightRequest rq = fetch::gemm_weight_request(i, lane, NG, P);
				w_piece[i] = rq.offset;
				w_issued[i] = rq.issued;
				// (gated: slot rows 16 .. 31 are rows 0 .. 15 of the second matrix)
				w_src[i] = (GATED && rq.row >= 16 ? w_up : w) +
				           static_cast<size_t>(fetch::gemm_weight_row(n_base, GATED ? (rq.row & 15) : rq.row, n)) * row_bytes;
			}
			const auto issue_w = [&](int c) {
#pragma unroll
				for (int i = 0; i < kWLoads; ++i)
				{
					if (64 * (i + 1) <= NG * 16 * P || w_issued[i])
					{
						const uint8_t* src = reinterpret_cast<const uint8_t*>(fetch::gemm_weight_piece(
						    reinterpret_cast<uintptr_t>(w_src[i]), c, F::kChunkBytes, F::kAligned16, w_piece[i]));
						const uint32_t dst = slot_lds + i * 1024;
						asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
						             :
						             : "s"(dst), "v"(src)
						             : "memory", "m0");
					}
				}
			};
			// this lane's row of group q inside the slot
			lds_bytes_t slot_rows[NG];
#pragma unroll
			for (int q = 0; q < NG; ++q)
			{
				slot_rows[q] = (lds_bytes_t)(lds) + kXRegion + wave * kSlotBytes + (16 * q + r) * kRowStride;
			}
			const uint8_t* lane_rows[NG]; // for the misalignment of a chunk start
#pragma unroll
			for (int q = 0; q < NG; ++q)
			{
				lane_rows[q] = (GATED && q == 1 ? w_up : w) +
				               static_cast<size_t>(fetch::gemm_weight_row(n_base, GATED ? r : 16 * q + r, n)) * row_bytes;
			}

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
			typename F::Raw raw[NG];
			typename F::Scale sc[NG];
			const auto lane_x = (lds_bytes_t)(lds) + x_group + lane * 16;
			const auto read_b = [&](int t, int buf_off, int s4) {
				b[t] = *(lds_u32x4_t)(lane_x + buf_off + t * (4 * kFragBytes) + s4 * kFragBytes);
			};
			const auto decode = [&](half8 (&a)[NG], int s) {
#pragma unroll
				for (int q = 0; q < NG; ++q)
				{
					uint32_t pk[4];
					F::frag(raw[q], sc[q], s, pk);
					const u32x4 v = { pk[0], pk[1], pk[2], pk[3] };
					a[q] = __builtin_bit_cast(half8, v);
				}
			};
			const auto load_raw = [&](int c) {
#pragma unroll
				for (int q = 0; q < NG; ++q)
				{
					const int mis = fetch::gemm_weight_misalignment(reinterpret_cast<uintptr_t>(lane_rows[q]), c,
					                                                F::kChunkBytes, F::kAligned16);
					raw[q] = F::load(slot_rows[q] + mis, g);
					sc[q] = F::prep(raw[q], g);
				}
			};
			// the MFMAs of the current step; fragment t is refilled from (buf_off, s4) right after its
			// last use
			const auto mfma_step = [&](bool refill, int buf_off, int s4) {
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
						read_b(t, buf_off, s4);
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
			const auto interleave = [&](auto extra_valu_tag) {
				constexpr int valu_per_tile = (F::kFragValu * NG + decltype(extra_valu_tag)::value + MT - 1) / MT;
#pragma unroll
				for (int t = 0; t < MT; ++t)
				{
					__builtin_amdgcn_sched_group_barrier(0x008, NG, 0);            // the MFMAs of one activation fragment
					__builtin_amdgcn_sched_group_barrier(0x100, 1, 0);             // its refill from LDS
					__builtin_amdgcn_sched_group_barrier(0x002, valu_per_tile, 0); // a share of the decode arithmetic
				}
			};
			const auto plain_step = [&](int buf_off, int s) { // steps 0..2 and 4..6: refill from the same half
				decode(a_nxt, s + 1);
				mfma_step(true, buf_off, (s + 1) & 3);
				interleave(std::integral_constant<int, 0>{});
				__builtin_amdgcn_sched_barrier(0);
				rotate();
			};

			// Half h of the K walk lives in buffer h % 3.  `cur`, `nxt`, `far` are the byte offsets of
			// the buffers of the current half, the next and the one after; they rotate per half.
			int cur = 0, nxt = kHalfBytes, far = 2 * kHalfBytes;
			const auto rotate_buffers = [&]() {
				const int t = cur;
				cur = nxt;
				nxt = far;
				far = t;
			};
			const auto chunk = [&](auto has_next_tag, int c) {
				constexpr bool has_next = decltype(has_next_tag)::value;
				// first half: steps 0..3 out of `cur`
				if (has_next)
				{
					issue_x(2 * c + 2, far);
					// The weight slot is about to be overwritten: the reads that moved chunk c out of it
					// (issued one step ago, waited for only as the decode needs them) must have returned.
					// Under LDS contention a late read can otherwise meet a request served from L2.
					asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
					issue_w(c + 1);
				}
				plain_step(cur, 0);
				plain_step(cur, 1);
				plain_step(cur, 2);
				// the second half of this chunk (requested one half ago) must be complete, in every
				// wavefront's share; what was requested at the top of this half may stay in flight
				if (has_next)
				{
					vm_wait<kXLoads + kWLoads>();
				}
				else
				{
					vm_wait<0>();
				}
				__syncthreads();
				decode(a_nxt, 4);
				mfma_step(true, nxt, 0);
				interleave(std::integral_constant<int, 0>{});
				__builtin_amdgcn_sched_barrier(0);
				rotate();
				rotate_buffers();
				// second half: steps 4..7; the barrier above freed the buffer of the previous half
				if (has_next)
				{
					issue_x(2 * c + 3, far);
				}
				plain_step(cur, 4);
				plain_step(cur, 5);
				plain_step(cur, 6);
				if (has_next)
				{
					// next chunk: its first half and its weights have landed
					vm_wait<kXLoads>();
					__syncthreads();
					load_raw(c + 1);
					decode(a_nxt, 0);
					mfma_step(true, nxt, 0);
					interleave(std::integral_constant<int, 16 * NG>{});
					__builtin_amdgcn_sched_barrier(0);
					rotate();
					rotate_buffers();
				}
				else
				{
					mfma_step(false, 0, 0);
				}
			};

			issue_w(c_begin);
			issue_x(2 * c_begin, 0);
			issue_x(2 * c_begin + 1, kHalfBytes);
			vm_wait<0>();
			__syncthreads();
			load_raw(c_begin);
#pragma unroll
			for (int t = 0; t < MT; ++t)
			{
				read_b(t, 0, 0);
			}
			decode(a_cur, 0);
			using std::false_type;
			using std::true_type;
			int c = c_begin;
			for (; c + 1 < c_end; ++c)
			{
				chunk(true_type{}, c);
			}
			chunk(false_type{}, c);

			if constexpr (KS == 2)
			{
				// group 1 hands its accumulators to group 0 through the activation buffers, which are idle
				// once every wavefront has passed the first barrier; a lane's 16 bytes per accumulator lie
				// lane by lane (no bank conflicts).  K order: group 0's range, then group 1's.
				__syncthreads();
				auto* const handed = reinterpret_cast<floatx4*>(lds) + (wv * (NG * MT)) * 64 + lane;
				if (kgroup == 1)
				{
#pragma unroll
					for (int q = 0; q < NG; ++q)
					{
#pragma unroll
						for (int t = 0; t < MT; ++t)
						{
							handed[(q * MT + t) * 64] = acc[q][t];
						}
					}
				}
				__syncthreads();
				if (kgroup == 1)
				{
					return;
				}
#pragma unroll
				for (int q = 0; q < NG; ++q)
				{
#pragma unroll
					for (int t = 0; t < MT; ++t)
					{
						acc[q][t] += handed[(q * MT + t) * 64];
					}
				}
				static_assert(static_cast<size_t>(WG) * NG * MT * 64 * 16 <= static_cast<size_t>(kXRegion), "hand-over fits the activation buffers");
			}

			// D layout: lane holds activation row j = lane % 16 and weight rows 4 (lane / 16) + 0..3
			const bool vec_ok = (n & 3) == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0 &&
			                    (!residual || (reinterpret_cast<uintptr_t>(residual) & 15) == 0);
			// tile by tile, the weight groups of a tile back to back: a lane's 16 bytes, its three
			// neighbours' and the next group's make one 128-byte line of an output row, and stores that
			// follow each other closely are combined before they leave the L2
			if constexpr (GATED)
			{
#pragma unroll
				for (int t = 0; t < MT; ++t)
				{
					const int n0 = n_base + 4 * g;
					const int mm = (mt_base + t) * 16 + r;
					if (mm < m)
					{
						float* dst = y + static_cast<size_t>(mm) * n + n0;
						const float us = unscale[mm];
						const float gate[4] = { acc[0][t].x * us, acc[0][t].y * us, acc[0][t].z * us, acc[0][t].w * us };
						const float upv[4] = { acc[1][t].x * us, acc[1][t].y * us, acc[1][t].z * us, acc[1][t].w * us };
						float vals[4];
#pragma unroll
						for (int e = 0; e < 4; ++e)
						{
							const float sig = __fdiv_rn(1.0f, __fadd_rn(1.0f, expf(-gate[e])));
							vals[e] = __fmul_rn(__fmul_rn(gate[e], sig), upv[e]);
						}
						if (vec_ok && n0 + 3 < n)
						{
							*reinterpret_cast<float4*>(dst) = float4{ vals[0], vals[1], vals[2], vals[3] };
						}
						else
						{
#pragma unroll
							for (int e = 0; e < 4; ++e)
							{
								if (n0 + e < n)
								{
									dst[e] = vals[e];
								}
							}
						}
					}
				}
				return;
			}
#pragma unroll
			for (int t = 0; t < MT; ++t)
			{
#pragma unroll
				for (int q = 0; q < NG; ++q)
				{
					const int n0 = n_base + 16 * q + 4 * g;
					const int mm = (mt_base + t) * 16 + r;
					if (mm < m)
					{
						// the second K range of a split walk leaves its product beside y (no residual)
						float* dst = (blockIdx.z == 0 ? y : partial + (blockIdx.z - 1) * (static_cast<size_t>(m) * n)) +
						             static_cast<size_t>(mm) * n + n0;
						const float* res =
						    residual && blockIdx.z == 0 ? residual + static_cast<size_t>(mm) * n + n0 : nullptr;
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

		template <typename F, int MT, int NG, int WAVES, int KS = 1>
		__global__ __launch_bounds__(64 * WAVES) void gemm_q_kernel(const GemmMats mats, const uint8_t* __restrict__ xf,
		                                                             const float* __restrict__ unscale,
		                                                             const float* __restrict__ residual, int k, int m,
		                                                             int m_tiles, size_t row_bytes)
		{
			int grid_x, grid_y;
			gemm_grid_position(grid_x, grid_y);
			LITENN_GEMM_PICK_MATRIX(mats, grid_x);
			gemm_q_body<F, MT, NG, WAVES, false, KS>(w, nullptr, y, n, block_x, mats.partial, xf, unscale, residual, k, m,
			                                         m_tiles, row_bytes, grid_y);
		}

		// gate (mats.w[0]) and up (mats.w[1]) projections of n[0] rows each with SwiGLU's product in the
		// epilogue: y[0][M, n[0]] = silu(x . gate^T) * (x . up^T); strips along grid x are strips of both
		template <typename F, int MT, int WAVES>
		__global__ __launch_bounds__(64 * WAVES) void gemm_q_gated_kernel(const GemmMats mats,
		                                                                   const uint8_t* __restrict__ xf,
		                                                                   const float* __restrict__ unscale, int k, int m,
		                                                                   int m_tiles, size_t row_bytes)
		{
			int grid_x, grid_y;
			gemm_grid_position(grid_x, grid_y);
			gemm_q_body<F, MT, 2, WAVES, true>(mats.w[0], mats.w[1], mats.y[0], mats.n[0], grid_x, mats.partial, xf, unscale,
			                                   nullptr, k, m, m_tiles, row_bytes, grid_y);
		}

		// Matrices of two formats that share their activations (q and k in one, v in another): the
		// strips from `second_block` on belong to the second format, which reads its own copy of the
		// activations (its decoder's fragment order) and its own row size.  A workgroup runs one of the
		// two bodies; the branch is uniform.
		template <typename F0, typename F1, int MT, int NG, int WAVES>
		__global__ __launch_bounds__(64 * WAVES) void gemm_q_pair_kernel(const GemmMats mats, int second_block,
		                                                                  const uint8_t* __restrict__ xf0,
		                                                                  const uint8_t* __restrict__ xf1,
		                                                                  const float* __restrict__ unscale0,
		                                                                  const float* __restrict__ unscale1, int k,
		                                                                  int m, int m_tiles, size_t row_bytes0,
		                                                                  size_t row_bytes1)
		{
			int grid_x, grid_y;
			gemm_grid_position(grid_x, grid_y);
			LITENN_GEMM_PICK_MATRIX(mats, grid_x);
			// (grid z is 1 here and mats.partial unused; a literal null in its place makes this
			// compiler's inliner fall over)
			if (grid_x < second_block)
			{
				gemm_q_body<F0, MT, NG, WAVES>(w, nullptr, y, n, block_x, mats.partial, xf0, unscale0, nullptr, k, m, m_tiles,
				                               row_bytes0, grid_y);
			}
			else
			{
				gemm_q_body<F1, MT, NG, WAVES>(w, nullptr, y, n, block_x, mats.partial, xf1, unscale1, nullptr, k, m, m_tiles,
				                               row_bytes1, grid_y);
			}
		}

#undef LITENN_GEMM_PICK_MATRIX

		// ---- the GEMM for few activation rows ------------------------------------------------------
		// With 16 or 32 activation rows the product is a stream of the weights, like the single-row
		// GEMV, and is built like it: one workgroup of eight or sixteen wavefronts per CU, always a single round,
		// each workgroup owning a run of consecutive weight rows.  The rows are walked in tiles of 16;
		// wavefront w multiplies the tile's chunks [w CPW, (w + 1) CPW) of K, whose activation
		// fragments (already fp16, in MFMA order) it holds in registers for the whole launch, and
		// keeps PD tiles' worth of its slice of the raw blocks in flight towards its LDS slots with
		// direct-to-LDS loads.  The wavefronts' partial products of a tile meet in LDS and are added in
		// wavefront order, so the result does not depend on scheduling.  One launch, no second pass
		// over y, every weight byte read once.
		constexpr int kStreamTilesInFlight = 2;

		struct GemmStreamArgs
		{
			const uint8_t* w;
			float* y;
			const uint8_t* xf;
			const float* unscale;
			const float* residual;
			int n, k, m, m_tiles;
			size_t row_bytes;
			int rows_per_block; // consecutive weight rows of a workgroup, a multiple of 4
			int round_tiles;    // tiles whose partial products LDS holds before they are added and stored
		};

		template <typename F, int CPW>
		constexpr int stream_slot_bytes()
		{
			return 16 * 16 * fetch::gemm_weight_pieces(CPW * F::kChunkBytes, F::kAligned16);
		}

		template <typename F, int MT, int CPW, int kStreamWaves>
		__global__ __launch_bounds__(64 * kStreamWaves) void gemm_stream_kernel(const GemmStreamArgs a)
		{
			constexpr int PD = kStreamTilesInFlight;
			constexpr int kSliceBytes = CPW * F::kChunkBytes; // a wavefront's share of one row
			constexpr int P = fetch::gemm_weight_pieces(kSliceBytes, F::kAligned16);
			constexpr int kRowStride = 16 * P;
			constexpr int kSlotBytes = 16 * kRowStride;
			constexpr int kWLoads = (16 * P + 63) / 64;
			static_assert(kSlotBytes == stream_slot_bytes<F, CPW>(), "slot size");
			static_assert(PD * kWLoads <= 63, "vmcnt range");
			extern __shared__ __attribute__((aligned(16))) uint8_t lds[]; // [waves][PD][slot] [round][waves][MT][1 KB]
			const int lane = threadIdx.x & 63;
			const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
			const int r = lane & 15, g = lane >> 4;
			const int chunks = a.k / kChunk;
			const int row0 = static_cast<int>(blockIdx.x) * a.rows_per_block;
			const int block_rows = min(a.rows_per_block, a.n - row0);
			const int last_row = row0 + block_rows - 1;
			const int tiles = (block_rows + 15) >> 4;
			const uint32_t lds_base =
			    static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) const uint8_t*)(lds)));
			const uint32_t slots_lds = lds_base + wave * (PD * kSlotBytes);
			const int part_base = kStreamWaves * PD * kSlotBytes;

			// ---- weight requests: piece p = 64 i + lane of a slot is piece p % P of tile row p / P.
			// Rows past the workgroup's run re-read its last row (same bytes as a neighbouring lane:
			// no further traffic); their products are never stored.  The address arithmetic is the
			// matrix-core GEMM's (fetch_model.hpp) with the wavefront's slice in the place of a chunk.
			int w_row[kWLoads], w_piece[kWLoads];
			bool w_issued[kWLoads];
#pragma unroll
			for (int i = 0; i < kWLoads; ++i)
			{
				const fetch::GemmWeightRequest rq = fetch::gemm_weight_request(i, lane, 1, P);
				w_row[i] = rq.row;
				w_piece[i] = rq.offset;
				w_issued[i] = rq.issued;
			}
			const auto issue_tile = [&](int t, int slot) {
#pragma unroll
				for (int i = 0; i < kWLoads; ++i)
				{
					if (64 * (i + 1) <= 16 * P || w_issued[i])
					{
						const int row = fetch::gemm_weight_row(row0 + 16 * t, w_row[i], last_row + 1);
						const uint8_t* row_start = a.w + static_cast<size_t>(row) * a.row_bytes;
						const uint8_t* src = reinterpret_cast<const uint8_t*>(fetch::gemm_weight_piece(
						    reinterpret_cast<uintptr_t>(row_start), wave, kSliceBytes, F::kAligned16, w_piece[i]));
						const uint32_t dst = slots_lds + slot * kSlotBytes + i * 1024;
						asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
						             :
						             : "s"(dst), "v"(src)
						             : "memory", "m0");
					}
				}
			};
			// ---- this wavefront's activation fragments: chunks [wave CPW, (wave + 1) CPW), every step,
			// MT tiles (a tile past the end repeats the last one; its products are not stored), and the
			// factor that undoes the pre-pass's scaling of this thread's activation row (the same row in
			// every round: MT divides the number of wavefronts).  They are requested before the first
			// weight tiles: a wavefront's loads return in order, the fragments come from the L2 the
			// pre-pass left them in, and behind the tiles they would arrive a memory latency later
			// than they could.  The loads are issued from assembly like the tiles' so that the wait
			// below can let the tiles stay in flight; a wait of the compiler's own would cover
			// everything outstanding.
			u32x4 b[CPW][8][MT];
#pragma unroll
			for (int ci = 0; ci < CPW; ++ci)
			{
#pragma unroll
				for (int t = 0; t < MT; ++t)
				{
					const int mt = min(t, a.m_tiles - 1);
					const uint8_t* tile = a.xf + (static_cast<size_t>(mt) * chunks + wave * CPW + ci) * kChunkTileBytes + lane * 16;
#pragma unroll
					for (int st = 0; st < 8; ++st)
					{
						asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(b[ci][st][t]) : "v"(tile + st * kFragBytes) : "memory");
					}
				}
			}
			const int my_mm = ((threadIdx.x >> 6) % MT) * 16 + (lane & 15);
			float my_unscale;
			asm volatile("global_load_dword %0, %1, off" : "=v"(my_unscale) : "v"(a.unscale + min(my_mm, 16 * a.m_tiles - 1)) : "memory");
#pragma unroll
			for (int t = 0; t < PD; ++t)
			{
				if (t < tiles) // uniform
				{
					issue_tile(t, t);
				}
			}
			// fragments and factor have landed once only the tiles requested after them are outstanding
			if (tiles >= PD)
			{
				vm_wait<PD * kWLoads>();
			}
			else
			{
				vm_wait<0>();
			}
			asm volatile("" : "+v"(my_unscale));
#pragma unroll
			for (int ci = 0; ci < CPW; ++ci)
			{
#pragma unroll
				for (int st = 0; st < 8; ++st)
				{
#pragma unroll
					for (int t = 0; t < MT; ++t)
					{
						asm volatile("" : "+v"(b[ci][st][t]));
					}
				}
			}
			static_assert(kStreamWaves % MT == 0, "a thread keeps one activation row through the rounds");

			const int round_tiles = a.round_tiles;
			const bool vec_ok = (a.n & 3) == 0 && (reinterpret_cast<uintptr_t>(a.y) & 15) == 0 &&
			                    (!a.residual || (reinterpret_cast<uintptr_t>(a.residual) & 15) == 0);
			// adds the wavefronts' partial products of tiles [first, first + count) in wavefront order and stores them
			const auto finish_round = [&](int first, int count) {
				__syncthreads();
				for (int idx = threadIdx.x; idx < count * MT * 64; idx += 64 * kStreamWaves)
				{
					const int ti = idx / (MT * 64), t = (idx >> 6) % MT, ln = idx & 63;
					const uint8_t* src = lds + part_base + ((ti * kStreamWaves) * MT + t) * 1024 + ln * 16;
					floatx4 sum = *reinterpret_cast<const floatx4*>(src);
#pragma unroll
					for (int wv = 1; wv < kStreamWaves; ++wv)
					{
						const floatx4 v = *reinterpret_cast<const floatx4*>(src + wv * MT * 1024);
						sum.x += v.x, sum.y += v.y, sum.z += v.z, sum.w += v.w;
					}
					// D layout: lane holds activation row ln % 16 and weight rows 4 (ln / 16) + 0 .. 3
					const int mm = t * 16 + (ln & 15);
					const int n0 = row0 + 16 * (first + ti) + 4 * (ln >> 4);
					if (mm < a.m && n0 <= last_row)
					{
						float* dst = a.y + static_cast<size_t>(mm) * a.n + n0;
						const float* res = a.residual ? a.residual + static_cast<size_t>(mm) * a.n + n0 : nullptr;
						const float us = my_unscale;
						const float vals[4] = { sum.x * us, sum.y * us, sum.z * us, sum.w * us };
						if (vec_ok && n0 + 3 <= last_row)
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
								if (n0 + e <= last_row)
								{
									dst[e] = res ? res[e] + vals[e] : vals[e];
								}
							}
						}
					}
				}
				__syncthreads();
			};

			int slot = 0, in_round = 0, round_first = 0;
			for (int t = 0; t < tiles; ++t)
			{
				// tile t has landed once only the tiles requested after it are outstanding
				if (t + PD - 1 < tiles)
				{
					vm_wait<(PD - 1) * kWLoads>();
				}
				else
				{
					vm_wait<0>();
				}
				const int row = fetch::gemm_weight_row(row0 + 16 * t, r, last_row + 1);
				const int mis = fetch::gemm_weight_misalignment(
				    reinterpret_cast<uintptr_t>(a.w + static_cast<size_t>(row) * a.row_bytes), wave, kSliceBytes, F::kAligned16);
				lds_bytes_t mine = (lds_bytes_t)(lds) + wave * (PD * kSlotBytes) + slot * kSlotBytes + r * kRowStride + mis;
				typename F::Raw raw[CPW];
				typename F::Scale sc[CPW];
#pragma unroll
				for (int ci = 0; ci < CPW; ++ci)
				{
					raw[ci] = F::load(mine + ci * F::kChunkBytes, g);
				}
				// the slot is free once those reads have returned: refill it before the arithmetic
				asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
				if (t + PD < tiles)
				{
					issue_tile(t + PD, slot);
				}
				floatx4 acc[MT];
#pragma unroll
				for (int mt = 0; mt < MT; ++mt)
				{
					acc[mt] = floatx4{ 0.0f, 0.0f, 0.0f, 0.0f };
				}
#pragma unroll
				for (int ci = 0; ci < CPW; ++ci)
				{
					sc[ci] = F::prep(raw[ci], g);
#pragma unroll
					for (int st = 0; st < 8; ++st)
					{
						uint32_t pk[4];
						F::frag(raw[ci], sc[ci], st, pk);
						const u32x4 v = { pk[0], pk[1], pk[2], pk[3] };
						const half8 av = __builtin_bit_cast(half8, v);
#pragma unroll
						for (int mt = 0; mt < MT; ++mt)
						{
							// D[i = weight row][j = activation row] += A[i][k] * B[k][j]
							acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, __builtin_bit_cast(half8, b[ci][st][mt]), acc[mt],
							                                                 0, 0, 0);
						}
					}
				}
#pragma unroll
				for (int mt = 0; mt < MT; ++mt)
				{
					*reinterpret_cast<floatx4*>(lds + part_base + ((in_round * kStreamWaves + wave) * MT + mt) * 1024 + lane * 16) =
					    acc[mt];
				}
				slot = slot + 1 == PD ? 0 : slot + 1;
				if (++in_round == round_tiles || t + 1 == tiles)
				{
					finish_round(round_first, in_round);
					round_first += in_round;
					in_round = 0;
				}
			}
		}

#pragma clang diagnostic pop

		// What the calling thread's last matrix-core launch was (litenn_hip_gemm_last_launch formats it)
		struct GemmLaunchRecord
		{
			const char* kernel = nullptr; // gemm_q_kernel, gemm_q_pair_kernel, gemm_q_gated_kernel or gemm_stream_kernel
			int a = 0, b = 0, c = 0, d = 0; // the instance's integer template arguments (d: K groups of a tile, 0 where there is none)
			unsigned grid_x = 0, grid_y = 0, grid_z = 0, threads = 0;
			size_t lds = 0;
		};
		thread_local GemmLaunchRecord t_last_gemm_launch;

		struct GemmCall
		{
			int count;
			const uint8_t* w[3];
			float* y[3];
			int n[3];
			const uint8_t* xf;
			const float* unscale;
			const float* residual;
			int k, m, m_tiles;
			size_t row_bytes;
			int tile;       // MT * 100 + NG * 10 + WAVES
			int k_splits;   // 1, 2 or 4 workgroups share a tile's K walk; all but the first write `partial`
			float* partial; // room for the later K ranges' products, or null: K is never split
			size_t partial_floats;
			hipStream_t stream;
		};

		template <typename F, int MT, int NG, int WAVES, int KS = 1>
		void launch_variant(const GemmCall& c)
		{
			if constexpr (KS > 1)
			{
				// the K groups of a workgroup pass the same barriers: their ranges must be equally long
				if (!fetch::gemm_ranges_equal(c.k / kChunk, c.k_splits * KS))
				{
					launch_variant<F, MT, NG, WAVES / KS, 1>(c);
					return;
				}
			}
			constexpr size_t lds = gemm_lds_bytes<F, MT, NG, WAVES, KS>();
			static_assert(lds <= kLdsLimit, "LDS budget");
			allow_dynamic_lds(reinterpret_cast<const void*>(&gemm_q_kernel<F, MT, NG, WAVES, KS>), lds);
			constexpr int bn = 16 * (WAVES / KS) * NG;
			GemmMats mats;
			mats.partial = c.partial;
			int blocks = 0;
			for (int i = 0; i < 3; ++i)
			{
				mats.w[i] = i < c.count ? c.w[i] : nullptr;
				mats.y[i] = i < c.count ? c.y[i] : nullptr;
				mats.n[i] = i < c.count ? c.n[i] : 0;
				mats.first_block[i] = i < c.count ? blocks : 0x7fffffff;
				blocks += i < c.count ? (c.n[i] + bn - 1) / bn : 0;
			}
			const dim3 grid(blocks, (c.m_tiles + MT - 1) / MT, c.k_splits);
			t_last_gemm_launch = { "gemm_q_kernel", MT, NG, WAVES, KS, grid.x, grid.y, grid.z, 64u * WAVES, lds };
			gemm_q_kernel<F, MT, NG, WAVES, KS><<<grid, dim3(64 * WAVES), lds, c.stream>>>(mats, c.xf, c.unscale, c.residual,
			                                                                              c.k, c.m, c.m_tiles, c.row_bytes);
		}

		// Two formats in one launch: matrices [0, second) in F0, [second, count) in F1, single-group tiles.
		template <typename F0, typename F1, int MT, int WAVES>
		void launch_pair_variant(const GemmCall& c, int second, const uint8_t* xf1, const float* unscale1,
		                         size_t row_bytes1)
		{
			constexpr size_t lds = std::max(gemm_lds_bytes<F0, MT, 1, WAVES>(), gemm_lds_bytes<F1, MT, 1, WAVES>());
			static_assert(lds <= kLdsLimit, "LDS budget");
			allow_dynamic_lds(reinterpret_cast<const void*>(&gemm_q_pair_kernel<F0, F1, MT, 1, WAVES>), lds);
			constexpr int bn = 16 * WAVES;
			GemmMats mats;
			mats.partial = nullptr;
			int blocks = 0;
			for (int i = 0; i < 3; ++i)
			{
				mats.w[i] = i < c.count ? c.w[i] : nullptr;
				mats.y[i] = i < c.count ? c.y[i] : nullptr;
				mats.n[i] = i < c.count ? c.n[i] : 0;
				mats.first_block[i] = i < c.count ? blocks : 0x7fffffff;
				blocks += i < c.count ? (c.n[i] + bn - 1) / bn : 0;
			}
			const dim3 grid(blocks, (c.m_tiles + MT - 1) / MT, 1);
			t_last_gemm_launch = { "gemm_q_pair_kernel", MT, 1, WAVES, 0, grid.x, grid.y, grid.z, 64u * WAVES, lds };
			gemm_q_pair_kernel<F0, F1, MT, 1, WAVES><<<grid, dim3(64 * WAVES), lds, c.stream>>>(
			    mats, mats.first_block[second], c.xf, xf1, c.unscale, unscale1, c.k, c.m, c.m_tiles, c.row_bytes, row_bytes1);
		}

		// Tile choice: MT activation tiles per workgroup so that a weight is decoded as few times as
		// possible; two weight groups per wavefront (each activation fragment read from LDS feeds two
		// MFMAs) when that still nearly fills the card.
		// y += partial[0] + partial[1] + ..., element by element in K order: the fixed order keeps the
		// result independent of scheduling
		__global__ __launch_bounds__(256) void add_partial_kernel(float* __restrict__ y, const float* __restrict__ partial,
		                                                           size_t total, int parts)
		{
			const size_t i = (static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x) * 4;
			if (i + 3 < total && (total & 3) == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0 &&
			    (reinterpret_cast<uintptr_t>(partial) & 15) == 0)
			{
				float4 a = *reinterpret_cast<float4*>(y + i);
				for (int p = 0; p < parts; ++p)
				{
					const float4 b = *reinterpret_cast<const float4*>(partial + p * total + i);
					a.x += b.x, a.y += b.y, a.z += b.z, a.w += b.w;
				}
				*reinterpret_cast<float4*>(y + i) = a;
			}
			else
			{
				for (size_t e = i; e < total && e < i + 4; ++e)
				{
					float a = y[e];
					for (int p = 0; p < parts; ++p)
					{
						a += partial[p * total + e];
					}
					y[e] = a;
				}
			}
		}

		// tile code of the 64 x 64 tile worked by two groups of four wavefronts, each on half of K
		constexpr int kTileTwoGroups = 2414;

		// K from which splitting pays: the extra pass over y costs about 7 us
		constexpr int kSplitMinK = 8192;

		template <typename F>
		void choose_tile(GemmCall& c, int cus)
		{
			const auto blocks = [&](int mt, int bn) {
				long nb = 0;
				for (int i = 0; i < c.count; ++i)
				{
					nb += (c.n[i] + bn - 1) / bn;
				}
				return nb * ((c.m_tiles + mt - 1) / mt);
			};
			static const int forced = env_int("LITENN_HIP_GEMM_TILE", 0); // MT * 100 + NG * 10 + WAVES
			static const int split_ok = env_int("LITENN_HIP_GEMM_SPLITK", 1);
			int pick = forced;
			c.k_splits = 1;
			if (pick == 0)
			{
				// measured on the MI355X (K = 4096, N = 4096 and 14336, M = 16 .. 512): the widest tile
				// wins once it nearly fills the card, otherwise the tallest single-group tile that
				// still gives (nearly) every CU a workgroup.  A single matrix with a long K whose
				// 128 x 128 tiles fill only half the card (N = 4096 at M = 512) keeps that tile and
				// cuts K in two when the caller lends a buffer for the second product: each weight is
				// then decoded four times instead of eight, and one pass adds the two products.
				const int m_tiles = c.m_tiles;
				// the most K ranges (1, 2 or 4) that keep the workgroup count within `limit`, every range at
				// least four chunks long, and whose extra products fit the room the caller lends
				const auto ranges = [&](long tiles, long limit) {
					int r = 1;
					const size_t one = static_cast<size_t>(c.m) * c.n[0];
					while (r < 4 && tiles * (2 * r) <= limit && c.k / kChunk / (2 * r) >= 4 &&
					       c.partial_floats >= static_cast<size_t>(2 * r - 1) * one)
					{
						r *= 2;
					}
					return r;
				};
				const bool may_split = split_ok && c.partial && c.count == 1;
				const int split8 = may_split && m_tiles >= 8 ? ranges(blocks(8, 128), cus) : 1;
				const int split4 = may_split && m_tiles >= 4 ? ranges(blocks(4, 64), c.k >= kSplitMinK ? 2L * cus : cus) : 1;
				// (the wide tile, too, from 5/8 of the CUs on: 22016 x 4096 at M = 256, 172 workgroups,
				// 74.9 against 84.7 us; 12288 x 4096 at M = 512, 192: 78.9 against 86.2; 5120 x 4096 at
				// M = 1024, 160: 77.7 against 87.9; at half the CUs and below the narrower tiles win)
				// (and where the 128 x 128 tiles would need a second round of workgroups that the wide ones,
				// on at least half of the CUs, do not: 12288 x 4096 at M = 384, 144 wide workgroups against 288,
				// 72.3 against 81.8 us; 14336 x 4096 at M = 384: 73.6 against 85.5)
				const auto rounds = [&](long workgroups) { return (workgroups + cus - 1) / cus; };
				if (m_tiles >= 8 && F::kWideTile &&
				    (8 * blocks(8, 256) >= 5 * cus ||
				     (2 * blocks(8, 256) >= cus && 10 * rounds(blocks(8, 256)) <= 7 * rounds(blocks(8, 128)))))
				{
					pick = 828;
				}
				else if (m_tiles >= 8 && 8 * blocks(8, 128) >= 5 * cus)
				{
					// from 5/8 of the CUs on the 128-row tile beats the 64-row one, which decodes every
					// weight twice as often (gate/up 22016 x 4096 at M = 128, 172 workgroups: 45.4 against
					// 50.3 us; q/k 5120 x 4096 at M = 512, 160 workgroups: 47.4 against 53.3 us); at half
					// the CUs it loses (4096 x 4096 at M = 512, 128 workgroups: 45.9 against 38.5 us)
					pick = 818;
				}
				else if (m_tiles >= 4 && gemm_lds_bytes<F, 4, 1, 8, 2>() <= kLdsLimit && blocks(4, 64) <= cus &&
				         c.k < kSplitMinK && (c.k / kChunk) % 2 == 0 && split4 != 4)
				{
					// 64-row tiles that give a CU one workgroup at most: eight wavefronts in two groups, each on
					// half of the K range, so that every SIMD has two instruction streams (the four-wavefront tile
					// is bound by its one in-order stream per SIMD: MFMA busy 17 % of the time, 19 % in waits).
					// Measured against the tile this replaced (us, pre-pass included), K = 4096: M = 64: Q4_K
					// 14336 rows 23.1 against 27.1, Q4_0 12288 22.6 against 25.4; M = 128: Q4_K 8192 23.8 against
					// 28.1, 5120 22.0 against 26.0; M = 192: Q4_K 5120 23.8 against 33.7, 4096 22.8 against 27.4;
					// M = 256: 4096 24.7 against 28.9, Q6_K 30.3 against 34.0.  With more such tiles than CUs the
					// four-wavefront tile has two workgroups per CU anyway and wins (M = 64, 22016 rows: 33.4
					// against 37.2).  Two K ranges on top where they still leave a workgroup per CU (M = 64: Q4_K
					// 5120 18.4 against 20.1, 8192 19.9 against 20.6); four ranges on the four-wavefront tile stay
					// ahead where they fit (4096 rows at M = 64: 16.5 against 17.1), a long K keeps its ranges too
					// (Q6_K 4096 x 14336 at M = 64: 34.5 against 43.8).
					pick = kTileTwoGroups;
					const int chunks = c.k / kChunk;
					if (may_split && 2 * blocks(4, 64) <= cus && chunks % 4 == 0 && chunks >= 8 &&
					    c.partial_floats >= static_cast<size_t>(c.m) * c.n[0])
					{
						c.k_splits = 2;
					}
				}
				else if (split8 > 1 && 8 * blocks(8, 128) * split8 >= 5 * cus &&
				         (c.k >= kSplitMinK || (split8 == 2 && (m_tiles + 7) / 8 * 8 - m_tiles <= m_tiles / 8)))
				{
					// the 128-row tile on few weight rows (N = 4096): K walked in 2 or 4 ranges by as many
					// workgroups, the ranges' products added in K order by one more pass.  Measured (us, with the
					// pre-pass and that pass): 4096 x 11008 Q4_0 at M = 256 44.5 in four ranges against 58.5
					// unsplit on 64 x 64 tiles, 4096 x 14336 Q6_K 65.5 against 94.3; at M = 512 two ranges,
					// also for K = 4096 (Q6_K 4096 x 4096 43.6 against 49.1, Q4_K 38.3 against 39.5).  Four
					// ranges of a short K do not pay (4096 x 4096 at M = 256: 28.5 against 27.4).
					pick = 818;
					c.k_splits = split8;
				}
				else if (split4 > 1 && 2 * blocks(4, 64) * split4 >= cus && !(m_tiles < 8 && blocks(2, 64) >= cus))
				{
					// the 64-row tile, which decodes a weight once per 64 activation rows, on fewer workgroups
					// than CUs: K ranges bring it to one workgroup per CU (two, which fit a CU side by side,
					// for a long K).  Measured at M = 64: Q6_K 4096 x 4096 17.9 against 23.2 on 16-row tiles,
					// 4096 x 14336 33.9 against 60.0, Q4_0 4096 x 11008 25.6 against 33.1, Q4_K 4096 x 4096
					// 16.5 against 17.3; at M = 128, 4096 x 11008 33.0 against 39.0; Q6_K 1024 x 4096 at
					// M = 256 19.9 against 24.7.  Where the 32-row tile fills the card without ranges it is
					// as fast (8192 x 4096 at M = 64: 21.4 against 21.9) and stays.
					pick = 414;
					c.k_splits = split4;
				}
				else if (m_tiles >= 4 && 5 * blocks(4, 64) >= 4 * cus)
				{
					pick = 414;
				}
				else if (m_tiles >= 2 && 5 * blocks(2, 64) >= 4 * cus)
				{
					pick = 214;
				}
				else
				{
					pick = 114;
				}
			}
			c.tile = pick;
			// Few rows of activations: the launch is a stream of the weights, and the four-wavefront
			// tiles keep too few bytes in flight to fill the memory system (one chunk per wavefront).
			// More workgroups over the same tiles, each walking a part of K, put them there.
			if (forced == 0 && split_ok && c.k_splits == 1 && c.partial && c.count == 1 && (pick == 114 || pick == 214))
			{
				const long waves = blocks(pick / 100, 64) * 4;
				const size_t one = static_cast<size_t>(c.m) * c.n[0];
				const int chunks = c.k / kChunk;
				int splits = 1;
				while (splits < 4 && waves * splits < 8L * cus && chunks / (2 * splits) >= 2 &&
				       c.partial_floats >= (2 * splits - 1) * one)
				{
					splits *= 2;
				}
				c.k_splits = splits;
			}
			// (measurement only: LITENN_HIP_GEMM_KSPLITS forces the number of K ranges for a single matrix
			// when the caller's workspace holds the extra products and every range keeps two chunks)
			static const int forced_splits = env_int("LITENN_HIP_GEMM_KSPLITS", 0);
			if ((forced_splits == 2 || forced_splits == 4) && c.partial && c.count == 1 &&
			    c.k / kChunk >= 2 * forced_splits &&
			    c.partial_floats >= static_cast<size_t>(forced_splits - 1) * c.m * c.n[0])
			{
				c.k_splits = forced_splits;
			}
		}

		template <typename F>
		void launch_format(const GemmCall& c)
		{
#define LITENN_GEMM_CASE(MT_, NG_, WV_)                                                                              \
	if constexpr (gemm_lds_bytes<F, MT_, NG_, WV_>() <= kLdsLimit && (NG_ == 1 || F::kWideTile))                   \
	{                                                                                                              \
		if (pick == MT_ * 100 + NG_ * 10 + WV_)                                                                    \
		{                                                                                                          \
			launch_variant<F, MT_, NG_, WV_>(c);                                                                   \
			return;                                                                                                \
		}                                                                                                          \
	}
			const int pick = c.tile;
			LITENN_GEMM_CASE(8, 2, 8)
			LITENN_GEMM_CASE(8, 1, 8)
			if constexpr (gemm_lds_bytes<F, 4, 1, 8, 2>() <= kLdsLimit)
			{
				if (pick == kTileTwoGroups)
				{
					launch_variant<F, 4, 1, 8, 2>(c);
					return;
				}
			}
			if (pick == kTileTwoGroups)
			{
				launch_variant<F, 4, 1, 4>(c);
				return;
			}
			LITENN_GEMM_CASE(4, 1, 4)
			LITENN_GEMM_CASE(2, 1, 4)
			LITENN_GEMM_CASE(1, 1, 4)
			launch_variant<F, 1, 1, 4>(c);
#undef LITENN_GEMM_CASE
		}

		// The streaming form takes a single matrix against at most 32 activation rows when K is a whole
		// number of chunks per wavefront (2048 elements) whose fragments fit the registers and the slots
		// fit LDS.  Returns false, launching nothing, otherwise.
		template <typename F, int MT, int CPW, int kStreamWaves>
		bool launch_stream_variant(const GemmCall& c, int cus)
		{
			constexpr size_t slots = static_cast<size_t>(kStreamWaves) * kStreamTilesInFlight * stream_slot_bytes<F, CPW>();
			constexpr size_t per_round_tile = static_cast<size_t>(kStreamWaves) * MT * 1024;
			if constexpr (slots + per_round_tile > kLdsLimit)
			{
				return false;
			}
			else
			{
				GemmStreamArgs a{};
				a.w = c.w[0];
				a.y = c.y[0];
				a.xf = c.xf;
				a.unscale = c.unscale;
				a.residual = c.residual;
				a.n = c.n[0];
				a.k = c.k;
				a.m = c.m;
				a.m_tiles = c.m_tiles;
				a.row_bytes = c.row_bytes;
				int rows = (c.n[0] + cus - 1) / cus;
				rows = (rows + 3) / 4 * 4;
				a.rows_per_block = rows;
				const int blocks = (c.n[0] + rows - 1) / rows;
				const int tiles = (rows + 15) / 16;
				int round = static_cast<int>((kLdsLimit - slots) / per_round_tile);
				round = std::max(1, std::min(std::min(round, tiles), 8));
				a.round_tiles = round;
				const size_t lds = slots + round * per_round_tile;
				allow_dynamic_lds(reinterpret_cast<const void*>(&gemm_stream_kernel<F, MT, CPW, kStreamWaves>), kLdsLimit);
				t_last_gemm_launch = { "gemm_stream_kernel", MT, CPW, kStreamWaves, 0, static_cast<unsigned>(blocks), 1u, 1u,
					                   64u * kStreamWaves, lds };
				gemm_stream_kernel<F, MT, CPW, kStreamWaves><<<dim3(blocks), dim3(64 * kStreamWaves), lds, c.stream>>>(a);
				return true;
			}
		}

		template <typename F>
		bool launch_stream_form(const GemmCall& c, int cus)
		{
			static const int use_stream = env_int("LITENN_HIP_GEMM_STREAM", 1);
			if (!use_stream || c.count != 1 || c.m_tiles > 2 || c.k % (kChunk * 8) != 0)
			{
				return false;
			}
			// Sixteen wavefronts (K cut sixteen ways) where a workgroup's run holds two tiles and more:
			// with four wavefronts per SIMD more of the fragment decode hides behind the row stream
			// (Q4_K 14336 x 4096: 15.2 us against 16.7 with eight).  A run of a single tile is faster
			// with eight (Q6_K 4096 x 4096: 11.1 us against 11.8).
			const int rows = ((c.n[0] + cus - 1) / cus + 3) / 4 * 4;
			if (c.m_tiles == 1)
			{
				// (only where the sixteen-wavefront instance keeps its registers: one chunk per wavefront,
				// one activation tile, and not the formats whose decoders need the most of them)
				constexpr bool wide_fits = !std::is_same<F, Q3_KFrag>::value && !std::is_same<F, Q6_KFrag>::value &&
				                           !std::is_same<F, Q8_0Frag>::value;
				if constexpr (wide_fits)
				{
					if (rows > 16 && c.k == kChunk * 16)
					{
						return launch_stream_variant<F, 1, 1, 16>(c, cus);
					}
				}
				switch (c.k / (kChunk * 8))
				{
				case 1: return launch_stream_variant<F, 1, 1, 8>(c, cus);
				case 2: return launch_stream_variant<F, 1, 2, 8>(c, cus);
				case 4:
					if constexpr (std::is_same<F, Q3_KFrag>::value)
					{
						return false; // its decoder and 128 registers of fragments do not fit: the tiled kernel takes it
					}
					else
					{
						return launch_stream_variant<F, 1, 4, 8>(c, cus);
					}
				default: return false;
				}
			}
			switch (c.k / (kChunk * 8))
			{
			case 1: return launch_stream_variant<F, 2, 1, 8>(c, cus);
			case 2: return launch_stream_variant<F, 2, 2, 8>(c, cus);
			default: return false;
			}
		}

		template <typename F>
		void launch_prepass_and_gemm(GemmCall& c, const float* x, const float* norm_w, double eps, const float* up,
		                             uint8_t* xf, float* unscale, int m_pad, int cus)
		{
			if (c.m_tiles <= 2)
			{
				to_half_kernel<F><<<dim3(static_cast<unsigned>(m_pad)), dim3(256), 0, c.stream>>>(x, xf, unscale, c.m, c.k,
				                                                                                 norm_w, eps, up);
				if (launch_stream_form<F>(c, cus))
				{
					return;
				}
				choose_tile<F>(c, cus);
				launch_format<F>(c);
				if (c.k_splits > 1)
				{
					const size_t total = static_cast<size_t>(c.m) * c.n[0];
					add_partial_kernel<<<dim3(static_cast<unsigned>((total / 4 + 255) / 256 + 1)), dim3(256), 0, c.stream>>>(
					    c.y[0], c.partial, total, c.k_splits - 1);
				}
				return;
			}
			choose_tile<F>(c, cus);
			to_half_kernel<F><<<dim3(static_cast<unsigned>(m_pad)), dim3(256), 0, c.stream>>>(x, xf, unscale, c.m, c.k,
			                                                                                 norm_w, eps, up);
			launch_format<F>(c);
			if (c.k_splits > 1)
			{
				const size_t total = static_cast<size_t>(c.m) * c.n[0];
				add_partial_kernel<<<dim3(static_cast<unsigned>((total / 4 + 255) / 256 + 1)), dim3(256), 0, c.stream>>>(
				    c.y[0], c.partial, total, c.k_splits - 1);
			}
		}
		// gate and up projections with SwiGLU's product in the epilogue; only where the two-group tile
		// is the one the two matrices would get anyway (the format has it and it nearly fills the card)
		template <typename F>
		bool launch_gated(GemmCall& c, const float* x, const float* norm_w, double eps, uint8_t* xf, float* unscale,
		                  int m_pad, int cus)
		{
			if constexpr (!F::kWideTile || gemm_lds_bytes<F, 8, 2, 8>() > kLdsLimit)
			{
				return false;
			}
			else
			{
				choose_tile<F>(c, cus);
				if (c.tile != 828 || c.k_splits != 1)
				{
					return false;
				}
				to_half_kernel<F><<<dim3(static_cast<unsigned>(m_pad)), dim3(256), 0, c.stream>>>(x, xf, unscale, c.m, c.k,
				                                                                                 norm_w, eps, nullptr);
				constexpr size_t lds = gemm_lds_bytes<F, 8, 2, 8>();
				allow_dynamic_lds(reinterpret_cast<const void*>(&gemm_q_gated_kernel<F, 8, 8>), lds);
				GemmMats mats{};
				mats.w[0] = c.w[0];
				mats.w[1] = c.w[1];
				mats.y[0] = c.y[0];
				mats.n[0] = c.n[0];
				const dim3 grid((c.n[0] + 127) / 128, (c.m_tiles + 7) / 8, 1);
				t_last_gemm_launch = { "gemm_q_gated_kernel", 8, 8, 0, 0, grid.x, grid.y, grid.z, 512u, lds };
				gemm_q_gated_kernel<F, 8, 8><<<grid, dim3(512), lds, c.stream>>>(mats, c.xf, c.unscale, c.k, c.m, c.m_tiles,
				                                                                c.row_bytes);
				return true;
			}
		}

		template <typename F0, typename F1>
		void launch_pair(GemmCall& c, int second, const float* x, const float* norm_w, double eps, uint8_t* xf0,
		                 uint8_t* xf1, float* unscale0, float* unscale1, size_t row_bytes1, int m_pad, int cus)
		{
			choose_tile<F1>(c, cus); // (F1 has no wide tile, and without a partial buffer K is not split)
			to_half_pair_kernel<F0, F1><<<dim3(static_cast<unsigned>(m_pad), 2), dim3(256), 0, c.stream>>>(
			    x, xf0, xf1, unscale0, unscale1, c.m, c.k, norm_w, eps);
			switch (c.tile)
			{
			case 828: case 818: launch_pair_variant<F0, F1, 8, 8>(c, second, xf1, unscale1, row_bytes1); break;
			case 414: case kTileTwoGroups: launch_pair_variant<F0, F1, 4, 4>(c, second, xf1, unscale1, row_bytes1); break;
			case 214: launch_pair_variant<F0, F1, 2, 4>(c, second, xf1, unscale1, row_bytes1); break;
			default: launch_pair_variant<F0, F1, 1, 4>(c, second, xf1, unscale1, row_bytes1); break;
			}
		}

		int compute_unit_count()
		{
			static const int cus = [] {
				int dev = 0;
				hipDeviceProp_t prop;
				if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess)
				{
					return 256;
				}
				return prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
			}();
			return cus;
		}

		bool is_gemm_format(int fmt)
		{
			switch (fmt)
			{
			case LITENN_FMT_Q4_0: case LITENN_FMT_Q4_1: case LITENN_FMT_Q5_0: case LITENN_FMT_Q5_1: case LITENN_FMT_Q8_0:
			case LITENN_FMT_Q2_K: case LITENN_FMT_Q3_K: case LITENN_FMT_Q4_K: case LITENN_FMT_Q5_K: case LITENN_FMT_Q6_K:
				return true;
			default:
				return false;
			}
		}

		// alignment the tiled kernel needs of a format's rows: Q6_K (210-byte) and Q3_K (110-byte) blocks
		// are fetched from the 16-byte boundary below them; the other formats' chunks must start on one
		uintptr_t weight_alignment(int fmt)
		{
			return fmt == LITENN_FMT_Q6_K || fmt == LITENN_FMT_Q3_K ? 2 : (fmt == LITENN_FMT_Q2_K ? 4 : 16);
		}
	} // namespace

	// halves of scratch launch_gemm needs for an m-row batch of width k
	size_t gemm_scratch_halves(size_t m, size_t k)
	{
		const size_t m_pad = (m + 15) / 16 * 16;
		return m_pad * k + 2 * m_pad; // fp16 rows, then one f32 factor per row
	}

	// One activation matrix against up to three quantised matrices of one format and width:
	//   y_i[M, n_i] = X'[M, K] . deq(W_i)^T   (+ residual, single matrix only)
	// where X' = x, or RMSNorm(x) * norm_w when norm_w is given, or silu(x) * up when up is given (the
	// producers run inside the fp16 pre-pass).  Returns false, launching nothing, when the shape is
	// not one this kernel takes (the caller then composes the operators and uses the GEMV): K must be
	// a whole number of 256-element chunks and at most 16384 (a thread of the pre-pass holds its share
	// of a row in registers), and the rows 16-byte aligned (2-byte for Q6_K).
	// partial: null, or partial_floats floats the launch may use to walk K in 2 or 4 parts at once
	// (single matrix): M x n[0] per part after the first.
	bool launch_gemm_group(int fmt, int count, const void* const* wq, const size_t* n, size_t k, const float* x,
	                       size_t m, float* const* y, const float* residual, const float* norm_w, double eps,
	                       const float* up, void* scratch_halves, float* partial, size_t partial_floats,
	                       hipStream_t stream)
	{
		const size_t rb = row_bytes(fmt, k);
		if (!is_gemm_format(fmt))
		{
			return false;
		}
		if (count < 1 || count > 3 || (count > 1 && residual) || (norm_w && up))
		{
			return false;
		}
		const uintptr_t w_align = weight_alignment(fmt);
		for (int i = 0; i < count; ++i)
		{
			if (reinterpret_cast<uintptr_t>(wq[i]) % w_align != 0 || n[i] == 0 || n[i] > 0x7fffffffu)
			{
				return false;
			}
		}
		if (k % kChunk != 0 || rb == 0 || (rb % w_align) != 0 || reinterpret_cast<uintptr_t>(x) % 16 != 0 ||
		    reinterpret_cast<uintptr_t>(scratch_halves) % 16 != 0 || !scratch_halves ||
		    2 * ((m + 15) / 16 * 16) * k >= (size_t{ 1 } << 32) || // 32-bit tile offsets
		    k > static_cast<size_t>(kHeldItems) * 256 * 8 ||
		    (norm_w && reinterpret_cast<uintptr_t>(norm_w) % 16 != 0) || (up && reinterpret_cast<uintptr_t>(up) % 16 != 0))
		{
			return false;
		}
		const int cus = compute_unit_count();
		const size_t m_pad = (m + 15) / 16 * 16;
		uint8_t* xf = static_cast<uint8_t*>(scratch_halves);
		float* unscale = reinterpret_cast<float*>(xf + 2 * m_pad * k); // after the fp16 tiles
		GemmCall c{};
		c.count = count;
		for (int i = 0; i < count; ++i)
		{
			c.w[i] = static_cast<const uint8_t*>(wq[i]);
			c.y[i] = y[i];
			c.n[i] = static_cast<int>(n[i]);
		}
		c.xf = xf;
		c.unscale = unscale;
		c.residual = residual;
		c.k = static_cast<int>(k);
		c.m = static_cast<int>(m);
		c.m_tiles = static_cast<int>(m_pad / 16);
		c.row_bytes = rb;
		c.partial = partial;
		c.partial_floats = partial ? partial_floats : 0;
		c.stream = stream;
		const int mp = static_cast<int>(m_pad);
		switch (fmt)
		{
		case LITENN_FMT_Q4_0: launch_prepass_and_gemm<Q4_0Frag>(c, x, norm_w, eps, up, xf, unscale, mp, cus); break;
		case LITENN_FMT_Q4_1: launch_prepass_and_gemm<Q4_1Frag>(c, x, norm_w, eps, up, xf, unscale, mp, cus); break;
		case LITENN_FMT_Q5_0: launch_prepass_and_gemm<Q5_0Frag>(c, x, norm_w, eps, up, xf, unscale, mp, cus); break;
		case LITENN_FMT_Q5_1: launch_prepass_and_gemm<Q5_1Frag>(c, x, norm_w, eps, up, xf, unscale, mp, cus); break;
		case LITENN_FMT_Q2_K: launch_prepass_and_gemm<Q2_KFrag>(c, x, norm_w, eps, up, xf, unscale, mp, cus); break;
		case LITENN_FMT_Q3_K: launch_prepass_and_gemm<Q3_KFrag>(c, x, norm_w, eps, up, xf, unscale, mp, cus); break;
		case LITENN_FMT_Q8_0: launch_prepass_and_gemm<Q8_0Frag>(c, x, norm_w, eps, up, xf, unscale, mp, cus); break;
		case LITENN_FMT_Q4_K: launch_prepass_and_gemm<Q4_KFrag>(c, x, norm_w, eps, up, xf, unscale, mp, cus); break;
		case LITENN_FMT_Q5_K: launch_prepass_and_gemm<Q5_KFrag>(c, x, norm_w, eps, up, xf, unscale, mp, cus); break;
		default: launch_prepass_and_gemm<Q6_KFrag>(c, x, norm_w, eps, up, xf, unscale, mp, cus); break;
		}
		return true;
	}

	// h[M, n] = silu(X' . deq(W_gate)^T) * (X' . deq(W_up)^T) with X' = x or RMSNorm(x) * norm_w: the gate and up
	// projections of a feed-forward block with SwiGLU's product (SwiGLU.h:63-66) in the launch's
	// epilogue, so that neither projection is written out.  Takes the shapes whose two matrices would
	// run on the 128 x 256 tile; returns false, launching nothing, for anything else (the caller then
	// multiplies the two and lets the next pre-pass form the product).
	bool launch_gemm_gated(int fmt, const void* w_gate, const void* w_up, size_t n, size_t k, const float* x, size_t m,
	                       float* h, const float* norm_w, double eps, void* scratch_halves, hipStream_t stream)
	{
		const size_t rb = row_bytes(fmt, k);
		const uintptr_t w_align = weight_alignment(fmt);
		if (!is_gemm_format(fmt) || reinterpret_cast<uintptr_t>(w_gate) % w_align != 0 ||
		    reinterpret_cast<uintptr_t>(w_up) % w_align != 0 || n == 0 || n > 0x3fffffffu || k % kChunk != 0 || rb == 0 ||
		    rb % w_align != 0 || reinterpret_cast<uintptr_t>(x) % 16 != 0 || !scratch_halves ||
		    reinterpret_cast<uintptr_t>(scratch_halves) % 16 != 0 || 2 * ((m + 15) / 16 * 16) * k >= (size_t{ 1 } << 32) ||
		    k > static_cast<size_t>(kHeldItems) * 256 * 8 || (norm_w && reinterpret_cast<uintptr_t>(norm_w) % 16 != 0))
		{
			return false;
		}
		const int cus = compute_unit_count();
		const size_t m_pad = (m + 15) / 16 * 16;
		uint8_t* xf = static_cast<uint8_t*>(scratch_halves);
		float* unscale = reinterpret_cast<float*>(xf + 2 * m_pad * k);
		GemmCall c{};
		c.count = 2;
		c.w[0] = static_cast<const uint8_t*>(w_gate);
		c.w[1] = static_cast<const uint8_t*>(w_up);
		c.y[0] = h;
		c.y[1] = nullptr;
		c.n[0] = c.n[1] = static_cast<int>(n);
		c.xf = xf;
		c.unscale = unscale;
		c.k = static_cast<int>(k);
		c.m = static_cast<int>(m);
		c.m_tiles = static_cast<int>(m_pad / 16);
		c.row_bytes = rb;
		c.stream = stream;
		const int mp = static_cast<int>(m_pad);
		switch (fmt)
		{
		case LITENN_FMT_Q4_0: return launch_gated<Q4_0Frag>(c, x, norm_w, eps, xf, unscale, mp, cus);
		case LITENN_FMT_Q4_1: return launch_gated<Q4_1Frag>(c, x, norm_w, eps, xf, unscale, mp, cus);
		case LITENN_FMT_Q5_0: return launch_gated<Q5_0Frag>(c, x, norm_w, eps, xf, unscale, mp, cus);
		case LITENN_FMT_Q5_1: return launch_gated<Q5_1Frag>(c, x, norm_w, eps, xf, unscale, mp, cus);
		case LITENN_FMT_Q2_K: return launch_gated<Q2_KFrag>(c, x, norm_w, eps, xf, unscale, mp, cus);
		case LITENN_FMT_Q3_K: return launch_gated<Q3_KFrag>(c, x, norm_w, eps, xf, unscale, mp, cus);
		case LITENN_FMT_Q8_0: return launch_gated<Q8_0Frag>(c, x, norm_w, eps, xf, unscale, mp, cus);
		case LITENN_FMT_Q4_K: return launch_gated<Q4_KFrag>(c, x, norm_w, eps, xf, unscale, mp, cus);
		case LITENN_FMT_Q5_K: return launch_gated<Q5_KFrag>(c, x, norm_w, eps, xf, unscale, mp, cus);
		default: return launch_gated<Q6_KFrag>(c, x, norm_w, eps, xf, unscale, mp, cus);
		}
	}

	// Two or three matrices in two formats that share the activations (q and k in Q4_K or Q5_K beside
	// a Q6_K v): y_i[M, n_i] = X'[M, K] . deq(W_i)^T with X' = x or RMSNorm(x) * norm_w, one pre-pass
	// launch (the rows in both decoders' fragment orders) and one GEMM launch.  The formats must be a
	// run of the first followed by a run of the second.  scratch_halves holds `scratch_capacity`
	// halves and must have room for two batches (2 * gemm_scratch_halves(m, k)).  Returns false,
	// launching nothing, for anything else; the caller then goes format by format.
	bool launch_gemm_group_mixed(const int* fmts, int count, const void* const* wq, const size_t* n, size_t k,
	                             const float* x, size_t m, float* const* y, const float* norm_w, double eps,
	                             void* scratch_halves, size_t scratch_capacity, hipStream_t stream)
	{
		if (count < 2 || count > 3)
		{
			return false;
		}
		int second = 1;
		while (second < count && fmts[second] == fmts[0])
		{
			++second;
		}
		if (second == count)
		{
			return false;
		}
		for (int i = second; i < count; ++i)
		{
			if (fmts[i] != fmts[second])
			{
				return false;
			}
		}
		const int f0 = fmts[0], f1 = fmts[second];
		if ((f0 != LITENN_FMT_Q4_K && f0 != LITENN_FMT_Q5_K) || f1 != LITENN_FMT_Q6_K)
		{
			return false;
		}
		const size_t rb0 = row_bytes(f0, k), rb1 = row_bytes(f1, k);
		for (int i = 0; i < count; ++i)
		{
			const uintptr_t align = weight_alignment(i < second ? f0 : f1);
			if (reinterpret_cast<uintptr_t>(wq[i]) % align != 0 || n[i] == 0 || n[i] > 0x7fffffffu)
			{
				return false;
			}
		}
		const size_t m_pad = (m + 15) / 16 * 16;
		const size_t one = gemm_scratch_halves(m, k);
		if (k % kChunk != 0 || rb0 == 0 || rb1 == 0 || rb0 % weight_alignment(f0) != 0 || rb1 % weight_alignment(f1) != 0 ||
		    reinterpret_cast<uintptr_t>(x) % 16 != 0 || !scratch_halves ||
		    reinterpret_cast<uintptr_t>(scratch_halves) % 16 != 0 || (one & 7) != 0 || 2 * one > scratch_capacity ||
		    2 * m_pad * k >= (size_t{ 1 } << 32) || k > static_cast<size_t>(kHeldItems) * 256 * 8 ||
		    (norm_w && reinterpret_cast<uintptr_t>(norm_w) % 16 != 0))
		{
			return false;
		}
		const int cus = compute_unit_count();
		uint8_t* xf0 = static_cast<uint8_t*>(scratch_halves);
		float* unscale0 = reinterpret_cast<float*>(xf0 + 2 * m_pad * k);
		uint8_t* xf1 = xf0 + 2 * one;
		float* unscale1 = reinterpret_cast<float*>(xf1 + 2 * m_pad * k);
		GemmCall c{};
		c.count = count;
		for (int i = 0; i < count; ++i)
		{
			c.w[i] = static_cast<const uint8_t*>(wq[i]);
			c.y[i] = y[i];
			c.n[i] = static_cast<int>(n[i]);
		}
		c.xf = xf0;
		c.unscale = unscale0;
		c.residual = nullptr;
		c.k = static_cast<int>(k);
		c.m = static_cast<int>(m);
		c.m_tiles = static_cast<int>(m_pad / 16);
		c.row_bytes = rb0;
		c.partial = nullptr;
		c.partial_floats = 0;
		c.stream = stream;
		const int mp = static_cast<int>(m_pad);
		if (f0 == LITENN_FMT_Q4_K)
		{
			launch_pair<Q4_KFrag, Q6_KFrag>(c, second, x, norm_w, eps, xf0, xf1, unscale0, unscale1, rb1, mp, cus);
		}
		else
		{
			launch_pair<Q5_KFrag, Q6_KFrag>(c, second, x, norm_w, eps, xf0, xf1, unscale0, unscale1, rb1, mp, cus);
		}
		return true;
	}

	bool launch_gemm(int fmt, const void* wq, size_t n, size_t k, const float* x, size_t m, float* y,
	                 const float* residual, void* scratch_halves, float* partial, size_t partial_floats,
	                 hipStream_t stream)
	{
		const void* w[1] = { wq };
		float* ys[1] = { y };
		return launch_gemm_group(fmt, 1, w, &n, k, x, m, ys, residual, nullptr, 0.0, nullptr, scratch_halves, partial,
		                         partial_floats, stream);
	}
} // namespace litenn_hip

extern "C" int litenn_hip_gemm_last_launch(char* out, size_t capacity)
{
	using namespace litenn_hip;
	if (!out || capacity == 0)
	{
		return fail("describe the last matrix-core launch", "destination is null or empty");
	}
	const GemmLaunchRecord& r = t_last_gemm_launch;
	if (!r.kernel)
	{
		std::snprintf(out, capacity, "none");
		return 0;
	}
	char args[64];
	if (std::strcmp(r.kernel, "gemm_q_kernel") == 0)
	{
		std::snprintf(args, sizeof args, "%d, %d, %d, %d", r.a, r.b, r.c, r.d);
	}
	else if (std::strcmp(r.kernel, "gemm_q_gated_kernel") == 0)
	{
		std::snprintf(args, sizeof args, "%d, %d", r.a, r.b);
	}
	else if (std::strcmp(r.kernel, "gemm_q_pair_kernel") == 0)
	{
		std::snprintf(args, sizeof args, "%d, %d, %d", r.a, r.b, r.c);
	}
	else
	{
		std::snprintf(args, sizeof args, "%d, %d, %d", r.a, r.b, r.c);
	}
	std::snprintf(out, capacity, "%s<%s> grid %u x %u x %u, %u threads, %zu B LDS", r.kernel, args, r.grid_x, r.grid_y,
	              r.grid_z, r.threads, r.lds);
	return 0;
}
