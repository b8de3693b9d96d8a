// Streaming GEMV over GGUF block-quantised weights for gfx950.
//
//   y[n] = sum_k x[k] * deq(W)[n, k]        (+ residual[n])
//
// W is the raw .gguf payload: row n is K/block consecutive blocks.  The kernel is
// HBM-bound by construction: each weight byte is read exactly once with wide
// coalesced loads, and everything else stays on chip.
//
// Work decomposition
//   * a "unit" is 64 weights of one row handled by one lane: a Q4_0/Q8_0 block pair,
//     one 64-wide group of a Q4_K super-block, or a quarter of a Q6_K super-block.
//   * a wavefront owns one 4096-wide slice of K (64 lanes x 64 weights).  The lane keeps
//     its 64 activations in registers for the whole kernel, so the inner loop touches
//     neither LDS nor L2 for x: it is weight loads, nibble unpack and FMAs only.
//   * the wavefront walks down a run of consecutive rows (contiguous in memory), RU rows
//     per trip so RU independent wide loads are in flight per lane.
//   * per row the 64 lane partials are summed with DPP (no LDS); when K > 4096 the
//     slices of one row live in sibling wavefronts of the workgroup and meet in LDS.
//   * per-block constants are factored out of the inner loop:
//       sum_k (q_k - z) * s * x_k = s * (sum_k q_k x_k  -  z * sum_k x_k)
//     and sum_k x_k over each block is a per-lane constant computed once.
#include "common.hpp"

namespace litenn_hip
{
	namespace
	{
		typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
		typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

		// The payload is only guaranteed to be 2-byte aligned at block granularity
		// (18-, 34- and 210-byte blocks); global loads on gfx950 accept any byte address.
		struct __attribute__((packed, aligned(2))) U32x4A2 { u32x4 v; };
		struct __attribute__((packed, aligned(2))) U32x2A2 { u32x2 v; };
		struct __attribute__((packed, aligned(2))) U32A2 { uint32_t v; };
		struct __attribute__((packed, aligned(4))) U32x4A4 { u32x4 v; };

		__device__ __forceinline__ u32x4 ld4(const uint8_t* p) { return reinterpret_cast<const U32x4A2*>(p)->v; }
		__device__ __forceinline__ u32x2 ld2(const uint8_t* p) { return reinterpret_cast<const U32x2A2*>(p)->v; }
		__device__ __forceinline__ uint32_t ld1(const uint8_t* p) { return reinterpret_cast<const U32A2*>(p)->v; }
		__device__ __forceinline__ uint32_t ldh(const uint8_t* p) { return *reinterpret_cast<const uint16_t*>(p); }

		__device__ __forceinline__ float ub0(uint32_t v) { return static_cast<float>(v & 0xffu); }
		__device__ __forceinline__ float ub1(uint32_t v) { return static_cast<float>((v >> 8) & 0xffu); }
		__device__ __forceinline__ float ub2(uint32_t v) { return static_cast<float>((v >> 16) & 0xffu); }
		__device__ __forceinline__ float ub3(uint32_t v) { return static_cast<float>(v >> 24); }

		// acc += bytes(v)[0..3] . x[0..3]   (v_cvt_f32_ubyteN + v_fma)
		__device__ __forceinline__ float dot4u(uint32_t v, const float* x, float acc)
		{
			acc = fmaf(ub0(v), x[0], acc);
			acc = fmaf(ub1(v), x[1], acc);
			acc = fmaf(ub2(v), x[2], acc);
			acc = fmaf(ub3(v), x[3], acc);
			return acc;
		}

		__device__ __forceinline__ float sum_run(const float* x, int n)
		{
			float s = 0.0f;
#pragma unroll
			for (int i = 0; i < n; ++i)
			{
				s += x[i];
			}
			return s;
		}

		// ------------------------------------------------------------------
		// Per-format unit decoders.  Each provides
		//   kUnitsPerSlice      units in one 4096-wide slice (always 64)
		//   load_x(x, unit, xr) gather the unit's 64 activations (0 beyond K)
		//   prep(xr)            per-lane constants (block sums of x)
		//   Raw / load(row, unit)   the unit's bytes
		//   dot(raw, xr, prep)  the unit's contribution to the row
		// `unit` is the unit index within the row (K/64 units per row).
		// ------------------------------------------------------------------

		struct Q4_0Unit
		{
			static constexpr int kFmt = LITENN_FMT_Q4_0;
			struct Raw { u32x4 a, b; uint32_t c; };
			struct Prep { float s0, s1; };

			static __device__ __forceinline__ int x_offset(int unit, int i) { return unit * 64 + i; }
			static __device__ __forceinline__ Prep prep(const float* xr)
			{
				return { sum_run(xr, 32), sum_run(xr + 32, 32) };
			}
			static __device__ __forceinline__ Raw load(const uint8_t* row, int unit)
			{
				const uint8_t* p = row + static_cast<size_t>(unit) * 36; // two 18-byte blocks
				Raw r;
				r.a = ld4(p);
				r.b = ld4(p + 16);
				r.c = ld1(p + 32);
				return r;
			}
			// one block: 16 bytes, low nibbles -> elements 0..15, high nibbles -> 16..31
			static __device__ __forceinline__ float block(uint32_t q0, uint32_t q1, uint32_t q2, uint32_t q3,
			                                             const float* x)
			{
				const uint32_t q[4] = { q0, q1, q2, q3 };
				float lo = 0.0f, hi = 0.0f;
#pragma unroll
				for (int i = 0; i < 4; ++i)
				{
					lo = dot4u(q[i] & 0x0f0f0f0fu, x + 4 * i, lo);
					hi = dot4u((q[i] >> 4) & 0x0f0f0f0fu, x + 16 + 4 * i, hi);
				}
				return lo + hi;
			}
			static __device__ __forceinline__ float dot(const Raw& r, const float* xr, const Prep& pz)
			{
				// block 0 occupies bytes 0..17, block 1 bytes 18..35 of the 9 dwords
				const float d0 = f16_bits_to_f32(r.a.x);
				const float d1 = f16_bits_to_f32(r.b.x >> 16);
				const float a0 = block(__builtin_amdgcn_alignbit(r.a.y, r.a.x, 16),
				                       __builtin_amdgcn_alignbit(r.a.z, r.a.y, 16),
				                       __builtin_amdgcn_alignbit(r.a.w, r.a.z, 16),
				                       __builtin_amdgcn_alignbit(r.b.x, r.a.w, 16), xr);
				const float a1 = block(r.b.y, r.b.z, r.b.w, r.c, xr + 32);
				return d0 * (a0 - 8.0f * pz.s0) + d1 * (a1 - 8.0f * pz.s1);
			}
		};

		struct Q8_0Unit
		{
			static constexpr int kFmt = LITENN_FMT_Q8_0;
			struct Raw { u32x4 a, b, c, d; uint32_t e; };
			struct Prep { float s0, s1; };

			static __device__ __forceinline__ int x_offset(int unit, int i) { return unit * 64 + i; }
			static __device__ __forceinline__ Prep prep(const float* xr)
			{
				return { sum_run(xr, 32), sum_run(xr + 32, 32) };
			}
			static __device__ __forceinline__ Raw load(const uint8_t* row, int unit)
			{
				const uint8_t* p = row + static_cast<size_t>(unit) * 68; // two 34-byte blocks
				Raw r;
				r.a = ld4(p);
				r.b = ld4(p + 16);
				r.c = ld4(p + 32);
				r.d = ld4(p + 48);
				r.e = ld1(p + 64);
				return r;
			}
			static __device__ __forceinline__ float dot(const Raw& r, const float* xr, const Prep& pz)
			{
				const uint32_t w[17] = { r.a.x, r.a.y, r.a.z, r.a.w, r.b.x, r.b.y, r.b.z, r.b.w, r.c.x,
					                     r.c.y, r.c.z, r.c.w, r.d.x, r.d.y, r.d.z, r.d.w, r.e };
				// int8 -> biased uint8 (q + 128) so the byte converters apply; the bias
				// leaves through the block sum of x.
				const float d0 = f16_bits_to_f32(w[0]);
				const float d1 = f16_bits_to_f32(w[8] >> 16);
				float a0 = 0.0f, a1 = 0.0f;
#pragma unroll
				for (int i = 0; i < 8; ++i)
				{
					const uint32_t q = __builtin_amdgcn_alignbit(w[i + 1], w[i], 16) ^ 0x80808080u;
					a0 = dot4u(q, xr + 4 * i, a0);
				}
#pragma unroll
				for (int i = 0; i < 8; ++i)
				{
					a1 = dot4u(w[9 + i] ^ 0x80808080u, xr + 32 + 4 * i, a1);
				}
				return d0 * (a0 - 128.0f * pz.s0) + d1 * (a1 - 128.0f * pz.s1);
			}
		};

		struct Q4_KUnit
		{
			static constexpr int kFmt = LITENN_FMT_Q4_K;
			struct Raw { u32x4 h, a, b; };
			struct Prep { float s0, s1; };

			static __device__ __forceinline__ int x_offset(int unit, int i) { return unit * 64 + i; }
			static __device__ __forceinline__ Prep prep(const float* xr)
			{
				return { sum_run(xr, 32), sum_run(xr + 32, 32) };
			}
			static __device__ __forceinline__ Raw load(const uint8_t* row, int unit)
			{
				// super-block = 16-byte header {d, dmin, scales[12]} + 4 groups of 32 nibble bytes
				const uint8_t* sb = row + static_cast<size_t>(unit >> 2) * 144;
				const uint8_t* q = sb + 16 + (unit & 3) * 32;
				Raw r;
				r.h = ld4(sb);
				r.a = ld4(q);
				r.b = ld4(q + 16);
				return r;
			}
			static __device__ __forceinline__ float dot(const Raw& r, const float* xr, const Prep& pz, int unit)
			{
				const int g = unit & 3;
				const float d = f16_bits_to_f32(r.h.x);
				const float dmin = f16_bits_to_f32(r.h.x >> 16);
				// 6-bit (scale, min) of sub-blocks 2g and 2g+1, two per 16-bit lane
				const int sh = (g & 1) * 16;
				const uint32_t s_lo = (r.h.y >> sh) & 0xffffu; // scales bytes 2g', 2g'+1
				const uint32_t s_mid = (r.h.z >> sh) & 0xffffu; // bytes 4+2g', 5+2g'
				const uint32_t s_hi = (r.h.w >> sh) & 0xffffu; // bytes 8+2g', 9+2g'
				uint32_t sc, mn;
				if (g < 2)
				{
					sc = s_lo & 0x3f3fu;
					mn = s_mid & 0x3f3fu;
				}
				else
				{
					sc = (s_hi & 0x0f0fu) | ((s_lo >> 2) & 0x3030u);
					mn = ((s_hi >> 4) & 0x0f0fu) | ((s_mid >> 2) & 0x3030u);
				}
				const uint32_t q[8] = { r.a.x, r.a.y, r.a.z, r.a.w, r.b.x, r.b.y, r.b.z, r.b.w };
				float lo = 0.0f, hi = 0.0f;
#pragma unroll
				for (int i = 0; i < 8; ++i)
				{
					lo = dot4u(q[i] & 0x0f0f0f0fu, xr + 4 * i, lo);
					hi = dot4u((q[i] >> 4) & 0x0f0f0f0fu, xr + 32 + 4 * i, hi);
				}
				const float sum = ub0(sc) * lo + ub1(sc) * hi;
				const float off = ub0(mn) * pz.s0 + ub1(mn) * pz.s1;
				return d * sum - dmin * off;
			}
		};

		struct Q6_KUnit
		{
			static constexpr int kFmt = LITENN_FMT_Q6_K;
			struct Raw { u32x4 la, lb, h; u32x2 sc; uint32_t d; };
			struct Prep { float s[4]; };

			// unit = 4 * super-block + 2 * half + (l0 / 16); it covers four runs of 16
			// consecutive elements: 128*half + 32*r + l0 + [0,16), r = 0..3
			static __device__ __forceinline__ int x_offset(int unit, int i)
			{
				return (unit >> 2) * 256 + ((unit >> 1) & 1) * 128 + (i >> 4) * 32 + (unit & 1) * 16 + (i & 15);
			}
			static __device__ __forceinline__ Prep prep(const float* xr)
			{
				Prep p;
#pragma unroll
				for (int r = 0; r < 4; ++r)
				{
					p.s[r] = sum_run(xr + 16 * r, 16);
				}
				return p;
			}
			static __device__ __forceinline__ Raw load(const uint8_t* row, int unit)
			{
				// super-block = ql[128] qh[64] scales[16] d
				const uint8_t* sb = row + static_cast<size_t>(unit >> 2) * 210;
				const int half = (unit >> 1) & 1;
				const int l0 = (unit & 1) * 16;
				Raw r;
				r.la = ld4(sb + 64 * half + l0);
				r.lb = ld4(sb + 64 * half + 32 + l0);
				r.h = ld4(sb + 128 + 32 * half + l0);
				r.sc = ld2(sb + 192 + 8 * half);
				r.d = ldh(sb + 208);
				return r;
			}
			static __device__ __forceinline__ float dot(const Raw& r, const float* xr, const Prep& pz, int unit)
			{
				const uint32_t la[4] = { r.la.x, r.la.y, r.la.z, r.la.w };
				const uint32_t lb[4] = { r.lb.x, r.lb.y, r.lb.z, r.lb.w };
				const uint32_t hh[4] = { r.h.x, r.h.y, r.h.z, r.h.w };
				float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f, a3 = 0.0f;
#pragma unroll
				for (int i = 0; i < 4; ++i)
				{
					const uint32_t q1 = (la[i] & 0x0f0f0f0fu) | ((hh[i] << 4) & 0x30303030u);
					const uint32_t q2 = (lb[i] & 0x0f0f0f0fu) | ((hh[i] << 2) & 0x30303030u);
					const uint32_t q3 = ((la[i] >> 4) & 0x0f0f0f0fu) | (hh[i] & 0x30303030u);
					const uint32_t q4 = ((lb[i] >> 4) & 0x0f0f0f0fu) | ((hh[i] >> 2) & 0x30303030u);
					a0 = dot4u(q1, xr + 4 * i, a0);
					a1 = dot4u(q2, xr + 16 + 4 * i, a1);
					a2 = dot4u(q3, xr + 32 + 4 * i, a2);
					a3 = dot4u(q4, xr + 48 + 4 * i, a3);
				}
				// int8 scales of the four runs: scales[is], [is+2], [is+4], [is+6], is = l0/16
				const int is = unit & 1;
				const uint32_t s01 = r.sc.x >> (8 * is); // byte0 = sc[is], byte2 = sc[is+2]
				const uint32_t s23 = r.sc.y >> (8 * is);
				const float c0 = static_cast<float>(static_cast<int8_t>(s01 & 0xffu));
				const float c1 = static_cast<float>(static_cast<int8_t>((s01 >> 16) & 0xffu));
				const float c2 = static_cast<float>(static_cast<int8_t>(s23 & 0xffu));
				const float c3 = static_cast<float>(static_cast<int8_t>((s23 >> 16) & 0xffu));
				const float sum = c0 * (a0 - 32.0f * pz.s[0]) + c1 * (a1 - 32.0f * pz.s[1]) +
				                  c2 * (a2 - 32.0f * pz.s[2]) + c3 * (a3 - 32.0f * pz.s[3]);
				return f16_bits_to_f32(r.d) * sum;
			}
		};

		template <typename U>
		struct HasUnitArg { static constexpr bool value = false; };
		template <>
		struct HasUnitArg<Q4_KUnit> { static constexpr bool value = true; };
		template <>
		struct HasUnitArg<Q6_KUnit> { static constexpr bool value = true; };

		template <typename U>
		__device__ __forceinline__ float unit_dot(const typename U::Raw& r, const float* xr,
		                                          const typename U::Prep& p, int unit)
		{
			if constexpr (HasUnitArg<U>::value)
			{
				return U::dot(r, xr, p, unit);
			}
			else
			{
				return U::dot(r, xr, p);
			}
		}

		constexpr int kMaxSlices = 8;       // K <= 32768
		constexpr int kMaxRowsPerWave = 64; // bound of the LDS exchange buffer

		// grid.x workgroups; workgroup = slices x groups wavefronts.  Wavefront (s, g) of
		// workgroup b handles slice s of rows [ (b*groups + g) * rows_per_wave, +rows_per_wave ).
		template <typename U, int RU>
		__global__ __launch_bounds__(512) void gemv_kernel(const uint8_t* __restrict__ w,
		                                                    const float* __restrict__ x, float* __restrict__ y,
		                                                    const float* __restrict__ residual, int n, int k,
		                                                    size_t row_bytes, int slices, int groups,
		                                                    int rows_per_wave)
		{
			extern __shared__ float part[]; // [slices][groups * rows_per_wave] when slices > 1
			const int lane = threadIdx.x & 63;
			const int wave = threadIdx.x >> 6;
			const int s = wave % slices;
			const int g = wave / slices;
			const int unit = s * 64 + lane; // unit index within the row
			const int units_per_row = k >> 6;
			const bool active = unit < units_per_row;

			float xr[64];
			if (active)
			{
				// x_offset maps runs of >= 16 consecutive i to consecutive k: 128-bit loads
#pragma unroll
				for (int i = 0; i < 64; i += 4)
				{
					const float4 v = *reinterpret_cast<const float4*>(x + U::x_offset(unit, i));
					xr[i] = v.x;
					xr[i + 1] = v.y;
					xr[i + 2] = v.z;
					xr[i + 3] = v.w;
				}
			}
			else
			{
#pragma unroll
				for (int i = 0; i < 64; ++i)
				{
					xr[i] = 0.0f;
				}
			}
			const typename U::Prep pz = U::prep(xr);

			const int row0 = (blockIdx.x * groups + g) * rows_per_wave;
			const int row_end = min(row0 + rows_per_wave, n);
			const int safe_unit = active ? unit : 0; // inactive lanes load a valid address, contribute 0

			for (int r = row0; r < row_end; r += RU)
			{
				typename U::Raw raw[RU];
#pragma unroll
				for (int u = 0; u < RU; ++u)
				{
					const int rr = min(r + u, row_end - 1);
					raw[u] = U::load(w + static_cast<size_t>(rr) * row_bytes, safe_unit);
				}
#pragma unroll
				for (int u = 0; u < RU; ++u)
				{
					float p = unit_dot<U>(raw[u], xr, pz, safe_unit);
					p = active ? p : 0.0f;
					const float total = wave_sum(p);
					const int rr = r + u;
					if (rr < row_end && lane == 0)
					{
						if (slices == 1)
						{
							y[rr] = residual ? residual[rr] + total : total;
						}
						else
						{
							part[s * (groups * rows_per_wave) + g * rows_per_wave + (rr - row0)] = total;
						}
					}
				}
			}

			if (slices > 1)
			{
				__syncthreads();
				const int per_block = groups * rows_per_wave;
				for (int t = threadIdx.x; t < per_block; t += blockDim.x)
				{
					const int gg = t / rows_per_wave;
					const int rr = (blockIdx.x * groups + gg) * rows_per_wave + (t % rows_per_wave);
					if (rr < n)
					{
						float total = part[t];
						for (int ss = 1; ss < slices; ++ss)
						{
							total += part[ss * per_block + t];
						}
						y[rr] = residual ? residual[rr] + total : total;
					}
				}
			}
		}

		// ------------------------------------------------------------------
		// Shape-agnostic fallback: any K that is a whole number of blocks, any alignment,
		// plus the plain F32/F16 "formats".  One wavefront per row, one block (or 64
		// plain elements) per lane per trip, byte-granular loads.  Correct, not fast.
		// ------------------------------------------------------------------
		__device__ float generic_elem(int fmt, const uint8_t* row, int k_idx)
		{
			switch (fmt)
			{
			case LITENN_FMT_Q4_0:
			{
				const uint8_t* b = row + static_cast<size_t>(k_idx >> 5) * 18;
				const int j = k_idx & 31;
				const float d = f16_bits_to_f32(b[0] | (b[1] << 8));
				const int q = j < 16 ? (b[2 + j] & 0xF) : (b[2 + j - 16] >> 4);
				return static_cast<float>(q - 8) * d;
			}
			case LITENN_FMT_Q8_0:
			{
				const uint8_t* b = row + static_cast<size_t>(k_idx >> 5) * 34;
				const float d = f16_bits_to_f32(b[0] | (b[1] << 8));
				return static_cast<float>(static_cast<int8_t>(b[2 + (k_idx & 31)])) * d;
			}
			case LITENN_FMT_Q4_K:
			{
				const uint8_t* b = row + static_cast<size_t>(k_idx >> 8) * 144;
				const int e = k_idx & 255;
				const float d = f16_bits_to_f32(b[0] | (b[1] << 8));
				const float dmin = f16_bits_to_f32(b[2] | (b[3] << 8));
				const uint8_t* sc = b + 4;
				const int j = e >> 5; // sub-block
				int s, m;
				if (j < 4)
				{
					s = sc[j] & 63;
					m = sc[j + 4] & 63;
				}
				else
				{
					s = (sc[j + 4] & 0xF) | ((sc[j - 4] >> 6) << 4);
					m = (sc[j + 4] >> 4) | ((sc[j] >> 6) << 4);
				}
				const uint8_t byte = b[16 + (e >> 6) * 32 + (e & 31)];
				const int q = (e & 32) ? (byte >> 4) : (byte & 0xF);
				return d * static_cast<float>(s) * static_cast<float>(q) - dmin * static_cast<float>(m);
			}
			case LITENN_FMT_Q6_K:
			{
				const uint8_t* b = row + static_cast<size_t>(k_idx >> 8) * 210;
				const int e = k_idx & 255;
				const int half = e >> 7, r = (e >> 5) & 3, l = e & 31;
				const uint8_t* ql = b + 64 * half;
				const uint8_t* qh = b + 128 + 32 * half;
				const int8_t* sc = reinterpret_cast<const int8_t*>(b + 192 + 8 * half);
				const float d = f16_bits_to_f32(b[208] | (b[209] << 8));
				const uint8_t lo = ql[l + ((r & 1) ? 32 : 0)];
				const int low4 = (r & 2) ? (lo >> 4) : (lo & 0xF);
				const int high2 = (qh[l] >> (2 * r)) & 3;
				const int q = (low4 | (high2 << 4)) - 32;
				return d * static_cast<float>(sc[(l >> 4) + 2 * r]) * static_cast<float>(q);
			}
			case LITENN_FMT_F16:
				return f16_bits_to_f32(row[2 * k_idx] | (row[2 * k_idx + 1] << 8));
			case LITENN_FMT_F32:
			{
				uint32_t v = row[4 * k_idx] | (row[4 * k_idx + 1] << 8) | (row[4 * k_idx + 2] << 16) |
				             (static_cast<uint32_t>(row[4 * k_idx + 3]) << 24);
				return __uint_as_float(v);
			}
			default:
				return 0.0f;
			}
		}

		__global__ __launch_bounds__(256) void gemv_generic_kernel(int fmt, const uint8_t* __restrict__ w,
		                                                            const float* __restrict__ x,
		                                                            float* __restrict__ y,
		                                                            const float* __restrict__ residual, int n, int k,
		                                                            size_t row_bytes)
		{
			const int lane = threadIdx.x & 63;
			const int row = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
			if (row >= n)
			{
				return;
			}
			const uint8_t* rp = w + static_cast<size_t>(row) * row_bytes;
			float acc = 0.0f;
			for (int i = lane; i < k; i += 64)
			{
				acc = fmaf(generic_elem(fmt, rp, i), x[i], acc);
			}
			const float total = wave_sum(acc);
			if (lane == 0)
			{
				y[row] = residual ? residual[row] + total : total;
			}
		}

		__global__ void dequantize_kernel(int fmt, const uint8_t* __restrict__ w, float* __restrict__ dst, size_t rows,
		                                  int k, size_t row_bytes)
		{
			const size_t row = blockIdx.x;
			if (row >= rows)
			{
				return;
			}
			const uint8_t* rp = w + row * row_bytes;
			for (int i = threadIdx.x; i < k; i += blockDim.x)
			{
				dst[row * k + i] = generic_elem(fmt, rp, i);
			}
		}

		__global__ void get_rows_q_kernel(int fmt, const uint8_t* __restrict__ table, int rows, int k, size_t row_bytes,
		                                  const int32_t* __restrict__ ids, float* __restrict__ out, int* err_flag)
		{
			const int id = ids[blockIdx.x];
			if (id < 0 || id >= rows)
			{
				if (threadIdx.x == 0 && err_flag)
				{
					*err_flag = 1;
				}
				return;
			}
			const uint8_t* rp = table + static_cast<size_t>(id) * row_bytes;
			for (int i = threadIdx.x; i < k; i += blockDim.x)
			{
				out[static_cast<size_t>(blockIdx.x) * k + i] = generic_elem(fmt, rp, i);
			}
		}

		int env_int(const char* name, int fallback)
		{
			const char* v = getenv(name);
			return (v && *v) ? atoi(v) : fallback;
		}

		template <typename U>
		void launch_fast(const uint8_t* w, const float* x, float* y, const float* residual, int n, int k, size_t rb,
		                 hipStream_t stream)
		{
			const int slices = (k + 4095) / 4096;
			// LITENN_HIP_GEMV_WAVES: target number of resident wavefronts for the launch
			static const int target_waves = env_int("LITENN_HIP_GEMV_WAVES", 4096);
			int groups = 8 / slices;
			if (groups < 1)
			{
				groups = 1;
			}
			int rows_per_wave = (n * slices + target_waves - 1) / target_waves;
			rows_per_wave = rows_per_wave < 1 ? 1 : (rows_per_wave > kMaxRowsPerWave ? kMaxRowsPerWave : rows_per_wave);
			const int rows_per_block = groups * rows_per_wave;
			const int blocks = (n + rows_per_block - 1) / rows_per_block;
			const size_t lds = slices > 1 ? sizeof(float) * slices * rows_per_block : 0;
			gemv_kernel<U, 4><<<dim3(blocks), dim3(64 * slices * groups), lds, stream>>>(w, x, y, residual, n, k, rb,
			                                                                           slices, groups, rows_per_wave);
		}
	} // namespace

	// Launches y[m, n] = x[m, k] . W^T one activation row at a time through the GEMV.
	int launch_gemv(int fmt, const void* wq, size_t n, size_t k, const float* x, size_t m, float* y,
	                const float* residual, hipStream_t stream)
	{
		const size_t rb = row_bytes(fmt, k);
		const uint8_t* w = static_cast<const uint8_t*>(wq);
		const bool quant = fmt == LITENN_FMT_Q4_0 || fmt == LITENN_FMT_Q8_0 || fmt == LITENN_FMT_Q4_K ||
		                   fmt == LITENN_FMT_Q6_K;
		// fast path: whole 64-weight units, 16-byte aligned activations, K within the slice budget
		const bool fast = quant && (k % 256 == 0) && k <= static_cast<size_t>(kMaxSlices) * 4096 &&
		                  (reinterpret_cast<uintptr_t>(x) % 16 == 0) && (reinterpret_cast<uintptr_t>(w) % 4 == 0) &&
		                  env_int("LITENN_HIP_GEMV_GENERIC", 0) == 0;
		for (size_t i = 0; i < m; ++i)
		{
			const float* xi = x + i * k;
			float* yi = y + i * n;
			const float* ri = residual ? residual + i * n : nullptr;
			if (fast && (reinterpret_cast<uintptr_t>(xi) % 16 == 0))
			{
				switch (fmt)
				{
				case LITENN_FMT_Q4_0:
					launch_fast<Q4_0Unit>(w, xi, yi, ri, static_cast<int>(n), static_cast<int>(k), rb, stream);
					break;
				case LITENN_FMT_Q8_0:
					launch_fast<Q8_0Unit>(w, xi, yi, ri, static_cast<int>(n), static_cast<int>(k), rb, stream);
					break;
				case LITENN_FMT_Q4_K:
					launch_fast<Q4_KUnit>(w, xi, yi, ri, static_cast<int>(n), static_cast<int>(k), rb, stream);
					break;
				default:
					launch_fast<Q6_KUnit>(w, xi, yi, ri, static_cast<int>(n), static_cast<int>(k), rb, stream);
					break;
				}
			}
			else
			{
				const int waves = 4;
				gemv_generic_kernel<<<dim3((n + waves - 1) / waves), dim3(64 * waves), 0, stream>>>(
				    fmt, w, xi, yi, ri, static_cast<int>(n), static_cast<int>(k), rb);
			}
		}
		return 0;
	}

	void launch_dequantize(int fmt, const void* wq, size_t rows, size_t k, float* dst, hipStream_t stream)
	{
		dequantize_kernel<<<dim3(rows), dim3(256), 0, stream>>>(fmt, static_cast<const uint8_t*>(wq), dst, rows,
		                                                         static_cast<int>(k), row_bytes(fmt, k));
	}

	void launch_get_rows_q(int fmt, const void* table, size_t rows, size_t k, const int32_t* ids, size_t n_ids,
	                       float* out, int* err_flag, hipStream_t stream)
	{
		get_rows_q_kernel<<<dim3(n_ids), dim3(256), 0, stream>>>(fmt, static_cast<const uint8_t*>(table),
		                                                          static_cast<int>(rows), static_cast<int>(k),
		                                                          row_bytes(fmt, k), ids, out, err_flag);
	}
} // namespace litenn_hip
