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

#include <cstdlib>

namespace litenn_hip
{
	namespace
	{
		typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
		typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

		// The payload is only guaranteed to be 2-byte aligned at block granularity (18-, 34- and
		// 210-byte blocks); global loads on gfx950 accept any byte address.  Weights are read exactly
		// once, so the loads carry the non-temporal hint and do not displace x or the KV cache in L2.
		typedef u32x4 u32x4_a2 __attribute__((aligned(2)));
		typedef u32x2 u32x2_a2 __attribute__((aligned(2)));
		typedef uint32_t u32_a2 __attribute__((aligned(2)));

		__device__ __forceinline__ u32x4 ld4(const uint8_t* p)
		{
			return __builtin_nontemporal_load(reinterpret_cast<const u32x4_a2*>(p));
		}
		__device__ __forceinline__ u32x2 ld2(const uint8_t* p)
		{
			return __builtin_nontemporal_load(reinterpret_cast<const u32x2_a2*>(p));
		}
		__device__ __forceinline__ uint32_t ld1(const uint8_t* p)
		{
			return __builtin_nontemporal_load(reinterpret_cast<const u32_a2*>(p));
		}
		__device__ __forceinline__ uint32_t ldh(const uint8_t* p)
		{
			return __builtin_nontemporal_load(reinterpret_cast<const uint16_t*>(p));
		}

		// ---- manually ordered LDS access --------------------------------------------------------
		// The streaming kernel fills LDS with direct global->LDS loads (global_load_lds_dwordx4)
		// and consumes it row by row while later rows are still in flight.  The compiler can only
		// order such loads against ordinary LDS reads by waiting for ALL of them, so every LDS
		// access of that kernel is issued here through inline assembly and ordered by hand with
		// s_waitcnt: vmcnt(N) for "all but the N youngest global->LDS loads have landed" (they
		// complete in issue order) and lgkmcnt(0) before a value read from LDS is used.
		typedef __attribute__((address_space(1))) const void* global_ptr_t;
		typedef __attribute__((address_space(3))) void* lds_ptr_t;

		__device__ __forceinline__ uint32_t lds_address(const void* p)
		{
			return static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
			    (__attribute__((address_space(3))) const uint8_t*)(p)));
		}
		template <int OFF>
		__device__ __forceinline__ u32x4 lds_rd128(uint32_t addr)
		{
			u32x4 v;
			asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF) : "memory");
			return v;
		}
		template <int OFF>
		__device__ __forceinline__ u32x2 lds_rd64(uint32_t addr)
		{
			u32x2 v;
			asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF) : "memory");
			return v;
		}
		template <int OFF>
		__device__ __forceinline__ uint32_t lds_rd32(uint32_t addr)
		{
			uint32_t v;
			asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF) : "memory");
			return v;
		}
		template <int OFF>
		__device__ __forceinline__ uint32_t lds_rd16(uint32_t addr)
		{
			uint32_t v;
			asm volatile("ds_read_u16 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF) : "memory");
			return v;
		}
		typedef float f32x4 __attribute__((ext_vector_type(4)));
		__device__ __forceinline__ void lds_wr128(uint32_t addr, f32x4 v)
		{
			asm volatile("ds_write_b128 %0, %1" : : "v"(addr), "v"(v) : "memory");
		}
		__device__ __forceinline__ void lds_wr32(uint32_t addr, float v)
		{
			asm volatile("ds_write_b32 %0, %1" : : "v"(addr), "v"(v) : "memory");
		}
		// the "+v" operands tie the wait to the registers it protects: no consumer can be scheduled
		// ahead of it
		__device__ __forceinline__ void lds_wait(u32x4& a) { asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a) : : "memory"); }
		__device__ __forceinline__ void lds_wait(u32x4& a, u32x4& b, u32x4& c)
		{
			asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a), "+v"(b), "+v"(c) : : "memory");
		}
		__device__ __forceinline__ void lds_wait(u32x4& a, u32x4& b, uint32_t& c)
		{
			asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a), "+v"(b), "+v"(c) : : "memory");
		}
		__device__ __forceinline__ void lds_wait(u32x4& a, u32x4& b, u32x4& c, u32x4& d, uint32_t& e)
		{
			asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d), "+v"(e) : : "memory");
		}
		__device__ __forceinline__ void lds_wait(u32x4& a, u32x4& b, u32x4& c, u32x2& d, uint32_t& e)
		{
			asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d), "+v"(e) : : "memory");
		}
		// 128-bit global load issued outside the compiler's view (it must not fold its own, coarser
		// wait for it into the schedule); the value is valid only after a vm_wait_x that covers it
		__device__ __forceinline__ f32x4 asm_global_load128(const float* base, uint32_t byte_off)
		{
			f32x4 v;
			asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(v) : "v"(byte_off), "s"(base) : "memory");
			return v;
		}
		__device__ __forceinline__ void lds_wait(float& a) { asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a) : : "memory"); }
		__device__ __forceinline__ void lds_fence() { asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory"); }
		__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" : : : "memory"); }
		template <int N>
		__device__ __forceinline__ void vm_wait() { asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory"); }

		__device__ __forceinline__ float ub0(uint32_t v) { return static_cast<float>(v & 0xffu); }
		__device__ __forceinline__ float ub1(uint32_t v) { return static_cast<float>((v >> 8) & 0xffu); }

		// Small unsigned integers are fed to the FMA as binary16 SUBNORMALS: the 16-bit pattern
		// 0x0000..0x03ff read as a half is exactly value * 2^-24, so a masked nibble or byte is a
		// ready-made operand and no integer->float conversion is issued.  v_fma_mix_f32 widens the
		// half to f32 inside the multiply-add (exactly), accumulating in f32; the 2^24 leaves
		// through the block scale.
		typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
		constexpr float kHalfSubnormalScale = 16777216.0f; // 2^24

		// acc += lo16(pair) * x0 + hi16(pair) * x1, the halves taken as subnormal binary16
		__device__ __forceinline__ float fma_pair(uint32_t pair, float x0, float x1, float acc)
		{
			const half2_t h = __builtin_bit_cast(half2_t, pair);
			acc = __builtin_fmaf(static_cast<float>(h.x), x0, acc);
			acc = __builtin_fmaf(static_cast<float>(h.y), x1, acc);
			return acc;
		}

		// acc += bytes(v)[0..3] . x[0..3] with bytes as unsigned integers (result scaled by 2^-24)
		__device__ __forceinline__ float dot4_bytes(uint32_t v, const float* x, float acc)
		{
			const uint32_t even = __builtin_amdgcn_perm(0u, v, 0x0c020c00u); // {b0, b2} as 16-bit lanes
			const uint32_t odd = __builtin_amdgcn_perm(0u, v, 0x0c030c01u);  // {b1, b3}
			acc = fma_pair(even, x[0], x[2], acc);
			acc = fma_pair(odd, x[1], x[3], acc);
			return acc;
		}

		// One dword of packed nibbles: low nibbles of bytes 0..3 pair with xl[0..3], high nibbles
		// with xh[0..3].  lo accumulates at scale 2^-24, hi at 2^-20 (the nibble sits 4 bits up).
		__device__ __forceinline__ void dot8_nibbles(uint32_t v, const float* xl, const float* xh, float& lo,
		                                              float& hi)
		{
			const uint32_t t = v >> 8;
			lo = fma_pair(v & 0x000f000fu, xl[0], xl[2], lo);
			hi = fma_pair(v & 0x00f000f0u, xh[0], xh[2], hi);
			lo = fma_pair(t & 0x000f000fu, xl[1], xl[3], lo);
			hi = fma_pair(t & 0x00f000f0u, xh[1], xh[3], hi);
		}
		constexpr float kLoNibbleScale = 16777216.0f; // 2^24
		constexpr float kHiNibbleScale = 1048576.0f;  // 2^20

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
			struct Raw { u32x4 a, b; uint32_t c; };
			struct Prep { float s0, s1; };

			static __device__ __forceinline__ int x_offset(int unit, int i) { return unit * 64 + i; }
			// (unit, index within the unit) that activation k belongs to
			static __device__ __forceinline__ int unit_of(int k) { return k >> 6; }
			static __device__ __forceinline__ int index_of(int k) { return k & 63; }
			static __device__ __forceinline__ Prep prep(const float* xr)
			{
				return { sum_run(xr, 32), sum_run(xr + 32, 32) };
			}
			static __device__ __forceinline__ Raw load(const uint8_t* row, int unit)
			{
				const uint8_t* p = row + static_cast<uint32_t>(unit) * 36u; // two 18-byte blocks
				Raw r;
				r.a = ld4(p);
				r.b = ld4(p + 16);
				r.c = ld1(p + 32);
				return r;
			}
			static constexpr int kSliceBytes = 128 * 18; // 4096 weights
			static __device__ __forceinline__ uint32_t lds_lane_offset(int u) { return static_cast<uint32_t>(u) * 36u; }
			static __device__ __forceinline__ Raw lds_load(uint32_t p)
			{
				Raw r;
				r.a = lds_rd128<0>(p);
				r.b = lds_rd128<16>(p);
				r.c = lds_rd32<32>(p);
				lds_wait(r.a, r.b, r.c);
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
					dot8_nibbles(q[i], x + 4 * i, x + 16 + 4 * i, lo, hi);
				}
				return lo * kLoNibbleScale + hi * kHiNibbleScale;
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
			struct Raw { u32x4 a, b, c, d; uint32_t e; };
			struct Prep { float s0, s1; };

			static __device__ __forceinline__ int x_offset(int unit, int i) { return unit * 64 + i; }
			// (unit, index within the unit) that activation k belongs to
			static __device__ __forceinline__ int unit_of(int k) { return k >> 6; }
			static __device__ __forceinline__ int index_of(int k) { return k & 63; }
			static __device__ __forceinline__ Prep prep(const float* xr)
			{
				return { sum_run(xr, 32), sum_run(xr + 32, 32) };
			}
			static __device__ __forceinline__ Raw load(const uint8_t* row, int unit)
			{
				const uint8_t* p = row + static_cast<uint32_t>(unit) * 68u; // two 34-byte blocks
				Raw r;
				r.a = ld4(p);
				r.b = ld4(p + 16);
				r.c = ld4(p + 32);
				r.d = ld4(p + 48);
				r.e = ld1(p + 64);
				return r;
			}
			static constexpr int kSliceBytes = 128 * 34;
			static __device__ __forceinline__ uint32_t lds_lane_offset(int u) { return static_cast<uint32_t>(u) * 68u; }
			static __device__ __forceinline__ Raw lds_load(uint32_t p)
			{
				Raw r;
				r.a = lds_rd128<0>(p);
				r.b = lds_rd128<16>(p);
				r.c = lds_rd128<32>(p);
				r.d = lds_rd128<48>(p);
				r.e = lds_rd32<64>(p);
				lds_wait(r.a, r.b, r.c, r.d, r.e);
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
					a0 = dot4_bytes(q, xr + 4 * i, a0);
				}
#pragma unroll
				for (int i = 0; i < 8; ++i)
				{
					a1 = dot4_bytes(w[9 + i] ^ 0x80808080u, xr + 32 + 4 * i, a1);
				}
				return d0 * (a0 * kHalfSubnormalScale - 128.0f * pz.s0) + d1 * (a1 * kHalfSubnormalScale - 128.0f * pz.s1);
			}
		};

		struct Q4_KUnit
		{
			struct Raw { u32x4 h, a, b; };
			struct Prep { float s0, s1; };

			static __device__ __forceinline__ int x_offset(int unit, int i) { return unit * 64 + i; }
			// (unit, index within the unit) that activation k belongs to
			static __device__ __forceinline__ int unit_of(int k) { return k >> 6; }
			static __device__ __forceinline__ int index_of(int k) { return k & 63; }
			static __device__ __forceinline__ Prep prep(const float* xr)
			{
				return { sum_run(xr, 32), sum_run(xr + 32, 32) };
			}
			static __device__ __forceinline__ Raw load(const uint8_t* row, int unit)
			{
				// super-block = 16-byte header {d, dmin, scales[12]} + 4 groups of 32 nibble bytes
				const uint8_t* sb = row + static_cast<uint32_t>(unit >> 2) * 144u;
				const uint8_t* q = sb + 16u + static_cast<uint32_t>(unit & 3) * 32u;
				Raw r;
				r.h = ld4(sb);
				r.a = ld4(q);
				r.b = ld4(q + 16);
				return r;
			}
			static constexpr int kSliceBytes = 16 * 144;
			// header at the returned offset, nibbles of the lane's group 16 + 32 g bytes further
			static __device__ __forceinline__ uint32_t lds_lane_offset(int u)
			{
				return static_cast<uint32_t>(u >> 2) * 144u + static_cast<uint32_t>(u & 3) * 32u;
			}
			static __device__ __forceinline__ Raw lds_load(uint32_t p, int u)
			{
				Raw r;
				r.h = lds_rd128<0>(p - static_cast<uint32_t>(u & 3) * 32u);
				r.a = lds_rd128<16>(p);
				r.b = lds_rd128<32>(p);
				lds_wait(r.h, r.a, r.b);
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
					dot8_nibbles(q[i], xr + 4 * i, xr + 32 + 4 * i, lo, hi);
				}
				const float sum = (ub0(sc) * kLoNibbleScale) * lo + (ub1(sc) * kHiNibbleScale) * hi;
				const float off = ub0(mn) * pz.s0 + ub1(mn) * pz.s1;
				return d * sum - dmin * off;
			}
		};

		struct Q6_KUnit
		{
			struct Raw { u32x4 la, lb, h; u32x2 sc; uint32_t d; };
			struct Prep { float s[4]; };

			// unit = 4 * super-block + 2 * half + (l0 / 16); it covers four runs of 16
			// consecutive elements: 128*half + 32*r + l0 + [0,16), r = 0..3
			static __device__ __forceinline__ int x_offset(int unit, int i)
			{
				return (unit >> 2) * 256 + ((unit >> 1) & 1) * 128 + (i >> 4) * 32 + (unit & 1) * 16 + (i & 15);
			}
			static __device__ __forceinline__ int unit_of(int k)
			{
				return (k >> 8) * 4 + ((k >> 7) & 1) * 2 + ((k >> 4) & 1);
			}
			static __device__ __forceinline__ int index_of(int k) { return ((k >> 5) & 3) * 16 + (k & 15); }
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
				const uint8_t* sb = row + static_cast<uint32_t>(unit >> 2) * 210u;
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
			static constexpr int kSliceBytes = 16 * 210;
			static __device__ __forceinline__ uint32_t lds_lane_offset(int u)
			{
				return static_cast<uint32_t>(u >> 2) * 210u;
			}
			static __device__ __forceinline__ Raw lds_load(uint32_t sb, int u)
			{
				const uint32_t half = static_cast<uint32_t>(u >> 1) & 1u;
				const uint32_t l0 = static_cast<uint32_t>(u & 1) * 16u;
				const uint32_t ql = sb + 64u * half + l0;
				Raw r;
				r.la = lds_rd128<0>(ql);
				r.lb = lds_rd128<32>(ql);
				r.h = lds_rd128<128>(sb + 32u * half + l0);
				r.sc = lds_rd64<192>(sb + 8u * half);
				r.d = lds_rd16<208>(sb);
				lds_wait(r.la, r.lb, r.h, r.sc, r.d);
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
					a0 = dot4_bytes(q1, xr + 4 * i, a0);
					a1 = dot4_bytes(q2, xr + 16 + 4 * i, a1);
					a2 = dot4_bytes(q3, xr + 32 + 4 * i, a2);
					a3 = dot4_bytes(q4, xr + 48 + 4 * i, a3);
				}
				// int8 scales of the four runs: scales[is], [is+2], [is+4], [is+6], is = l0/16
				const int is = unit & 1;
				const uint32_t s01 = r.sc.x >> (8 * is); // byte0 = sc[is], byte2 = sc[is+2]
				const uint32_t s23 = r.sc.y >> (8 * is);
				const float c0 = static_cast<float>(static_cast<int8_t>(s01 & 0xffu));
				const float c1 = static_cast<float>(static_cast<int8_t>((s01 >> 16) & 0xffu));
				const float c2 = static_cast<float>(static_cast<int8_t>(s23 & 0xffu));
				const float c3 = static_cast<float>(static_cast<int8_t>((s23 >> 16) & 0xffu));
				const float sum = c0 * (a0 * kHalfSubnormalScale - 32.0f * pz.s[0]) +
				                  c1 * (a1 * kHalfSubnormalScale - 32.0f * pz.s[1]) +
				                  c2 * (a2 * kHalfSubnormalScale - 32.0f * pz.s[2]) +
				                  c3 * (a3 * kHalfSubnormalScale - 32.0f * pz.s[3]);
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
		constexpr int kLdsUnitStride = 68;  // floats between the staged activations of consecutive units
		constexpr size_t kMaxLdsBytes = 96 * 1024;
		constexpr int kXPerThread = 8;      // float4 loads of x per thread while staging

		template <typename U, int RU>
		__device__ __forceinline__ void load_batch(typename U::Raw (&raw)[RU], const uint8_t* __restrict__ w,
		                                           size_t row_bytes, int r, int row_end, int unit)
		{
#pragma unroll
			for (int u = 0; u < RU; ++u)
			{
				const int rr = min(r + u, row_end - 1); // the tail repeats the last row; results are dropped
				raw[u] = U::load(w + static_cast<size_t>(rr) * row_bytes, unit);
			}
		}

		// grid.x workgroups; workgroup = slices x groups wavefronts.  Wavefront (s, g) of
		// workgroup b handles slice s of rows [ (b*groups + g) * rows_per_wave, +rows_per_wave ).
		// Dynamic LDS: [k/64 units of staged x when x_in_lds][slices * groups * rows_per_wave partials
		// when slices > 1].
		template <typename U, int RU>
		__global__ __launch_bounds__(512) void gemv_kernel(const uint8_t* __restrict__ w,
		                                                    const float* __restrict__ x, float* __restrict__ y,
		                                                    const float* __restrict__ residual, int n, int k,
		                                                    size_t row_bytes, int slices, int groups,
		                                                    int rows_per_wave, int x_in_lds)
		{
			extern __shared__ __attribute__((aligned(16))) float smem[];
			float* part = smem + (x_in_lds ? (k >> 6) * kLdsUnitStride : 0);
			const int lane = threadIdx.x & 63;
			// the wavefront index is uniform: keeping it in a scalar register makes every row
			// address, bound and branch below scalar work
			const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
			const int s = wave % slices;
			const int g = wave / slices;
			const int unit = s * 64 + lane; // unit index within the row
			const int units_per_row = k >> 6;
			const bool active = unit < units_per_row;
			const int row0 = (blockIdx.x * groups + g) * rows_per_wave;
			const int row_end = min(row0 + rows_per_wave, n);
			const bool has_rows = row0 < row_end;

			// 1. activations: the oldest loads in flight, so waiting for them never waits for weights
			float4 xv[kXPerThread];
			if (x_in_lds)
			{
#pragma unroll
				for (int j = 0; j < kXPerThread; ++j)
				{
					const int i = (threadIdx.x + j * blockDim.x) * 4;
					if (i < k)
					{
						xv[j] = *reinterpret_cast<const float4*>(x + i);
					}
				}
			}

			// 2. the first two weight batches go out before anything is waited for
			typename U::Raw a[RU], b[RU];
			if (active && has_rows)
			{
				load_batch<U, RU>(a, w, row_bytes, row0, row_end, unit);
				if (row0 + RU < row_end)
				{
					load_batch<U, RU>(b, w, row_bytes, row0 + RU, row_end, unit);
				}
			}

			// 3. activations are staged once per workgroup in LDS; each float4 lands in the slot of
			// the unit that will consume it.  Units are kLdsUnitStride floats apart so that the
			// per-lane 128-bit reads below (one unit per lane) fall on distinct banks.  Each lane
			// then keeps its 64 values in registers for the whole row loop.
			float xr[64];
			if (x_in_lds)
			{
#pragma unroll
				for (int j = 0; j < kXPerThread; ++j)
				{
					const int i = (threadIdx.x + j * blockDim.x) * 4;
					if (i < k)
					{
						*reinterpret_cast<float4*>(smem + U::unit_of(i) * kLdsUnitStride + U::index_of(i)) = xv[j];
					}
				}
				__syncthreads();
			}
			if (active)
			{
				// x_offset maps runs of >= 16 consecutive i to consecutive k: 128-bit accesses
				if (x_in_lds)
				{
#pragma unroll
					for (int i = 0; i < 64; i += 4)
					{
						const float4 v = *reinterpret_cast<const float4*>(smem + unit * kLdsUnitStride + i);
						xr[i] = v.x;
						xr[i + 1] = v.y;
						xr[i + 2] = v.z;
						xr[i + 3] = v.w;
					}
				}
				else
				{
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

			// lane i keeps the total of row row0 + i; everything is written once after the loop, so no
			// store or residual load sits between the weight loads in flight
			float res = 0.0f;
			auto emit = [&](int rr, float total) { res = (lane == rr - row0) ? total : res; };
			auto compute = [&](const typename U::Raw (&raw)[RU], int r) {
#pragma unroll
				for (int u = 0; u < RU; ++u)
				{
					const float p = active ? unit_dot<U>(raw[u], xr, pz, unit) : 0.0f;
					emit(r + u, wave_sum(p));
				}
			};

			// ping-pong over two register batches: while one is unpacked and accumulated, the other
			// (and the reload of the one just consumed) is in flight
			for (int r = row0; r < row_end;)
			{
				compute(a, r);
				r += RU;
				if (r >= row_end)
				{
					break;
				}
				if (active && r + RU < row_end)
				{
					load_batch<U, RU>(a, w, row_bytes, r + RU, row_end, unit);
				}
				compute(b, r);
				r += RU;
				if (active && r + RU < row_end)
				{
					load_batch<U, RU>(b, w, row_bytes, r + RU, row_end, unit);
				}
			}

			const int count = row_end - row0;
			if (slices == 1)
			{
				if (lane < count)
				{
					y[row0 + lane] = residual ? residual[row0 + lane] + res : res;
				}
				return;
			}
			if (lane < count)
			{
				part[s * (groups * rows_per_wave) + g * rows_per_wave + lane] = res;
			}
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


		// ------------------------------------------------------------------
		// Streaming kernel: rows go HBM -> LDS with direct, fully coalesced 128-bit loads.
		//
		// Each wavefront owns RB consecutive rows of one 4096-wide slice and keeps PD of them in
		// flight: consecutive lanes fetch consecutive 16-byte chunks, every cache line is consumed by
		// one instruction and nothing passes through registers.  It walks the rows in order: wait
		// until row r has landed (vmcnt), let every lane pull its unit out of LDS, unpack,
		// multiply-accumulate against the activations held in registers, reduce across the
		// wavefront, then request row r + PD.  All wavefronts advance at the same pace, so rows
		// arrive in the order they are consumed and only the last row's arithmetic is exposed after
		// the last byte has arrived.
		// LDS (dynamic): [staged activations][nwaves x RB row slots of kSliceBytes][slice partials].
		// ------------------------------------------------------------------
		template <typename U>
		__device__ __forceinline__ typename U::Raw unit_lds_load(uint32_t p, int u)
		{
			if constexpr (HasUnitArg<U>::value)
			{
				return U::lds_load(p, u);
			}
			else
			{
				return U::lds_load(p);
			}
		}

		// Row R has landed once only the loads of the rows issued after it are outstanding.  Rows are
		// issued PD ahead of the row being consumed, so that is min(PD - 1, RB - 1 - R) rows of
		// `loads_per_row` instructions each (uniform over the wavefront).
		template <int RB, int PD, int R>
		__device__ __forceinline__ void wait_row_landed(int loads_per_row)
		{
			constexpr int kYounger = (PD - 1) < (RB - 1 - R) ? (PD - 1) : (RB - 1 - R);
			switch (loads_per_row)
			{
			case 1: vm_wait<kYounger * 1>(); break;
			case 2: vm_wait<kYounger * 2>(); break;
			case 3: vm_wait<kYounger * 3>(); break;
			case 4: vm_wait<kYounger * 4>(); break;
			default: vm_wait<kYounger * 5>(); break;
			}
		}

		template <int RB, int PD, int R>
		struct RowLoop
		{
			template <typename I, typename F>
			static __device__ __forceinline__ void run(int loads_per_row, I&& issue, F&& body)
			{
				wait_row_landed<RB, PD, R>(loads_per_row);
				body(R);
				if constexpr (R + PD < RB)
				{
					issue(R + PD);
				}
				RowLoop<RB, PD, R + 1>::run(loads_per_row, issue, body);
			}
		};
		template <int RB, int PD>
		struct RowLoop<RB, PD, RB>
		{
			template <typename I, typename F>
			static __device__ __forceinline__ void run(int, I&&, F&&) {}
		};

#ifdef LITENN_GEMV_TRACE
		__device__ unsigned long long g_trace[4096 * 16];
#define GEMV_TRACE(slot)                                                                                               \
	if (lane == 0)                                                                                                     \
	{                                                                                                                  \
		g_trace[(blockIdx.x * 8 + wave) % 4096 * 16 + (slot)] = __builtin_readcyclecounter();                          \
	}
#else
#define GEMV_TRACE(slot)
#endif

		constexpr int kMaxStreamRows = 8;
		constexpr size_t kStreamLdsLimit = 160 * 1024;

		template <typename U, int RB, int PD, int XP>
		__global__ __launch_bounds__(512) void gemv_stream_kernel(const uint8_t* __restrict__ w,
		                                                           const float* __restrict__ x,
		                                                           float* __restrict__ y,
		                                                           const float* __restrict__ residual, int n, int k,
		                                                           uint32_t row_bytes, int slices, int groups)
		{
			constexpr int kLoadsPerRowMax = (U::kSliceBytes + 1023) / 1024;
			static_assert(kLoadsPerRowMax <= 5 && (PD - 1) * kLoadsPerRowMax <= 63 &&
			                  PD * kLoadsPerRowMax <= 63,
			              "vmcnt range");
			extern __shared__ __attribute__((aligned(16))) uint8_t smem_b[];
			const uint32_t lds0 = lds_address(smem_b);
			const int lane = threadIdx.x & 63;
			const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
			const int s = wave % slices;
			const int g = wave / slices;
			const int unit = s * 64 + lane;
			const int units_per_row = k >> 6;
			const bool active = unit < units_per_row;
			const int nwaves = slices * groups;
			const uint32_t x_bytes = static_cast<uint32_t>(units_per_row) * kLdsUnitStride * 4u;
			const uint32_t rows_base = x_bytes + static_cast<uint32_t>(wave) * (RB * U::kSliceBytes);
			const uint32_t part_base = x_bytes + static_cast<uint32_t>(nwaves) * (RB * U::kSliceBytes);
			const int row0 = (blockIdx.x * groups + g) * RB;
			const int count = max(0, min(RB, n - row0));
			const uint32_t slice_off = static_cast<uint32_t>(s) * U::kSliceBytes;
			const uint32_t slice_len = min(static_cast<uint32_t>(U::kSliceBytes), row_bytes - slice_off);
			const int loads_per_row = static_cast<int>((slice_len + 1023u) >> 10);

			GEMV_TRACE(0);
			// 1. activations first: the oldest loads in flight.  XP 128-bit loads per thread, clamped
			// so that every lane issues every one of them.
			f32x4 xv[XP];
#pragma unroll
			for (int j = 0; j < XP; ++j)
			{
				const int i = min(static_cast<int>(threadIdx.x + j * blockDim.x) * 4, k - 4);
				xv[j] = asm_global_load128(x, static_cast<uint32_t>(i) * 4u);
			}

			// 2. the first PD rows of the wavefront, straight into their LDS slots.  Rows past the end
			// of the matrix re-read the last row so that the number of loads in flight is the same
			// for every wavefront (the waits count them).
			auto issue_row = [&](int r) {
				const int rr = min(row0 + r, n - 1);
				const uint8_t* grow = w + static_cast<size_t>(rr) * row_bytes + slice_off;
				uint8_t* slot = smem_b + rows_base + r * U::kSliceBytes;
#pragma unroll
				for (int i = 0; i < kLoadsPerRowMax; ++i)
				{
					if (i * 1024 < static_cast<int>(slice_len)) // uniform
					{
						const uint32_t off = static_cast<uint32_t>(i) * 1024u + static_cast<uint32_t>(lane) * 16u;
						if (off < slice_len)
						{
							__builtin_amdgcn_global_load_lds((global_ptr_t)(grow + off), (lds_ptr_t)(slot + i * 1024),
							                                 16, 0, 0);
						}
					}
				}
			};
			constexpr int kFirstRows = RB < PD ? RB : PD; // rows in flight before the loop starts
#pragma unroll
			for (int r = 0; r < kFirstRows; ++r)
			{
				issue_row(r);
			}

			// 3. activations into LDS as soon as THEY have arrived (the row loads issued after them
			// stay in flight): each float4 lands in the slot of the unit that consumes it, units
			// kLdsUnitStride floats apart to keep the 128-bit reads below conflict-free
			// (the kFirstRows rows issued after the activations may stay in flight; the activation
			// registers are only ever read by the LDS writes below, after this wait)
			switch (loads_per_row)
			{
			case 1: vm_wait<kFirstRows * 1>(); break;
			case 2: vm_wait<kFirstRows * 2>(); break;
			case 3: vm_wait<kFirstRows * 3>(); break;
			case 4: vm_wait<kFirstRows * 4>(); break;
			default: vm_wait<kFirstRows * 5>(); break;
			}
#pragma unroll
			for (int j = 0; j < XP; ++j)
			{
				const int i = (threadIdx.x + j * blockDim.x) * 4;
				if (i < k)
				{
					lds_wr128(lds0 + static_cast<uint32_t>(U::unit_of(i) * kLdsUnitStride + U::index_of(i)) * 4u, xv[j]);
				}
			}
			GEMV_TRACE(1);
			lds_barrier();
			GEMV_TRACE(2);

			// 4. the lane's 64 activations move to registers for good
			float xr[64];
			if (active)
			{
				const uint32_t xb = lds0 + static_cast<uint32_t>(unit) * (kLdsUnitStride * 4u);
				u32x4 t[16];
				t[0] = lds_rd128<0>(xb);
				t[1] = lds_rd128<16>(xb);
				t[2] = lds_rd128<32>(xb);
				t[3] = lds_rd128<48>(xb);
				t[4] = lds_rd128<64>(xb);
				t[5] = lds_rd128<80>(xb);
				t[6] = lds_rd128<96>(xb);
				t[7] = lds_rd128<112>(xb);
				t[8] = lds_rd128<128>(xb);
				t[9] = lds_rd128<144>(xb);
				t[10] = lds_rd128<160>(xb);
				t[11] = lds_rd128<176>(xb);
				t[12] = lds_rd128<192>(xb);
				t[13] = lds_rd128<208>(xb);
				t[14] = lds_rd128<224>(xb);
				t[15] = lds_rd128<240>(xb);
				asm volatile("s_waitcnt lgkmcnt(0)"
				             : "+v"(t[0]), "+v"(t[1]), "+v"(t[2]), "+v"(t[3]), "+v"(t[4]), "+v"(t[5]), "+v"(t[6]),
				               "+v"(t[7]), "+v"(t[8]), "+v"(t[9]), "+v"(t[10]), "+v"(t[11]), "+v"(t[12]), "+v"(t[13]),
				               "+v"(t[14]), "+v"(t[15])
				             :
				             : "memory");
#pragma unroll
				for (int i = 0; i < 16; ++i)
				{
					xr[4 * i] = __uint_as_float(t[i].x);
					xr[4 * i + 1] = __uint_as_float(t[i].y);
					xr[4 * i + 2] = __uint_as_float(t[i].z);
					xr[4 * i + 3] = __uint_as_float(t[i].w);
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
			GEMV_TRACE(3);

			// 5. rows in arrival order; lane r keeps the total of row row0 + r
			const uint32_t lane_p = lds0 + rows_base + U::lds_lane_offset(lane);
			float res = 0.0f;
			RowLoop<RB, PD, 0>::run(loads_per_row, issue_row, [&](int r) {
				GEMV_TRACE(4 + r);
				const typename U::Raw raw = unit_lds_load<U>(lane_p + static_cast<uint32_t>(r) * U::kSliceBytes, lane);
				const float p = active ? unit_dot<U>(raw, xr, pz, unit) : 0.0f;
				const float total = wave_sum(p);
				res = (lane == r) ? total : res;
			});
			GEMV_TRACE(15);

			if (slices == 1)
			{
				if (lane < count)
				{
					y[row0 + lane] = residual ? residual[row0 + lane] + res : res;
				}
				return;
			}
			// slices of one row meet in LDS
			if (lane < RB)
			{
				lds_wr32(lds0 + part_base + static_cast<uint32_t>((s * groups + g) * RB + lane) * 4u, res);
			}
			lds_barrier();
			const int t = threadIdx.x;
			if (t < groups * RB)
			{
				const int gg = t / RB, rl = t % RB;
				const int rr = (blockIdx.x * groups + gg) * RB + rl;
				if (rr < n)
				{
					float total = 0.0f;
					for (int ss = 0; ss < slices; ++ss)
					{
						float v = __uint_as_float(
						    lds_rd32<0>(lds0 + part_base + static_cast<uint32_t>((ss * groups + gg) * RB + rl) * 4u));
						lds_wait(v);
						total += v;
					}
					y[rr] = residual ? residual[rr] + total : total;
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

		template <typename U, int RU>
		void launch_fast_ru(const uint8_t* w, const float* x, float* y, const float* residual, int n, int k, size_t rb,
		                    hipStream_t stream)
		{
			const int slices = (k + 4095) / 4096;
			// LITENN_HIP_GEMV_WAVES: wavefronts the launch is spread over (default: 8 per CU on 256 CUs)
			static const int target_waves = env_int("LITENN_HIP_GEMV_WAVES", 2048);
			int groups = 8 / slices;
			if (groups < 1)
			{
				groups = 1;
			}
			int rows_per_wave = (n * slices + target_waves - 1) / target_waves;
			rows_per_wave = rows_per_wave < 1 ? 1 : (rows_per_wave > kMaxRowsPerWave ? kMaxRowsPerWave : rows_per_wave);
			const int rows_per_block = groups * rows_per_wave;
			const int blocks = (n + rows_per_block - 1) / rows_per_block;
			const size_t part_bytes = slices > 1 ? sizeof(float) * slices * rows_per_block : 0;
			static const int lds_x = env_int("LITENN_HIP_GEMV_LDS_X", 1);
			const size_t x_bytes = sizeof(float) * (static_cast<size_t>(k) / 64) * kLdsUnitStride;
			const int x_in_lds = (lds_x && x_bytes + part_bytes <= kMaxLdsBytes &&
			                      k <= 64 * slices * groups * 4 * kXPerThread)
			                         ? 1
			                         : 0;
			const size_t lds = part_bytes + (x_in_lds ? x_bytes : 0);
			static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemv_kernel<U, RU>),
			                                                   hipFuncAttributeMaxDynamicSharedMemorySize,
			                                                   static_cast<int>(kMaxLdsBytes));
			(void)attr;
			gemv_kernel<U, RU><<<dim3(blocks), dim3(64 * slices * groups), lds, stream>>>(
			    w, x, y, residual, n, k, rb, slices, groups, rows_per_wave, x_in_lds);
		}

		template <typename U, int RB, int PD, int XP>
		void launch_stream_rb_pd_xp(const uint8_t* w, const float* x, float* y, const float* residual, int n, int k,
		                            size_t rb, int slices, int groups, size_t lds, hipStream_t stream)
		{
			static const hipError_t attr =
			    hipFuncSetAttribute(reinterpret_cast<const void*>(&gemv_stream_kernel<U, RB, PD, XP>),
			                        hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(kStreamLdsLimit));
			(void)attr;
			const int rows_per_block = groups * RB;
			const int blocks = (n + rows_per_block - 1) / rows_per_block;
			gemv_stream_kernel<U, RB, PD, XP><<<dim3(blocks), dim3(64 * slices * groups), lds, stream>>>(
			    w, x, y, residual, n, k, static_cast<uint32_t>(rb), slices, groups);
		}

		template <typename U, int RB, int PD>
		void launch_stream_rb_pd(const uint8_t* w, const float* x, float* y, const float* residual, int n, int k,
		                         size_t rb, int slices, int groups, size_t lds, hipStream_t stream)
		{
			// 128-bit activation loads per thread while staging x
			const int per_thread = (k / 4 + 64 * slices * groups - 1) / (64 * slices * groups);
			if (per_thread <= 2)
			{
				launch_stream_rb_pd_xp<U, RB, PD, 2>(w, x, y, residual, n, k, rb, slices, groups, lds, stream);
			}
			else if (per_thread <= 4)
			{
				launch_stream_rb_pd_xp<U, RB, PD, 4>(w, x, y, residual, n, k, rb, slices, groups, lds, stream);
			}
			else
			{
				launch_stream_rb_pd_xp<U, RB, PD, kXPerThread>(w, x, y, residual, n, k, rb, slices, groups, lds,
				                                               stream);
			}
		}

		template <typename U, int RB>
		void launch_stream_rb(const uint8_t* w, const float* x, float* y, const float* residual, int n, int k,
		                      size_t rb, int slices, int groups, size_t lds, hipStream_t stream)
		{
			// LITENN_HIP_GEMV_PREFETCH: rows kept in flight ahead of the row being consumed
			static const int pd = env_int("LITENN_HIP_GEMV_PREFETCH", 3);
			if (pd <= 2)
			{
				launch_stream_rb_pd<U, RB, 2>(w, x, y, residual, n, k, rb, slices, groups, lds, stream);
			}
			else
			{
				launch_stream_rb_pd<U, RB, 3>(w, x, y, residual, n, k, rb, slices, groups, lds, stream);
			}
		}

		// Returns false when the shape does not fit the streaming kernel (the register kernel runs then).
		template <typename U>
		bool launch_stream(const uint8_t* w, const float* x, float* y, const float* residual, int n, int k, size_t rb,
		                   hipStream_t stream)
		{
			const int slices = (k + 4095) / 4096;
			if (slices > 8 || rb % 16 != 0 || reinterpret_cast<uintptr_t>(w) % 16 != 0 || rb > 0xffffffffull)
			{
				return false;
			}
			const int groups = 8 / slices;
			if (k > 64 * slices * groups * 4 * kXPerThread)
			{
				return false;
			}
			// rows per wavefront: spread the matrix over about `target_waves` wavefronts, within LDS
			static const int target_waves = env_int("LITENN_HIP_GEMV_WAVES", 2048);
			static const int forced_rb = env_int("LITENN_HIP_GEMV_ROWS", 0);
			int want = forced_rb > 0 ? forced_rb : (n * slices + target_waves - 1) / target_waves;
			want = want < 1 ? 1 : (want > kMaxStreamRows ? kMaxStreamRows : want);
			const size_t x_bytes = sizeof(float) * (static_cast<size_t>(k) / 64) * kLdsUnitStride;
			auto lds_for = [&](int r) {
				return x_bytes + static_cast<size_t>(slices * groups) * r * U::kSliceBytes +
				       sizeof(float) * slices * groups * r;
			};
			while (want > 1 && lds_for(want) > kStreamLdsLimit)
			{
				--want;
			}
			if (lds_for(want) > kStreamLdsLimit)
			{
				return false;
			}
			const size_t lds = lds_for(want);
			switch (want)
			{
			case 1: launch_stream_rb<U, 1>(w, x, y, residual, n, k, rb, slices, groups, lds, stream); break;
			case 2: launch_stream_rb<U, 2>(w, x, y, residual, n, k, rb, slices, groups, lds, stream); break;
			case 3: launch_stream_rb<U, 3>(w, x, y, residual, n, k, rb, slices, groups, lds, stream); break;
			case 4: launch_stream_rb<U, 4>(w, x, y, residual, n, k, rb, slices, groups, lds, stream); break;
			case 5: launch_stream_rb<U, 5>(w, x, y, residual, n, k, rb, slices, groups, lds, stream); break;
			case 6: launch_stream_rb<U, 6>(w, x, y, residual, n, k, rb, slices, groups, lds, stream); break;
			case 7: launch_stream_rb<U, 7>(w, x, y, residual, n, k, rb, slices, groups, lds, stream); break;
			default: launch_stream_rb<U, 8>(w, x, y, residual, n, k, rb, slices, groups, lds, stream); break;
			}
			return true;
		}

		template <typename U>
		void launch_fast(const uint8_t* w, const float* x, float* y, const float* residual, int n, int k, size_t rb,
		                 hipStream_t stream)
		{
			// LITENN_HIP_GEMV_STREAM=0 keeps the rows in registers instead of LDS
			static const int use_stream = env_int("LITENN_HIP_GEMV_STREAM", 1);
			if (use_stream && launch_stream<U>(w, x, y, residual, n, k, rb, stream))
			{
				return;
			}
			static const int ru = env_int("LITENN_HIP_GEMV_RU", 1);
			if (ru >= 4)
			{
				launch_fast_ru<U, 4>(w, x, y, residual, n, k, rb, stream);
			}
			else if (ru == 1)
			{
				launch_fast_ru<U, 1>(w, x, y, residual, n, k, rb, stream);
			}
			else
			{
				launch_fast_ru<U, 2>(w, x, y, residual, n, k, rb, stream);
			}
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
