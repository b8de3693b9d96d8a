// Streaming GEMV over GGUF block-quantised weights for gfx950.
//
//   y[n] = sum_k x[k] * deq(W)[n, k]        (+ residual[n])
//
// W is the raw .gguf payload: row n is K/block consecutive blocks.  The kernels are HBM-bound by
// construction: each weight byte is read exactly once with wide coalesced loads, and everything
// else stays on chip.
//
// Work decomposition (both kernels)
//   * a "unit" is 64 weights of one row handled by one lane: a Q4_0/Q8_0 block pair, one 64-wide
//     group of a Q4_K super-block, or a quarter of a Q6_K super-block.
//   * a wavefront owns one 4096-wide slice of K (64 lanes x 64 weights).  The lane keeps its 64
//     activations in registers for the whole kernel (staged once per workgroup through LDS), so
//     the row loop is weight traffic, nibble unpack and FMAs only.
//   * the wavefront walks down a run of consecutive rows (contiguous in memory).
//   * per row the 64 lane partials are summed with DPP (no LDS); when K > 4096 the slices of one
//     row live in sibling wavefronts of the workgroup and meet in LDS.
//   * per-block constants are factored out of the inner loop:
//       sum_k (q_k - z) * s * x_k = s * (sum_k q_k x_k  -  z * sum_k x_k)
//     and sum_k x_k over each block is a per-lane constant computed once.
//   * quants enter the FMA as binary16 subnormals (value * 2^-24), so no int->float conversion
//     is issued: a mask produces the operand of v_fma_mix_f32.
#include "common.hpp"
#include "attn_math.hpp"
#include "fetch_model.hpp"

#include <type_traits>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>

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
		// Cache policy of the weight rows' loads: non-temporal (the `nt` bit).  Every weight byte is
		// read once per launch, and streamed past the caches instead of allocated in them the
		// north-star launch takes 7.74 us instead of 8.22 and the 7B-shape decode gives 724 tok/s
		// instead of 702; the sc0 / sc1 bits change nothing, alone or with nt, and a ring of two rows
		// per wavefront is still the best depth (1 / 2 / 3 / 4: 9.63 / 7.72 / 8.29 / 9.09 us).
		constexpr int kStreamOnce = 2;

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
		__device__ __forceinline__ void lds_wr64(uint32_t addr, double v)
		{
			asm volatile("ds_write_b64 %0, %1" : : "v"(addr), "v"(v) : "memory");
		}
		__device__ __forceinline__ double lds_rd_f64(uint32_t addr)
		{
			double v;
			asm volatile("ds_read_b64 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(addr) : "memory");
			return v;
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
		__device__ __forceinline__ void lds_wait(u32x4& a, u32x4& b, u32x2& c)
		{
			asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a), "+v"(b), "+v"(c) : : "memory");
		}
		__device__ __forceinline__ void lds_wait(u32x4& a, u32x4& b, u32x2& c, uint32_t& d)
		{
			asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d) : : "memory");
		}
		__device__ __forceinline__ void lds_wait(u32x4& a, u32x4& b, uint32_t& c)
		{
			asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a), "+v"(b), "+v"(c) : : "memory");
		}
		__device__ __forceinline__ void lds_wait(u32x4& a, u32x4& b, u32x4& c, u32x4& d, u32x4& e)
		{
			asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d), "+v"(e) : : "memory");
		}
		__device__ __forceinline__ void lds_wait(u32x4& a, u32x4& b, u32x4& c, u32x4& d, uint32_t& e)
		{
			asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d), "+v"(e) : : "memory");
		}
		__device__ __forceinline__ void lds_wait(u32x4& a, u32x4& b, uint32_t& c, uint32_t& d)
		{
			asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d) : : "memory");
		}
		__device__ __forceinline__ void lds_wait(u32x4& a, u32x4& b, u32x4& c, u32x4& d, u32x2& e, uint32_t& f, uint32_t& g)
		{
			asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d), "+v"(e), "+v"(f), "+v"(g) : : "memory");
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

		// sum of n (16 or 32) consecutive registers as a balanced tree (short dependency chains)
		__device__ __forceinline__ float sum_run(const float* x, int n)
		{
			float t[32];
#pragma unroll
			for (int i = 0; i < 32; ++i)
			{
				t[i] = i < n ? x[i] : 0.0f;
			}
#pragma unroll
			for (int w = 16; w >= 1; w >>= 1)
			{
#pragma unroll
				for (int i = 0; i < w; ++i)
				{
					t[i] += t[i + w];
				}
			}
			return t[0];
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

		// ---- the 32-element formats with a minimum and / or a fifth bit (units of two blocks) --------
		// one block's nibbles (as Q4_0: low nibbles are elements 0..15, high nibbles 16..31) and,
		// when qh is given, its fifth bits (bit j of the word belongs to element j):
		// returns sum((nibble + 16 bit) * x)
		template <bool FIFTH>
		__device__ __forceinline__ float block32(uint32_t q0, uint32_t q1, uint32_t q2, uint32_t q3, uint32_t qh,
		                                         const float* x)
		{
			const uint32_t q[4] = { q0, q1, q2, q3 };
			float lo = 0.0f, hi = 0.0f, fifth = 0.0f;
#pragma unroll
			for (int i = 0; i < 4; ++i)
			{
				dot8_nibbles(q[i], x + 4 * i, x + 16 + 4 * i, lo, hi);
			}
			if (FIFTH)
			{
#pragma unroll
				for (int i = 0; i < 8; ++i)
				{
					// four bits -> four 0/1 bytes: the multiplier copies the nibble to bit offsets 0, 7, 14, 21
					const uint32_t bits = (((qh >> (4 * i)) & 0xFu) * 0x00204081u) & 0x01010101u;
					fifth = dot4_bytes(bits, x + 4 * i, fifth);
				}
			}
			return lo * kLoNibbleScale + hi * kHiNibbleScale + fifth * (16.0f * kHalfSubnormalScale);
		}

		struct Q4_1Unit // block { fp16 d; fp16 m; u8 qs[16]; }: q d + m
		{
			struct Raw { u32x4 a, b; u32x2 c; };
			struct Prep { float s0, s1; };
			static __device__ __forceinline__ int x_offset(int unit, int i) { return unit * 64 + i; }
			static __device__ __forceinline__ int unit_of(int k) { return k >> 6; }
			static __device__ __forceinline__ int index_of(int k) { return k & 63; }
			static __device__ __forceinline__ Prep prep(const float* xr) { return { sum_run(xr, 32), sum_run(xr + 32, 32) }; }
			static __device__ __forceinline__ Raw load(const uint8_t* row, int unit)
			{
				const uint8_t* p = row + static_cast<uint32_t>(unit) * 40u;
				Raw r;
				r.a = ld4(p);
				r.b = ld4(p + 16);
				r.c = ld2(p + 32);
				return r;
			}
			static constexpr int kSliceBytes = 128 * 20;
			static __device__ __forceinline__ uint32_t lds_lane_offset(int u) { return static_cast<uint32_t>(u) * 40u; }
			static __device__ __forceinline__ Raw lds_load(uint32_t p)
			{
				Raw r;
				r.a = lds_rd128<0>(p);
				r.b = lds_rd128<16>(p);
				r.c = lds_rd64<32>(p);
				lds_wait(r.a, r.b, r.c);
				return r;
			}
			static __device__ __forceinline__ float dot(const Raw& r, const float* xr, const Prep& pz)
			{
				// dwords: {d0 m0} q q q q {d1 m1} q q q q
				const float d0 = f16_bits_to_f32(r.a.x), m0 = f16_bits_to_f32(r.a.x >> 16);
				const float d1 = f16_bits_to_f32(r.b.y), m1 = f16_bits_to_f32(r.b.y >> 16);
				const float a0 = block32<false>(r.a.y, r.a.z, r.a.w, r.b.x, 0u, xr);
				const float a1 = block32<false>(r.b.z, r.b.w, r.c.x, r.c.y, 0u, xr + 32);
				return d0 * a0 + m0 * pz.s0 + d1 * a1 + m1 * pz.s1;
			}
		};

		struct Q5_0Unit // block { fp16 d; u8 qh[4]; u8 qs[16]; }: ((nibble | bit << 4) - 16) d
		{
			struct Raw { u32x4 a, b; u32x2 c; uint32_t e; };
			struct Prep { float s0, s1; };
			static __device__ __forceinline__ int x_offset(int unit, int i) { return unit * 64 + i; }
			static __device__ __forceinline__ int unit_of(int k) { return k >> 6; }
			static __device__ __forceinline__ int index_of(int k) { return k & 63; }
			static __device__ __forceinline__ Prep prep(const float* xr) { return { sum_run(xr, 32), sum_run(xr + 32, 32) }; }
			static __device__ __forceinline__ Raw load(const uint8_t* row, int unit)
			{
				const uint8_t* p = row + static_cast<uint32_t>(unit) * 44u;
				Raw r;
				r.a = ld4(p);
				r.b = ld4(p + 16);
				r.c = ld2(p + 32);
				r.e = ld1(p + 40);
				return r;
			}
			static constexpr int kSliceBytes = 128 * 22;
			static __device__ __forceinline__ uint32_t lds_lane_offset(int u) { return static_cast<uint32_t>(u) * 44u; }
			static __device__ __forceinline__ Raw lds_load(uint32_t p)
			{
				Raw r;
				r.a = lds_rd128<0>(p);
				r.b = lds_rd128<16>(p);
				r.c = lds_rd64<32>(p);
				r.e = lds_rd32<40>(p);
				lds_wait(r.a, r.b, r.c, r.e);
				return r;
			}
			static __device__ __forceinline__ float dot(const Raw& r, const float* xr, const Prep& pz)
			{
				// block 0 is bytes 0..21 (d, qh at 2, qs at 6), block 1 bytes 22..43 (d at 22, qh at 24, qs at 28)
				const uint32_t w[11] = { r.a.x, r.a.y, r.a.z, r.a.w, r.b.x, r.b.y, r.b.z, r.b.w, r.c.x, r.c.y, r.e };
				const float d0 = f16_bits_to_f32(w[0]);
				const float d1 = f16_bits_to_f32(w[5] >> 16);
				const float a0 = block32<true>(__builtin_amdgcn_alignbit(w[2], w[1], 16), __builtin_amdgcn_alignbit(w[3], w[2], 16),
				                               __builtin_amdgcn_alignbit(w[4], w[3], 16), __builtin_amdgcn_alignbit(w[5], w[4], 16),
				                               __builtin_amdgcn_alignbit(w[1], w[0], 16), xr);
				const float a1 = block32<true>(w[7], w[8], w[9], w[10], w[6], xr + 32);
				return d0 * (a0 - 16.0f * pz.s0) + d1 * (a1 - 16.0f * pz.s1);
			}
		};

		struct Q5_1Unit // block { fp16 d; fp16 m; u8 qh[4]; u8 qs[16]; }: (nibble | bit << 4) d + m
		{
			struct Raw { u32x4 a, b, c; };
			struct Prep { float s0, s1; };
			static __device__ __forceinline__ int x_offset(int unit, int i) { return unit * 64 + i; }
			static __device__ __forceinline__ int unit_of(int k) { return k >> 6; }
			static __device__ __forceinline__ int index_of(int k) { return k & 63; }
			static __device__ __forceinline__ Prep prep(const float* xr) { return { sum_run(xr, 32), sum_run(xr + 32, 32) }; }
			static __device__ __forceinline__ Raw load(const uint8_t* row, int unit)
			{
				const uint8_t* p = row + static_cast<uint32_t>(unit) * 48u;
				Raw r;
				r.a = ld4(p);
				r.b = ld4(p + 16);
				r.c = ld4(p + 32);
				return r;
			}
			static constexpr int kSliceBytes = 128 * 24;
			static __device__ __forceinline__ uint32_t lds_lane_offset(int u) { return static_cast<uint32_t>(u) * 48u; }
			static __device__ __forceinline__ Raw lds_load(uint32_t p)
			{
				Raw r;
				r.a = lds_rd128<0>(p);
				r.b = lds_rd128<16>(p);
				r.c = lds_rd128<32>(p);
				lds_wait(r.a, r.b, r.c);
				return r;
			}
			static __device__ __forceinline__ float dot(const Raw& r, const float* xr, const Prep& pz)
			{
				// dwords: {d0 m0} qh q q q q {d1 m1} qh q q q q
				const float d0 = f16_bits_to_f32(r.a.x), m0 = f16_bits_to_f32(r.a.x >> 16);
				const float d1 = f16_bits_to_f32(r.b.z), m1 = f16_bits_to_f32(r.b.z >> 16);
				const float a0 = block32<true>(r.a.z, r.a.w, r.b.x, r.b.y, r.a.y, xr);
				const float a1 = block32<true>(r.c.x, r.c.y, r.c.z, r.c.w, r.b.w, xr + 32);
				return d0 * a0 + m0 * pz.s0 + d1 * a1 + m1 * pz.s1;
			}
		};

		// ---- Q2_K and Q3_K: 2-bit planes ---------------------------------------------------------------
		// Both store the low two bits of element e in plane (e % 128) / 32 of byte 32 (e / 128) + e % 32
		// of a 64-byte field, and a scale per 16 elements.  A unit is 64 consecutive elements: two
		// planes of one 32-byte half; its four 16-element groups have scale indices 4 u .. 4 u + 3.
		struct Q2_KUnit // { u8 scales[16]; u8 qs[64]; fp16 d; fp16 dmin; }: d (sc & 15) q - dmin (sc >> 4)
		{
			struct Raw { u32x4 qa, qb; uint32_t sc, dd; };
			struct Prep { float s[4]; };
			static __device__ __forceinline__ int x_offset(int unit, int i) { return unit * 64 + i; }
			static __device__ __forceinline__ int unit_of(int k) { return k >> 6; }
			static __device__ __forceinline__ int index_of(int k) { return k & 63; }
			static __device__ __forceinline__ Prep prep(const float* xr)
			{
				Prep p;
#pragma unroll
				for (int g = 0; g < 4; ++g)
				{
					p.s[g] = sum_run(xr + 16 * g, 16);
				}
				return p;
			}
			static __device__ __forceinline__ Raw load(const uint8_t* row, int unit)
			{
				const uint8_t* sb = row + static_cast<uint32_t>(unit >> 2) * 84u;
				const uint8_t* q = sb + 16u + static_cast<uint32_t>((unit >> 1) & 1) * 32u;
				Raw r;
				r.qa = ld4(q);
				r.qb = ld4(q + 16);
				r.sc = ld1(sb + 4u * static_cast<uint32_t>(unit & 3));
				r.dd = ld1(sb + 80);
				return r;
			}
			static constexpr int kSliceBytes = 16 * 84;
			static __device__ __forceinline__ uint32_t lds_lane_offset(int u) { return static_cast<uint32_t>(u >> 2) * 84u; }
			static __device__ __forceinline__ Raw lds_load(uint32_t sb, int u)
			{
				const uint32_t q = sb + static_cast<uint32_t>((u >> 1) & 1) * 32u;
				Raw r;
				r.qa = lds_rd128<16>(q);
				r.qb = lds_rd128<32>(q);
				r.sc = lds_rd32<0>(sb + 4u * static_cast<uint32_t>(u & 3));
				r.dd = lds_rd32<80>(sb);
				lds_wait(r.qa, r.qb, r.sc, r.dd);
				return r;
			}
			static __device__ __forceinline__ float dot(const Raw& r, const float* xr, const Prep& pz, int unit)
			{
				const uint32_t q[8] = { r.qa.x, r.qa.y, r.qa.z, r.qa.w, r.qb.x, r.qb.y, r.qb.z, r.qb.w };
				const int plane0 = (unit & 1) * 4; // bit offset of the unit's first plane
				const float d = f16_bits_to_f32(r.dd), dmin = f16_bits_to_f32(r.dd >> 16);
				float sum = 0.0f, off = 0.0f;
#pragma unroll
				for (int g = 0; g < 4; ++g) // group g: plane g / 2, bytes 16 (g % 2) .. + 15
				{
					float a = 0.0f;
#pragma unroll
					for (int i = 0; i < 4; ++i)
					{
						a = dot4_bytes((q[4 * (g & 1) + i] >> (plane0 + 2 * (g >> 1))) & 0x03030303u, xr + 16 * g + 4 * i, a);
					}
					const uint32_t sc = (r.sc >> (8 * g)) & 0xffu;
					sum += static_cast<float>(sc & 0xFu) * a;
					off += static_cast<float>(sc >> 4) * pz.s[g];
				}
				return d * (sum * kHalfSubnormalScale) - dmin * off;
			}
		};

		struct Q3_KUnit // { u8 hmask[32]; u8 qs[64]; u8 scales[12]; fp16 d; }: d (sc - 32) (q - (bit ? 0 : 4))
		{
			struct Raw { u32x4 ha, hb, qa, qb; u32x2 s01; uint32_t s2, d; };
			struct Prep { float s[4]; };
			static __device__ __forceinline__ int x_offset(int unit, int i) { return unit * 64 + i; }
			static __device__ __forceinline__ int unit_of(int k) { return k >> 6; }
			static __device__ __forceinline__ int index_of(int k) { return k & 63; }
			static __device__ __forceinline__ Prep prep(const float* xr)
			{
				Prep p;
#pragma unroll
				for (int g = 0; g < 4; ++g)
				{
					p.s[g] = sum_run(xr + 16 * g, 16);
				}
				return p;
			}
			static __device__ __forceinline__ Raw load(const uint8_t* row, int unit)
			{
				const uint8_t* sb = row + static_cast<uint32_t>(unit >> 2) * 110u;
				const uint8_t* q = sb + 32u + static_cast<uint32_t>((unit >> 1) & 1) * 32u;
				Raw r;
				r.ha = ld4(sb);
				r.hb = ld4(sb + 16);
				r.qa = ld4(q);
				r.qb = ld4(q + 16);
				r.s01 = ld2(sb + 96);
				r.s2 = ld1(sb + 104);
				r.d = ldh(sb + 108);
				return r;
			}
			static constexpr int kSliceBytes = 16 * 110;
			static __device__ __forceinline__ uint32_t lds_lane_offset(int u) { return static_cast<uint32_t>(u >> 2) * 110u; }
			static __device__ __forceinline__ Raw lds_load(uint32_t sb, int u)
			{
				const uint32_t q = sb + static_cast<uint32_t>((u >> 1) & 1) * 32u;
				Raw r;
				r.ha = lds_rd128<0>(sb);
				r.hb = lds_rd128<16>(sb);
				r.qa = lds_rd128<32>(q);
				r.qb = lds_rd128<48>(q);
				r.s01 = lds_rd64<96>(sb);
				r.s2 = lds_rd32<104>(sb);
				r.d = lds_rd16<108>(sb);
				lds_wait(r.ha, r.hb, r.qa, r.qb, r.s01, r.s2, r.d);
				return r;
			}
			static __device__ __forceinline__ float dot(const Raw& r, const float* xr, const Prep& pz, int unit)
			{
				const uint32_t q[8] = { r.qa.x, r.qa.y, r.qa.z, r.qa.w, r.qb.x, r.qb.y, r.qb.z, r.qb.w };
				const uint32_t hm[8] = { r.ha.x, r.ha.y, r.ha.z, r.ha.w, r.hb.x, r.hb.y, r.hb.z, r.hb.w };
				const int u = unit & 3;
				const int plane0 = (u & 1) * 4; // bit offset of the unit's first plane in the quant bytes
				const int hbit0 = 2 * u;        // ... and of its first high-bit plane in the mask bytes
				// the unit's four six-bit scales 4 u .. 4 u + 3: low four bits are the low (u < 2) or high
				// nibbles of scale bytes 4 (u & 1) .. + 3, the top two bits 2 u, 2 u + 1 of bytes 8 .. 11
				const uint32_t low_word = (u & 1) ? r.s01.y : r.s01.x;
				const uint32_t low4 = (low_word >> (4 * (u >> 1))) & 0x0f0f0f0fu;
				const uint32_t top2 = ((r.s2 >> (2 * u)) & 0x03030303u) << 4;
				const uint32_t scales = low4 | top2;
				float sum = 0.0f;
#pragma unroll
				for (int g = 0; g < 4; ++g) // group g: plane g / 2, bytes 16 (g % 2) .. + 15
				{
					float a = 0.0f;
#pragma unroll
					for (int i = 0; i < 4; ++i)
					{
						const int w = 4 * (g & 1) + i;
						const uint32_t two = (q[w] >> (plane0 + 2 * (g >> 1))) & 0x03030303u;
						const uint32_t high = (hm[w] >> (hbit0 + (g >> 1))) & 0x01010101u;
						a = dot4_bytes(two | (high << 2), xr + 16 * g + 4 * i, a); // q + 4 bit
					}
					const float sc = static_cast<float>(static_cast<int>((scales >> (8 * g)) & 0xffu) - 32);
					sum += sc * (a * kHalfSubnormalScale - 4.0f * pz.s[g]);
				}
				return f16_bits_to_f32(r.d) * sum;
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

		// Q5_K: Q4_K's nibbles plus a fifth bit per element.  Super-block = {fp16 d, fp16 dmin,
		// scales[12] (packed as in Q4_K), qh[32], qs[128]}: sub-block s takes the low (s even) or
		// high (s odd) nibbles of bytes 32 (s / 2) + l and bit s of qh[l]; value =
		// d sc (nibble + 16 bit) - dmin m.  A unit is the 64 elements of sub-blocks 2g, 2g+1.
		struct Q5_KUnit
		{
			struct Raw { u32x4 h, a, b, ha, hb; };
			struct Prep { float s0, s1; };

			static __device__ __forceinline__ int x_offset(int unit, int i) { return unit * 64 + i; }
			static __device__ __forceinline__ int unit_of(int k) { return k >> 6; }
			static __device__ __forceinline__ int index_of(int k) { return k & 63; }
			static __device__ __forceinline__ Prep prep(const float* xr)
			{
				return { sum_run(xr, 32), sum_run(xr + 32, 32) };
			}
			static __device__ __forceinline__ Raw load(const uint8_t* row, int unit)
			{
				const uint8_t* sb = row + static_cast<uint32_t>(unit >> 2) * 176u;
				const uint8_t* q = sb + 48u + static_cast<uint32_t>(unit & 3) * 32u;
				Raw r;
				r.h = ld4(sb);
				r.ha = ld4(sb + 16);
				r.hb = ld4(sb + 32);
				r.a = ld4(q);
				r.b = ld4(q + 16);
				return r;
			}
			static constexpr int kSliceBytes = 16 * 176;
			// the super-block at the returned offset; the nibbles of the lane's group 48 + 32 g further
			static __device__ __forceinline__ uint32_t lds_lane_offset(int u)
			{
				return static_cast<uint32_t>(u >> 2) * 176u;
			}
			static __device__ __forceinline__ Raw lds_load(uint32_t sb, int u)
			{
				const uint32_t q = sb + static_cast<uint32_t>(u & 3) * 32u;
				Raw r;
				r.h = lds_rd128<0>(sb);
				r.ha = lds_rd128<16>(sb);
				r.hb = lds_rd128<32>(sb);
				r.a = lds_rd128<48>(q);
				r.b = lds_rd128<64>(q);
				lds_wait(r.h, r.ha, r.hb, r.a, r.b);
				return r;
			}
			static __device__ __forceinline__ float dot(const Raw& r, const float* xr, const Prep& pz, int unit)
			{
				const int g = unit & 3;
				const float d = f16_bits_to_f32(r.h.x);
				const float dmin = f16_bits_to_f32(r.h.x >> 16);
				const int sh = (g & 1) * 16;
				const uint32_t s_lo = (r.h.y >> sh) & 0xffffu;
				const uint32_t s_mid = (r.h.z >> sh) & 0xffffu;
				const uint32_t s_hi = (r.h.w >> sh) & 0xffffu;
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
				const uint32_t qh[8] = { r.ha.x, r.ha.y, r.ha.z, r.ha.w, r.hb.x, r.hb.y, r.hb.z, r.hb.w };
				float lo = 0.0f, hi = 0.0f;   // nibble sums at 2^-24 / 2^-20
				float lo5 = 0.0f, hi5 = 0.0f; // fifth-bit sums at 2^-24
#pragma unroll
				for (int i = 0; i < 8; ++i)
				{
					dot8_nibbles(q[i], xr + 4 * i, xr + 32 + 4 * i, lo, hi);
					const uint32_t bits = qh[i] >> (2 * g);
					lo5 = dot4_bytes(bits & 0x01010101u, xr + 4 * i, lo5);
					hi5 = dot4_bytes((bits >> 1) & 0x01010101u, xr + 32 + 4 * i, hi5);
				}
				const float q0 = lo * kLoNibbleScale + lo5 * (16.0f * kHalfSubnormalScale);
				const float q1 = hi * kHiNibbleScale + hi5 * (16.0f * kHalfSubnormalScale);
				const float sum = ub0(sc) * q0 + ub1(sc) * q1;
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
		struct HasUnitArg<Q5_KUnit> { static constexpr bool value = true; };
		template <>
		struct HasUnitArg<Q2_KUnit> { static constexpr bool value = true; };
		template <>
		struct HasUnitArg<Q3_KUnit> { static constexpr bool value = true; };
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

		constexpr int kMaxSlices = 8;       // K <= 32768
		constexpr int kTwelveXp = 4;        // activation loads per thread of the twelve-wavefront instance
		constexpr int kMaxRowsPerWave = 64; // rows a wavefront of the register kernel may own
		constexpr int kLdsUnitStride = 68;  // floats between the staged activations of consecutive units
		constexpr int kXPerThread = 8;      // most 128-bit activation loads a thread issues while staging
		constexpr int kMaxStreamRows = 64;  // most rows a wavefront of the streaming kernel owns (one per lane)
		// Rows a wavefront keeps in flight (= its LDS row slots).  Two rows of eight wavefronts on
		// each of 256 CUs are about 9 MB, the card's bandwidth x latency product; deeper rings were
		// measured slower, each extra slot by 5 - 8 % on a 33 MB launch.
		constexpr int kPrefetchRows = 2;
		constexpr size_t kStreamLdsLimit = 160 * 1024;

#ifdef LITENN_GEMV_TRACE
		// Timeline build (lib/liblitenn_hip_trace.so only): lane 0 of every wavefront stamps the
		// card's constant 100 MHz clock, which all compute units share, at fixed points of the
		// streaming kernel.  Slots: 0 entry, 1 activations written to LDS, 2 barrier passed,
		// 3 activations in registers, 4 + r row r landed (r < 11), 15 last row consumed.
		constexpr int kTraceWaves = 4096, kTraceSlots = 16;
		__device__ unsigned long long g_trace[kTraceWaves * kTraceSlots];
		__device__ int g_trace_skip_arithmetic = 0; // 1: rows are fetched and read from LDS, not multiplied
#define GEMV_TRACE(slot)                                                                                               \
	if (lane == 0)                                                                                                     \
	{                                                                                                                  \
		g_trace[(blockIdx.x * 8 + wave) % kTraceWaves * kTraceSlots + (slot)] = __builtin_amdgcn_s_memrealtime();      \
	}
		// the decoder-block kernel's own points (attn_block.inc): 0 entry, 1 first phase's rows stored,
		// 2 first meeting passed, 3 second phase's triple stored, 4 second meeting passed, 5 activations
		// of the third phase in registers, 6 end
		constexpr int kBlockTraceSlots = 8;
		__device__ unsigned long long g_block_trace[kTraceWaves * kBlockTraceSlots];
#define BLOCK_TRACE(slot)                                                                                              \
	if (lane == 0)                                                                                                     \
	{                                                                                                                  \
		g_block_trace[(blockIdx.x * 8 + wave) % kTraceWaves * kBlockTraceSlots + (slot)] =                             \
		    __builtin_amdgcn_s_memrealtime();                                                                          \
	}
#else
#define GEMV_TRACE(slot)
#define BLOCK_TRACE(slot)
#endif

		// ------------------------------------------------------------------
		// Streaming kernel: rows go HBM -> LDS with direct, fully coalesced 128-bit loads.
		//
		// Each wavefront owns a run of consecutive rows of one 4096-wide slice and keeps
		// kPrefetchRows of them in flight, each in its own LDS slot: consecutive lanes fetch
		// consecutive 16-byte chunks, every cache line is consumed by one instruction and nothing
		// passes through registers.  It walks the rows in order: wait until row r has landed
		// (vmcnt), let every lane pull its unit out of LDS, unpack, multiply-accumulate against the
		// activations held in registers, reduce across the wavefront, then request row
		// r + kPrefetchRows into the slot just emptied.  The run length is a launch parameter, so a
		// launch is always one round of workgroups (at most one per CU) however many rows there
		// are: the start-up (activations to LDS to registers) is paid once per CU.
		//
		// One launch can serve the operator groups of the decoder block that share an input:
		//   * up to three matrices of one format over the same x (q/k/v projections): their rows
		//     are simply concatenated;
		//   * RMSNorm folded into the activation staging (x is normalised in f64 and scaled by the
		//     norm weight while it moves to LDS; every workgroup recomputes the 4096-element sum,
		//     which costs no HBM traffic and removes a kernel launch);
		//   * SwiGLU: gate and up rows interleaved, the epilogue writes silu(gate) * up;
		//   * a residual added to the output.
		//
		// LDS (dynamic): [staged activations][nwaves x kPrefetchRows row slots of kSliceBytes][slice partials]
		// [norm partial sums].
		// ------------------------------------------------------------------
		struct GemvArgs
		{
			const uint8_t* w[3];
			float* y[3];
			int n[3];              // rows of each matrix, 0 when unused
			const float* x;
			const float* residual; // added to y[0]; single-matrix launches only
			const float* norm_w;   // non-null: x is RMS-normalised and scaled by norm_w while staged
			double eps;
			int n_total;           // rows walked: n0 + n1 + n2, or 2 * n0 when interleaved
			int k;
			uint32_t row_bytes;
			int slices, groups;
			int rows_per_group;    // consecutive rows a wavefront group of the first half walks (<= 64)
			int run_diff;          // the groups of the second half walk this many rows fewer
			int silu_mul;          // 1: w[0] = gate, w[1] = up, row 2i + m; y[0][i] = silu(gate_i) * up_i
			// kBlockTeams vectors, partial_stride floats apart, that the decoder-block kernel left in place
			// of the attention half's result: added, in team order, onto x while it is staged
			// (partials_on == 1; K = 4096 only) or onto the residual in the epilogue (partials_on == 2)
			const float* partials;
			uint32_t partial_stride;
			int partials_on;
		};

		// teams of the decoder-block kernel (the card's XCDs)
		constexpr int kBlockTeams = 8;

		__device__ __forceinline__ void locate_row(const GemvArgs& a, int vr, int& m, int& local)
		{
			if (a.silu_mul)
			{
				m = vr & 1;
				local = vr >> 1;
				return;
			}
			m = 0;
			local = vr;
			if (local >= a.n[0])
			{
				local -= a.n[0];
				m = 1;
				if (local >= a.n[1])
				{
					local -= a.n[1];
					m = 2;
				}
			}
		}

		// vmcnt wait until at most ROWS rows of `loads_per_row` (1 .. 5, wavefront-uniform) load
		// instructions are outstanding
		template <int ROWS>
		__device__ __forceinline__ void wait_rows_outstanding(int loads_per_row)
		{
			if constexpr (ROWS == 0)
			{
				vm_wait<0>();
			}
			else
			{
				switch (loads_per_row)
				{
				case 1: vm_wait<ROWS * 1>(); break;
				case 2: vm_wait<ROWS * 2>(); break;
				case 3: vm_wait<ROWS * 3>(); break;
				case 4: vm_wait<ROWS * 4>(); break;
				default: vm_wait<ROWS * 5>(); break;
				}
			}
		}

		template <int MAX>
		__device__ __forceinline__ void wait_rows_outstanding_dyn(int rows, int loads_per_row)
		{
			if constexpr (MAX == 0)
			{
				vm_wait<0>();
			}
			else
			{
				if (rows >= MAX)
				{
					wait_rows_outstanding<MAX>(loads_per_row);
				}
				else
				{
					wait_rows_outstanding_dyn<MAX - 1>(rows, loads_per_row);
				}
			}
		}

		template <int Ctrl, int RowMask>
		__device__ __forceinline__ double dpp_f64(double x)
		{
			const unsigned long long b = __builtin_bit_cast(unsigned long long, x);
			const unsigned lo = static_cast<unsigned>(
			    __builtin_amdgcn_update_dpp(0, static_cast<int>(b), Ctrl, RowMask, 0xF, false));
			const unsigned hi = static_cast<unsigned>(
			    __builtin_amdgcn_update_dpp(0, static_cast<int>(b >> 32), Ctrl, RowMask, 0xF, false));
			return __builtin_bit_cast(double, (static_cast<unsigned long long>(hi) << 32) | lo);
		}

		// f64 sum over the wavefront with DPP on the two halves; the total is returned in every lane
		__device__ __forceinline__ double wave_sum_f64(double v)
		{
			v += dpp_f64<0xB1, 0xF>(v);
			v += dpp_f64<0x4E, 0xF>(v);
			v += dpp_f64<0x141, 0xF>(v);
			v += dpp_f64<0x140, 0xF>(v);
			v += dpp_f64<0x142, 0xA>(v);
			v += dpp_f64<0x143, 0xC>(v);
			const unsigned long long b = __builtin_bit_cast(unsigned long long, v);
			const unsigned lo = static_cast<unsigned>(__builtin_amdgcn_readlane(static_cast<int>(b), 63));
			const unsigned hi = static_cast<unsigned>(__builtin_amdgcn_readlane(static_cast<int>(b >> 32), 63));
			return __builtin_bit_cast(double, (static_cast<unsigned long long>(hi) << 32) | lo);
		}

		// silu(g) * u with the separately rounded steps of the reference chain
		// (Activation.h:22-35,56-63; SwiGLU.h:63-66)
		__device__ __forceinline__ float silu_mul_value(float g, float u)
		{
			const float sig = __fdiv_rn(1.0f, __fadd_rn(1.0f, expf(-g)));
			return __fmul_rn(__fmul_rn(g, sig), u);
		}

		// A launch is one or two parts: workgroups [0, blocks0) walk part 0, the rest part 1, whose
		// matrices may have another block format (q/k in one format and v in another share a launch).
		struct GemvLaunch
		{
			GemvArgs part[2];
			int blocks0;
		};

		// The statements live in gemv_stream_body.inc and are compiled into both forms below.
		// The first six arguments repeat fields of the argument block: the dispatcher hands the leading
		// kernel arguments over in registers (this file is compiled with kernel-argument preloading for
		// six of them), so the activation loads and the first row requests do not wait for the block to
		// be read from memory; on a card whose firmware does not preload, the kernel's compatibility
		// prologue loads them like any other argument.
		template <typename U, int XP, bool WHOLE, int THREADS = 512>
		__global__ __launch_bounds__(THREADS) void gemv_stream_kernel(const float* x_first, int k_first,
		                                                           const uint8_t* w0_first, uint32_t row_bytes_first,
		                                                           int rows_per_group_first, int n_total_first,
		                                                           const GemvArgs block_args)
		{
			GemvArgs a = block_args;
			a.x = x_first;
			a.k = k_first;
			a.w[0] = w0_first;
			a.row_bytes = row_bytes_first;
			a.rows_per_group = rows_per_group_first;
			a.n_total = n_total_first;
			const int block = static_cast<int>(blockIdx.x);
			constexpr bool kWholeSlices = WHOLE;
			constexpr bool kEarlyActivations = true;
			constexpr bool kTeamRows = false;
			constexpr int team = 0;
			constexpr int kTeamExtraLoads = 0;
			const auto team_prefetch = [] {};
#include "gemv_stream_body.inc"
		}

		template <typename U, int XP>
		__device__ __forceinline__ void gemv_stream_part(const GemvArgs a, const int block)
		{
			constexpr bool kWholeSlices = false;
			constexpr bool kEarlyActivations = false;
			constexpr bool kTeamRows = false;
			constexpr int team = 0;
			constexpr int kTeamExtraLoads = 0;
			const auto team_prefetch = [] {};
#include "gemv_stream_body.inc"
		}


		template <typename U0, typename U1, int XP>
		__global__ __launch_bounds__(512) void gemv_stream_pair_kernel(const GemvLaunch launch)
		{
			// uniform per workgroup
			if (static_cast<int>(blockIdx.x) < launch.blocks0)
			{
				gemv_stream_part<U0, XP>(launch.part[0], static_cast<int>(blockIdx.x));
			}
			else
			{
				gemv_stream_part<U1, XP>(launch.part[1], static_cast<int>(blockIdx.x) - launch.blocks0);
			}
		}

		// ------------------------------------------------------------------
		// Register kernel: the same decomposition with the rows loaded straight into registers.
		// Used for shapes the streaming kernel does not take (rows that are not a multiple of 16
		// bytes, K beyond what fits in LDS).  One row is prefetched while the previous one is
		// consumed.
		// ------------------------------------------------------------------
		template <typename U>
		__global__ __launch_bounds__(512) void gemv_kernel(const uint8_t* __restrict__ w, const float* __restrict__ x,
		                                                    float* __restrict__ y,
		                                                    const float* __restrict__ residual, int n, int k,
		                                                    size_t row_bytes, int slices, int groups,
		                                                    int rows_per_wave)
		{
			extern __shared__ __attribute__((aligned(16))) float part[]; // [slices][groups * rows_per_wave]
			const int lane = threadIdx.x & 63;
			const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
			const int s = wave % slices;
			const int g = wave / slices;
			const int unit = s * 64 + lane;
			const int units_per_row = k >> 6;
			const bool active = unit < units_per_row;
			const int row0 = (blockIdx.x * groups + g) * rows_per_wave;
			const int row_end = min(row0 + rows_per_wave, n);

			typename U::Raw cur, nxt;
			if (active && row0 < row_end)
			{
				cur = U::load(w + static_cast<size_t>(row0) * row_bytes, unit);
			}
			float xr[64];
			if (active)
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
			else
			{
#pragma unroll
				for (int i = 0; i < 64; ++i)
				{
					xr[i] = 0.0f;
				}
			}
			const typename U::Prep pz = U::prep(xr);

			float res = 0.0f; // lane i keeps the total of row row0 + i
			for (int r = row0; r < row_end; ++r)
			{
				if (active && r + 1 < row_end)
				{
					nxt = U::load(w + static_cast<size_t>(r + 1) * row_bytes, unit);
				}
				const float p = active ? unit_dot<U>(cur, xr, pz, unit) : 0.0f;
				const float total = wave_sum(p);
				res = (lane == r - row0) ? total : res;
				cur = nxt;
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
			case LITENN_FMT_Q4_1: // { fp16 d; fp16 m; u8 qs[16]; }: q d + m
			{
				const uint8_t* b = row + static_cast<size_t>(k_idx >> 5) * 20;
				const int j = k_idx & 31;
				const float d = f16_bits_to_f32(b[0] | (b[1] << 8));
				const float m = f16_bits_to_f32(b[2] | (b[3] << 8));
				const int q = j < 16 ? (b[4 + j] & 0xF) : (b[4 + j - 16] >> 4);
				return __fadd_rn(__fmul_rn(static_cast<float>(q), d), m);
			}
			case LITENN_FMT_Q5_0: // { fp16 d; u8 qh[4]; u8 qs[16]; }: bit j of qh is the fifth bit of element j
			{
				const uint8_t* b = row + static_cast<size_t>(k_idx >> 5) * 22;
				const int j = k_idx & 31;
				const float d = f16_bits_to_f32(b[0] | (b[1] << 8));
				const int high = (b[2 + (j >> 3)] >> (j & 7)) & 1;
				const int low = j < 16 ? (b[6 + j] & 0xF) : (b[6 + j - 16] >> 4);
				return static_cast<float>((low | (high << 4)) - 16) * d;
			}
			case LITENN_FMT_Q5_1: // { fp16 d; fp16 m; u8 qh[4]; u8 qs[16]; }
			{
				const uint8_t* b = row + static_cast<size_t>(k_idx >> 5) * 24;
				const int j = k_idx & 31;
				const float d = f16_bits_to_f32(b[0] | (b[1] << 8));
				const float m = f16_bits_to_f32(b[2] | (b[3] << 8));
				const int high = (b[4 + (j >> 3)] >> (j & 7)) & 1;
				const int low = j < 16 ? (b[8 + j] & 0xF) : (b[8 + j - 16] >> 4);
				return __fadd_rn(__fmul_rn(static_cast<float>(low | (high << 4)), d), m);
			}
			case LITENN_FMT_Q2_K: // { u8 scales[16]; u8 qs[64]; fp16 d; fp16 dmin; }
			{
				const uint8_t* b = row + static_cast<size_t>(k_idx >> 8) * 84;
				const int e = k_idx & 255;
				const int half = e >> 7, plane = (e >> 5) & 3, l = e & 31;
				const float d = f16_bits_to_f32(b[80] | (b[81] << 8));
				const float dmin = f16_bits_to_f32(b[82] | (b[83] << 8));
				const int sc = b[e >> 4];
				const int q = (b[16 + 32 * half + l] >> (2 * plane)) & 3;
				const float dl = __fmul_rn(d, static_cast<float>(sc & 0xF));
				const float ml = __fmul_rn(dmin, static_cast<float>(sc >> 4));
				return __fsub_rn(__fmul_rn(dl, static_cast<float>(q)), ml);
			}
			case LITENN_FMT_Q3_K: // { u8 hmask[32]; u8 qs[64]; u8 scales[12]; fp16 d; }
			{
				const uint8_t* b = row + static_cast<size_t>(k_idx >> 8) * 110;
				const int e = k_idx & 255;
				const int half = e >> 7, plane = (e >> 5) & 3, l = e & 31;
				const float d = f16_bits_to_f32(b[108] | (b[109] << 8));
				int q = (b[32 + 32 * half + l] >> (2 * plane)) & 3;
				if (!((b[l] >> (e >> 5)) & 1))
				{
					q -= 4;
				}
				// six-bit scale s, biased by 32: low four bits from nibble s / 8 of byte s % 8, top two
				// from bits 2 (s / 4) .. of byte 8 + s % 4
				const int s = e >> 4;
				const int low4 = (b[96 + (s & 7)] >> (4 * (s >> 3))) & 0xF;
				const int top2 = (b[104 + (s & 3)] >> (2 * (s >> 2))) & 3;
				const float dl = __fmul_rn(d, static_cast<float>((low4 | (top2 << 4)) - 32));
				return __fmul_rn(dl, static_cast<float>(q));
			}
			case LITENN_FMT_Q5_K: // { fp16 d; fp16 dmin; u8 scales[12]; u8 qh[32]; u8 qs[128]; }
			{
				const uint8_t* b = row + static_cast<size_t>(k_idx >> 8) * 176;
				const int e = k_idx & 255;
				const float d = f16_bits_to_f32(b[0] | (b[1] << 8));
				const float dmin = f16_bits_to_f32(b[2] | (b[3] << 8));
				const uint8_t* sc = b + 4;
				const int j = e >> 5, l = e & 31; // sub-block, element
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
				const uint8_t byte = b[48 + (j >> 1) * 32 + l];
				const int q = ((j & 1) ? (byte >> 4) : (byte & 0xF)) + 16 * ((b[16 + l] >> j) & 1);
				const float d1 = __fmul_rn(d, static_cast<float>(s));
				const float m1 = __fmul_rn(dmin, static_cast<float>(m));
				return __fsub_rn(__fmul_rn(d1, static_cast<float>(q)), m1);
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
			// several elements per thread in flight: the per-element decode is a chain of dependent
			// byte loads, and a single-token step waits for this kernel
#pragma unroll 4
			for (int i = threadIdx.x; i < k; i += blockDim.x)
			{
				out[static_cast<size_t>(blockIdx.x) * k + i] = generic_elem(fmt, rp, i);
			}
		}

		int compute_units()
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

		// What the calling thread's last streaming launch was (litenn_hip_gemv_last_launch formats it)
		struct StreamLaunchRecord
		{
			const char* kernel = nullptr; // gemv_stream_kernel or gemv_stream_pair_kernel
			const char* unit0 = "";
			const char* unit1 = "";
			int xp = 0, whole = 0, instance_threads = 0;
			int blocks = 0, threads = 0, rows = 0, run_diff = 0;
			size_t lds = 0;
		};
		thread_local StreamLaunchRecord t_last_stream_launch;

		template <typename U> constexpr const char* unit_name() { return "Unit"; }
		template <> constexpr const char* unit_name<Q4_0Unit>() { return "Q4_0Unit"; }
		template <> constexpr const char* unit_name<Q4_1Unit>() { return "Q4_1Unit"; }
		template <> constexpr const char* unit_name<Q5_0Unit>() { return "Q5_0Unit"; }
		template <> constexpr const char* unit_name<Q5_1Unit>() { return "Q5_1Unit"; }
		template <> constexpr const char* unit_name<Q8_0Unit>() { return "Q8_0Unit"; }
		template <> constexpr const char* unit_name<Q2_KUnit>() { return "Q2_KUnit"; }
		template <> constexpr const char* unit_name<Q3_KUnit>() { return "Q3_KUnit"; }
		template <> constexpr const char* unit_name<Q4_KUnit>() { return "Q4_KUnit"; }
		template <> constexpr const char* unit_name<Q5_KUnit>() { return "Q5_KUnit"; }
		template <> constexpr const char* unit_name<Q6_KUnit>() { return "Q6_KUnit"; }

		template <typename U0, typename U1>
		void record_stream_launch(const char* kernel, int xp, bool whole, int instance_threads, const GemvLaunch& launch,
		                          int blocks, int threads, size_t lds)
		{
			StreamLaunchRecord& r = t_last_stream_launch;
			r.kernel = kernel;
			r.unit0 = unit_name<U0>();
			r.unit1 = unit_name<U1>();
			r.xp = xp;
			r.whole = whole ? 1 : 0;
			r.instance_threads = instance_threads;
			r.blocks = blocks;
			r.threads = threads;
			r.rows = launch.part[0].rows_per_group;
			r.run_diff = launch.part[0].run_diff;
			r.lds = lds;
		}

		// Returns false, with nothing launched, when no instance of the kernel was compiled for the
		// geometry (the caller then takes the register kernel).
		template <typename U0, typename U1, int XP>
		bool launch_stream_variant(const GemvLaunch& launch, int blocks, int threads, size_t lds, hipStream_t stream)
		{
			if constexpr (std::is_same<U0, U1>::value)
			{
				const GemvArgs& g = launch.part[0];
				// K = 4096 is most of a decoder's launches: its own instance with the slice geometry folded
				if (XP == 2 && g.k == 4096 && threads == 512)
				{
					allow_dynamic_lds(reinterpret_cast<const void*>(&gemv_stream_kernel<U0, 2, true>), kStreamLdsLimit);
					gemv_stream_kernel<U0, 2, true><<<dim3(blocks), dim3(threads), lds, stream>>>(g.x, g.k, g.w[0], g.row_bytes,
					                                                                         g.rows_per_group, g.n_total, g);
					record_stream_launch<U0, U1>("gemv_stream_kernel", 2, true, 512, launch, blocks, threads, lds);
					return true;
				}
				if (threads > 512)
				{
					// twelve wavefronts (three-slice rows): an instance compiled for that many
					if constexpr (XP == kTwelveXp)
					{
						if (threads != 768)
						{
							return false;
						}
						allow_dynamic_lds(reinterpret_cast<const void*>(&gemv_stream_kernel<U0, XP, false, 768>), kStreamLdsLimit);
						gemv_stream_kernel<U0, XP, false, 768><<<dim3(blocks), dim3(threads), lds, stream>>>(
						    g.x, g.k, g.w[0], g.row_bytes, g.rows_per_group, g.n_total, g);
						record_stream_launch<U0, U1>("gemv_stream_kernel", XP, false, 768, launch, blocks, threads, lds);
						return true;
					}
					return false;
				}
				allow_dynamic_lds(reinterpret_cast<const void*>(&gemv_stream_kernel<U0, XP, false>), kStreamLdsLimit);
				gemv_stream_kernel<U0, XP, false><<<dim3(blocks), dim3(threads), lds, stream>>>(g.x, g.k, g.w[0], g.row_bytes,
				                                                                         g.rows_per_group, g.n_total, g);
				record_stream_launch<U0, U1>("gemv_stream_kernel", XP, false, 512, launch, blocks, threads, lds);
				return true;
			}
			else
			{
				if (threads > 512)
				{
					return false;
				}
				allow_dynamic_lds(reinterpret_cast<const void*>(&gemv_stream_pair_kernel<U0, U1, XP>), kStreamLdsLimit);
				gemv_stream_pair_kernel<U0, U1, XP><<<dim3(blocks), dim3(threads), lds, stream>>>(launch);
				record_stream_launch<U0, U1>("gemv_stream_pair_kernel", XP, false, 512, launch, blocks, threads, lds);
				return true;
			}
		}

		// Fills the launch geometry of one part for a budget of `max_blocks` workgroups (one round, at
		// most one per CU, every group walking the same number of rows, an even number when gate/up
		// rows are paired).  Returns false when the shape does not fit the streaming kernel.
		// twelve: the launch may use twelve wavefronts (the single-format kernel has an instance for
		// them; the two-format kernel has not)
		template <typename U>
		bool plan_stream(GemvArgs& a, int max_blocks, int& blocks, size_t& lds, bool twelve = false)
		{
			const int k = a.k;
			a.slices = (k + 4095) / 4096;
			if (a.slices > kMaxSlices || a.row_bytes % 16 != 0)
			{
				return false;
			}
			for (int m = 0; m < 3; ++m)
			{
				if (a.n[m] > 0 && reinterpret_cast<uintptr_t>(a.w[m]) % 16 != 0)
				{
					return false;
				}
			}
			if (reinterpret_cast<uintptr_t>(a.x) % 16 != 0 || (a.norm_w && reinterpret_cast<uintptr_t>(a.norm_w) % 16 != 0))
			{
				return false;
			}
			a.groups = 8 / a.slices;
			// Rows of three slices (8192 < K <= 12288): two groups of three wavefronts put two
			// wavefronts on two of the SIMDs and one on the other two; four groups give every SIMD
			// three (4096 x 11008: 8.9 -> 8.1 us, 7B-shape decode 752 -> 767 tok/s).
			static const int use_twelve = env_int("LITENN_HIP_GEMV_TWELVE", 1);
			if (twelve && use_twelve && a.slices == 3 && (k / 4 + 767) / 768 <= kTwelveXp && (k / 4 + 767) / 768 > kTwelveXp / 2 &&
			    sizeof(float) * (static_cast<size_t>(k) / 64) * kLdsUnitStride + 12 * kPrefetchRows * U::kSliceBytes + 4096 <=
			        kStreamLdsLimit)
			{
				a.groups = 4;
			}
			const int nwaves = a.slices * a.groups;
			if (k > 64 * nwaves * 4 * kXPerThread)
			{
				return false;
			}
			const size_t x_bytes = sizeof(float) * (static_cast<size_t>(k) / 64) * kLdsUnitStride;
			static const int forced_rows = env_int("LITENN_HIP_GEMV_ROWS", 0);
			int rows = (a.n_total + max_blocks * a.groups - 1) / (max_blocks * a.groups);
			if (forced_rows > 0)
			{
				rows = forced_rows;
			}
			rows = std::min(std::max(rows, 1), kMaxStreamRows);
			if (a.silu_mul && (rows & 1))
			{
				++rows;
			}
			int diff = 0;
			// Of the two wavefronts that share a SIMD the one that arrived first wins the issue
			// arbitration and finishes about a seventh of the walk ahead of the other (north-star
			// launch, 7 rows each: 5.85 against 6.79 us).  So the rows are dealt out per pair of
			// groups that share SIMDs - with eight wavefronts in an even number of groups, group g of
			// the first half and group g of the second - and the first takes about a seventh of the
			// pair's rows more than the second (8 and 6 rows: 7.80 -> 7.42 us; 7B-shape decode
			// 729 -> 738 tok/s; runs of 3 and 1 for 4096 x 4096: 6.28 -> 5.87 us).  The pair's total need
			// not be even (11 rows as 6 + 5 where equal runs would take 6 + 6 on fewer workgroups);
			// gate/up pairs keep both runs even.  The six wavefronts of K = 11008 gain nothing from an
			// uneven split (8.9 -> 8.85 us) and keep equal runs.
			static const int forced_diff = env_int("LITENN_HIP_GEMV_SKEW", -1); // 0: equal runs
			if (nwaves == 8 && a.groups % 2 == 0 && forced_rows <= 0 && forced_diff != 0)
			{
				const int unit = a.silu_mul ? 2 : 1; // a run is a whole number of these
				const int half_groups = a.groups / 2;
				int total = (a.n_total + max_blocks * half_groups - 1) / (max_blocks * half_groups); // rows of a pair
				total = std::max((total + unit - 1) / unit * unit, 2 * unit);
				// the nearest difference to a seventh of the total (at least one unit) that leaves both
				// runs whole numbers of units
				int best = -1;
				for (int d = 0; d < total; d += unit)
				{
					if ((total + d) % (2 * unit) != 0 || (total - d) / 2 < unit || (total + d) / 2 > kMaxStreamRows)
					{
						continue;
					}
					const int target = forced_diff > 0 ? 7 * forced_diff : std::max(total, 7 * unit);
					if (best < 0 || std::abs(7 * d - target) <= std::abs(7 * best - target))
					{
						best = d;
					}
				}
				if (best >= 0)
				{
					rows = (total + best) / 2;
					diff = best;
				}
			}
			a.rows_per_group = rows;
			a.run_diff = diff;
			const int block_rows = fetch::stream_block_rows(a.groups, rows, diff);
			blocks = (a.n_total + block_rows - 1) / block_rows;
			lds = x_bytes + static_cast<size_t>(nwaves) * kPrefetchRows * U::kSliceBytes +
			      ((sizeof(float) * nwaves * rows + 7) & ~size_t{ 7 }) + sizeof(double) * nwaves;
			return lds <= kStreamLdsLimit;
		}

		// more than half of the CU's LDS: the dispatcher cannot stack two of these workgroups on one
		// CU while another CU has none
		size_t exclusive_lds(size_t lds)
		{
			static const int exclusive = env_int("LITENN_HIP_GEMV_EXCLUSIVE", 1);
			return exclusive ? std::max(lds, kStreamLdsLimit / 2 + 1024) : lds;
		}

		template <typename U0, typename U1>
		bool launch_stream_xp(const GemvLaunch& launch, int blocks, size_t lds, hipStream_t stream)
		{
			const GemvArgs& a = launch.part[0];
			const int threads = 64 * a.slices * a.groups;
			const int per_thread = (a.k / 4 + threads - 1) / threads; // 128-bit activation loads per thread
			if (per_thread <= 2)
			{
				return launch_stream_variant<U0, U1, 2>(launch, blocks, threads, lds, stream);
			}
			if (per_thread <= 4)
			{
				return launch_stream_variant<U0, U1, 4>(launch, blocks, threads, lds, stream);
			}
			return launch_stream_variant<U0, U1, kXPerThread>(launch, blocks, threads, lds, stream);
		}

		template <typename U>
		bool launch_stream(GemvArgs a, hipStream_t stream, bool plan_only = false)
		{
			int blocks = 0;
			size_t lds = 0;
			if (!plan_stream<U>(a, compute_units(), blocks, lds, true))
			{
				return false;
			}
			if (plan_only)
			{
				return true;
			}
			GemvLaunch launch{};
			launch.part[0] = a;
			launch.blocks0 = blocks;
			return launch_stream_xp<U, U>(launch, blocks, exclusive_lds(lds), stream);
		}

		// Two parts of different block formats over the same activations in one launch.  The CUs are
		// shared out so that the slower part finishes as early as possible: a group's time goes with
		// its run length times the bytes of its rows.
		template <typename U0, typename U1>
		bool launch_stream_pair(GemvArgs a0, GemvArgs a1, hipStream_t stream)
		{
			const int cus = compute_units();
			long best_cost = -1;
			int best_b0 = 0;
			for (int b0 = 1; b0 < cus; ++b0)
			{
				GemvArgs t0 = a0, t1 = a1;
				int blocks0 = 0, blocks1 = 0;
				size_t lds0 = 0, lds1 = 0;
				if (!plan_stream<U0>(t0, b0, blocks0, lds0) || !plan_stream<U1>(t1, cus - b0, blocks1, lds1))
				{
					return false; // the fit does not depend on the share
				}
				const long cost = std::max(static_cast<long>(t0.rows_per_group) * t0.row_bytes,
				                           static_cast<long>(t1.rows_per_group) * t1.row_bytes);
				if (best_cost < 0 || cost < best_cost)
				{
					best_cost = cost;
					best_b0 = b0;
				}
			}
			int blocks0 = 0, blocks1 = 0;
			size_t lds0 = 0, lds1 = 0;
			if (best_cost < 0 || !plan_stream<U0>(a0, best_b0, blocks0, lds0) ||
			    !plan_stream<U1>(a1, cus - best_b0, blocks1, lds1) || a0.slices != a1.slices || a0.groups != a1.groups)
			{
				return false;
			}
			GemvLaunch launch{};
			launch.part[0] = a0;
			launch.part[1] = a1;
			launch.blocks0 = blocks0;
			return launch_stream_xp<U0, U1>(launch, blocks0 + blocks1, exclusive_lds(std::max(lds0, lds1)), stream);
		}

		template <typename U>
		void launch_register(const uint8_t* w, const float* x, float* y, const float* residual, int n, int k, size_t rb,
		                     hipStream_t stream)
		{
			const int slices = (k + 4095) / 4096;
			int groups = 8 / slices;
			if (groups < 1)
			{
				groups = 1;
			}
			const int target_waves = 8 * compute_units();
			int rows_per_wave = (n * slices + target_waves - 1) / target_waves;
			rows_per_wave = rows_per_wave < 1 ? 1 : (rows_per_wave > kMaxRowsPerWave ? kMaxRowsPerWave : rows_per_wave);
			const int rows_per_block = groups * rows_per_wave;
			const int blocks = (n + rows_per_block - 1) / rows_per_block;
			const size_t lds = slices > 1 ? sizeof(float) * slices * rows_per_block : 0;
			gemv_kernel<U><<<dim3(blocks), dim3(64 * slices * groups), lds, stream>>>(w, x, y, residual, n, k, rb, slices,
			                                                                         groups, rows_per_wave);
		}

		bool is_block_format(int fmt)
		{
			return fmt == LITENN_FMT_Q4_0 || fmt == LITENN_FMT_Q4_1 || fmt == LITENN_FMT_Q5_0 || fmt == LITENN_FMT_Q5_1 ||
			       fmt == LITENN_FMT_Q8_0 || fmt == LITENN_FMT_Q2_K || fmt == LITENN_FMT_Q3_K || fmt == LITENN_FMT_Q4_K ||
			       fmt == LITENN_FMT_Q5_K || fmt == LITENN_FMT_Q6_K;
		}

		bool stream_dispatch(int fmt, const GemvArgs& a, hipStream_t stream, bool plan_only = false)
		{
			// LITENN_HIP_GEMV_STREAM=0 keeps the rows in registers instead of LDS
			static const int use_stream = env_int("LITENN_HIP_GEMV_STREAM", 1);
			if (!use_stream || !is_block_format(fmt) || a.k % 256 != 0)
			{
				return false;
			}
			switch (fmt)
			{
			case LITENN_FMT_Q4_0: return launch_stream<Q4_0Unit>(a, stream, plan_only);
			case LITENN_FMT_Q4_1: return launch_stream<Q4_1Unit>(a, stream, plan_only);
			case LITENN_FMT_Q5_0: return launch_stream<Q5_0Unit>(a, stream, plan_only);
			case LITENN_FMT_Q5_1: return launch_stream<Q5_1Unit>(a, stream, plan_only);
			case LITENN_FMT_Q8_0: return launch_stream<Q8_0Unit>(a, stream, plan_only);
			case LITENN_FMT_Q2_K: return launch_stream<Q2_KUnit>(a, stream, plan_only);
			case LITENN_FMT_Q3_K: return launch_stream<Q3_KUnit>(a, stream, plan_only);
			case LITENN_FMT_Q4_K: return launch_stream<Q4_KUnit>(a, stream, plan_only);
			case LITENN_FMT_Q5_K: return launch_stream<Q5_KUnit>(a, stream, plan_only);
			default: return launch_stream<Q6_KUnit>(a, stream, plan_only);
			}
		}

		// the format pairs that share a launch: the K-quant mixes of llama.cpp keep some projections
		// (attn_v among q/k/v) in Q6_K beside Q4_K or Q5_K ones
		bool stream_dispatch_pair(int fmt0, int fmt1, const GemvArgs& a0, const GemvArgs& a1, hipStream_t stream)
		{
			static const int use_stream = env_int("LITENN_HIP_GEMV_STREAM", 1);
			static const int use_pairs = env_int("LITENN_HIP_GEMV_PAIRS", 1);
			if (!use_stream || !use_pairs || a0.k % 256 != 0)
			{
				return false;
			}
			if (fmt0 == LITENN_FMT_Q4_K && fmt1 == LITENN_FMT_Q6_K)
			{
				return launch_stream_pair<Q4_KUnit, Q6_KUnit>(a0, a1, stream);
			}
			if (fmt0 == LITENN_FMT_Q5_K && fmt1 == LITENN_FMT_Q6_K)
			{
				return launch_stream_pair<Q5_KUnit, Q6_KUnit>(a0, a1, stream);
			}
			return false;
		}

		// arguments of one part: `count` same-format matrices over x
		bool fill_args(GemvArgs& a, int fmt, int count, const void* const* w, float* const* y, const size_t* n, size_t k,
		               const float* x, const float* residual, const float* norm_w, double eps, bool silu_mul)
		{
			if (count < 1 || count > 3 || k > 0x7fffffffu || (silu_mul && (count != 2 || n[0] != n[1])) ||
			    (residual && count != 1))
			{
				return false;
			}
			a = GemvArgs{};
			size_t total = 0;
			for (int m = 0; m < count; ++m)
			{
				if (n[m] == 0 || n[m] > 0x3fffffffu)
				{
					return false;
				}
				a.w[m] = static_cast<const uint8_t*>(w[m]);
				a.y[m] = y[m];
				a.n[m] = static_cast<int>(n[m]);
				total += n[m];
			}
			if (total > 0x7fffffffu)
			{
				return false;
			}
			const size_t rb = row_bytes(fmt, k);
			if (rb == 0 || rb > 0xffffffffull)
			{
				return false;
			}
			a.x = x;
			a.residual = residual;
			a.norm_w = norm_w;
			a.eps = eps;
			a.n_total = static_cast<int>(total);
			a.k = static_cast<int>(k);
			a.row_bytes = static_cast<uint32_t>(rb);
			a.silu_mul = silu_mul ? 1 : 0;
			a.partials = nullptr;
			a.partial_stride = 0;
			a.partials_on = 0;
			return true;
		}

#include "attn_block.inc"
	} // namespace

	// One fused launch over up to three same-format matrices that share x (see GemvArgs).  Returns
	// false, launching nothing, when the streaming kernel does not take the shape; the caller then
	// composes the operators from separate launches.
	bool launch_gemv_fused(int fmt, int count, const void* const* w, float* const* y, const size_t* n, size_t k,
	                       const float* x, const float* residual, const float* norm_w, double eps, bool silu_mul,
	                       hipStream_t stream)
	{
		GemvArgs a;
		return fill_args(a, fmt, count, w, y, n, k, x, residual, norm_w, eps, silu_mul) && stream_dispatch(fmt, a, stream);
	}

	// The same for two or three matrices of two block formats (fmts[i] per matrix, equal formats
	// adjacent): one launch whose workgroups are shared out between the two formats.  Returns false,
	// launching nothing, when the formats are not such a pair or the shape does not fit.
	bool launch_gemv_fused_mixed(const int* fmts, int count, const void* const* w, float* const* y, const size_t* n,
	                             size_t k, const float* x, const float* norm_w, double eps, hipStream_t stream)
	{
		if (count < 2 || count > 3)
		{
			return false;
		}
		int first = 1; // matrices of the first format
		while (first < count && fmts[first] == fmts[0])
		{
			++first;
		}
		if (first == count)
		{
			return launch_gemv_fused(fmts[0], count, w, y, n, k, x, nullptr, norm_w, eps, false, stream);
		}
		for (int i = first + 1; i < count; ++i)
		{
			if (fmts[i] != fmts[first])
			{
				return false; // three formats
			}
		}
		GemvArgs a0, a1;
		if (!fill_args(a0, fmts[0], first, w, y, n, k, x, nullptr, norm_w, eps, false) ||
		    !fill_args(a1, fmts[first], count - first, w + first, y + first, n + first, k, x, nullptr, norm_w, eps, false))
		{
			return false;
		}
		return stream_dispatch_pair(fmts[0], fmts[first], a0, a1, stream);
	}

	// y[m, n] = x[m, k] . W^T (+ residual), one activation row at a time.
	int launch_gemv(int fmt, const void* wq, size_t n, size_t k, const float* x, size_t m, float* y,
	                const float* residual, hipStream_t stream)
	{
		const size_t rb = row_bytes(fmt, k);
		const uint8_t* w = static_cast<const uint8_t*>(wq);
		// register kernel: whole 64-weight units, 16-byte aligned activations, K within the slice budget
		const bool regs_ok = is_block_format(fmt) && (k % 256 == 0) && k <= static_cast<size_t>(kMaxSlices) * 4096 &&
		                     (reinterpret_cast<uintptr_t>(w) % 4 == 0) && env_int("LITENN_HIP_GEMV_GENERIC", 0) == 0;
		for (size_t i = 0; i < m; ++i)
		{
			const float* xi = x + i * k;
			float* yi = y + i * n;
			const float* ri = residual ? residual + i * n : nullptr;
			const void* ws[1] = { wq };
			float* ys[1] = { yi };
			const size_t ns[1] = { n };
			if (env_int("LITENN_HIP_GEMV_GENERIC", 0) == 0 &&
			    launch_gemv_fused(fmt, 1, ws, ys, ns, k, xi, ri, nullptr, 0.0, false, stream))
			{
				continue;
			}
			if (regs_ok && (reinterpret_cast<uintptr_t>(xi) % 16 == 0))
			{
				switch (fmt)
				{
				case LITENN_FMT_Q4_0:
					launch_register<Q4_0Unit>(w, xi, yi, ri, static_cast<int>(n), static_cast<int>(k), rb, stream);
					break;
				case LITENN_FMT_Q4_1:
					launch_register<Q4_1Unit>(w, xi, yi, ri, static_cast<int>(n), static_cast<int>(k), rb, stream);
					break;
				case LITENN_FMT_Q5_0:
					launch_register<Q5_0Unit>(w, xi, yi, ri, static_cast<int>(n), static_cast<int>(k), rb, stream);
					break;
				case LITENN_FMT_Q5_1:
					launch_register<Q5_1Unit>(w, xi, yi, ri, static_cast<int>(n), static_cast<int>(k), rb, stream);
					break;
				case LITENN_FMT_Q8_0:
					launch_register<Q8_0Unit>(w, xi, yi, ri, static_cast<int>(n), static_cast<int>(k), rb, stream);
					break;
				case LITENN_FMT_Q2_K:
					launch_register<Q2_KUnit>(w, xi, yi, ri, static_cast<int>(n), static_cast<int>(k), rb, stream);
					break;
				case LITENN_FMT_Q3_K:
					launch_register<Q3_KUnit>(w, xi, yi, ri, static_cast<int>(n), static_cast<int>(k), rb, stream);
					break;
				case LITENN_FMT_Q4_K:
					launch_register<Q4_KUnit>(w, xi, yi, ri, static_cast<int>(n), static_cast<int>(k), rb, stream);
					break;
				case LITENN_FMT_Q5_K:
					launch_register<Q5_KUnit>(w, xi, yi, ri, static_cast<int>(n), static_cast<int>(k), rb, stream);
					break;
				default:
					launch_register<Q6_KUnit>(w, xi, yi, ri, static_cast<int>(n), static_cast<int>(k), rb, stream);
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

	void launch_rmsnorm(const float* x, const float* w, double eps, size_t m, size_t d, float* y, hipStream_t s);
	void launch_silu_mul(const float* gate, const float* up, float* y, size_t n, hipStream_t s);

	// RMSNorm (optional) -> up to three same-format linears over one activation row -> SwiGLU or
	// residual (optional): one fused launch when the streaming kernel takes the shape, otherwise the
	// same operators from separate launches.  scratch_x holds k floats (used when norm_w is given and
	// the fused kernel is not applicable); scratch_gate / scratch_up hold n[0] floats (same, SwiGLU).
	// Returns false, with nothing launched, when the group needs the composed form and no scratch
	// was handed over (scratch_x null): the caller allocates k + 2 n[0] floats and calls again.
	bool launch_linear_group(int fmt, int count, const void* const* w, float* const* y, const size_t* n, size_t k,
	                         const float* x, const float* residual, const float* norm_w, double eps, bool silu_mul,
	                         float* scratch_x, float* scratch_gate, float* scratch_up, hipStream_t stream)
	{
		static const int fuse = env_int("LITENN_HIP_FUSE", 1);
		if (fuse && launch_gemv_fused(fmt, count, w, y, n, k, x, residual, norm_w, eps, silu_mul, stream))
		{
			return true;
		}
		if (!scratch_x && (norm_w || silu_mul))
		{
			return false;
		}
		const float* xin = x;
		if (norm_w)
		{
			launch_rmsnorm(x, norm_w, eps, 1, k, scratch_x, stream);
			xin = scratch_x;
		}
		if (silu_mul)
		{
			launch_gemv(fmt, w[0], n[0], k, xin, 1, scratch_gate, nullptr, stream);
			launch_gemv(fmt, w[1], n[1], k, xin, 1, scratch_up, nullptr, stream);
			launch_silu_mul(scratch_gate, scratch_up, y[0], n[0], stream);
			return true;
		}
		for (int m = 0; m < count; ++m)
		{
			launch_gemv(fmt, w[m], n[m], k, xin, 1, y[m], m == 0 ? residual : nullptr, stream);
		}
		return true;
	}


	// The launches that follow the decoder-block kernel: an operator group as launch_gemv_fused runs it,
	// with the kernel's eight partial vectors (`stride` floats apart) added in team order onto x while
	// it is staged (on_x; k must be 4096) or onto the residual in the epilogue (!on_x).  Returns false,
	// with nothing launched, when the streaming kernel does not take the shape; plan_only launches
	// nothing in either case.
	bool launch_gemv_fused_partials(int fmt, int count, const void* const* w, float* const* y, const size_t* n, size_t k,
	                                const float* x, const float* residual, const float* norm_w, double eps, bool silu_mul,
	                                const float* partials, size_t stride, bool on_x, bool plan_only, hipStream_t stream)
	{
		GemvArgs a;
		if (!fill_args(a, fmt, count, w, y, n, k, x, residual, norm_w, eps, silu_mul) || !partials ||
		    (on_x && k != 4096) || (!on_x && !residual))
		{
			return false;
		}
		a.partials = partials;
		a.partial_stride = static_cast<uint32_t>(stride);
		a.partials_on = on_x ? 1 : 2;
		return stream_dispatch(fmt, a, stream, plan_only);
	}

	// The attention half of a decoder block for one new row as one launch (attn_block.inc).  Returns
	// false, with nothing launched, when the shape is not one the kernel is built for: 4096-wide model,
	// 32 heads of 128, a KV head count that is a multiple of 8, a Float16 cache, a card of 256 CUs, and
	// one of the format combinations instantiated below (one format throughout, or q, k and the output
	// projection in Q4_K / Q5_K beside a Q6_K v).  plan_only launches nothing in either case.
	// scratch: q / k / v take the first phase's rows (n_head * 128 and n_kv_head * 128 twice), triples
	// n_head * 8 * 132 floats, flags 512 words (zero before the model's first launch), y_partial 8 * d
	// floats; counters = {position, tokens emitted, steps run}; bit 1 of *err is set when a wait inside
	// the kernel ran out (a wait polls at most spin_limit times).
	bool launch_attn_block(const int* fmts, const void* const* wqkv, const size_t* n_qkv, int fmt_o, const void* wo,
	                       size_t d, const float* x, const float* norm_w, double eps, float* q, float* k, float* v,
	                       void* kcache, void* vcache, int cache_dtype, const float* cos_t, const float* sin_t,
	                       size_t rope_dims, const int* counters, int layer, size_t n_head, size_t n_kv_head,
	                       size_t head_dim, float* triples, unsigned* flags, float* y_partial, int* err, int spin_limit,
	                       bool plan_only, hipStream_t stream)
	{
		const auto aligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
		if (d != 4096 || n_head != 32 || head_dim != 128 || n_kv_head == 0 || n_kv_head % 8 != 0 ||
		    n_kv_head > 32 || cache_dtype != LITENN_F16 || rope_dims % 8 != 0 || rope_dims > 128 || rope_dims == 0 ||
		    compute_units() != 256 || n_qkv[0] != d || n_qkv[1] != n_kv_head * 128 || n_qkv[2] != n_kv_head * 128 ||
		    !aligned(q) || !aligned(k) || !aligned(v) || !aligned(kcache) || !aligned(vcache) ||
		    !aligned(cos_t) || !aligned(sin_t) || !aligned(wo) || !aligned(triples) || !aligned(y_partial) || !norm_w ||
		    layer < 0 || layer > 254)
		{
			return false;
		}
		float* ys[3] = { q, k, v };
		AttnBlockPlan plan{};
		GemvArgs a0, a1;
		bool ok = false;
		const bool one_format = fmts[0] == fmts[1] && fmts[1] == fmts[2] && fmt_o == fmts[0];
		// q and k in one K-quant format beside a Q6_K v, the attn_v choice of llama.cpp's K-quant mixes
		const bool k_mix = fmts[0] == fmts[1] && fmts[2] == LITENN_FMT_Q6_K && fmt_o == fmts[0] &&
		                   (fmts[0] == LITENN_FMT_Q4_K || fmts[0] == LITENN_FMT_Q5_K);
		if (one_format)
		{
			if (!fill_args(a0, fmts[0], 3, wqkv, ys, n_qkv, d, x, nullptr, norm_w, eps, false))
			{
				return false;
			}
			a1 = a0;
		}
		else if (k_mix)
		{
			if (!fill_args(a0, fmts[0], 2, wqkv, ys, n_qkv, d, x, nullptr, norm_w, eps, false) ||
			    !fill_args(a1, fmts[2], 1, wqkv + 2, ys + 2, n_qkv + 2, d, x, nullptr, norm_w, eps, false))
			{
				return false;
			}
		}
		else
		{
			return false;
		}
		// the instances: every block format whose 512-column segment of a row is a whole number of
		// 16-byte pieces (Q2_K, Q3_K and Q6_K output projections are not)
#define LITENN_BLOCK_INSTANCE(DO)                                                                                      \
	if (one_format && fmts[0] == LITENN_FMT_Q4_0) { DO(Q4_0Unit, Q4_0Unit, Q4_0Unit, false); }                         \
	else if (one_format && fmts[0] == LITENN_FMT_Q4_1) { DO(Q4_1Unit, Q4_1Unit, Q4_1Unit, false); }                    \
	else if (one_format && fmts[0] == LITENN_FMT_Q5_0) { DO(Q5_0Unit, Q5_0Unit, Q5_0Unit, false); }                    \
	else if (one_format && fmts[0] == LITENN_FMT_Q5_1) { DO(Q5_1Unit, Q5_1Unit, Q5_1Unit, false); }                    \
	else if (one_format && fmts[0] == LITENN_FMT_Q8_0) { DO(Q8_0Unit, Q8_0Unit, Q8_0Unit, false); }                    \
	else if (one_format && fmts[0] == LITENN_FMT_Q4_K) { DO(Q4_KUnit, Q4_KUnit, Q4_KUnit, false); }                    \
	else if (one_format && fmts[0] == LITENN_FMT_Q5_K) { DO(Q5_KUnit, Q5_KUnit, Q5_KUnit, false); }                    \
	else if (k_mix && fmts[0] == LITENN_FMT_Q4_K) { DO(Q4_KUnit, Q6_KUnit, Q4_KUnit, true); }                          \
	else if (k_mix && fmts[0] == LITENN_FMT_Q5_K) { DO(Q5_KUnit, Q6_KUnit, Q5_KUnit, true); }
#define LITENN_BLOCK_PLAN(U0, U1, UO, TWO) ok = (plan_attn_block<U0, U1, UO>(plan, a0, a1, TWO))
		LITENN_BLOCK_INSTANCE(LITENN_BLOCK_PLAN)
#undef LITENN_BLOCK_PLAN
		if (!ok)
		{
			return false;
		}
		if (plan_only)
		{
			return true;
		}
		AttnBlockArgs& f = plan.args;
		f.wo = static_cast<const uint8_t*>(wo);
		f.wo_row_bytes = static_cast<uint32_t>(row_bytes(fmt_o, d));
		f.wo_seg_bytes = f.wo_row_bytes / kBlockTeams;
		f.q = q;
		f.k_new = k;
		f.v_new = v;
		f.kcache = static_cast<uint16_t*>(kcache);
		f.vcache = static_cast<uint16_t*>(vcache);
		f.cos_t = cos_t;
		f.sin_t = sin_t;
		f.past_dev = counters;
		f.triples = triples;
		f.flags = flags;
		f.layer = layer;
		f.y_partial = y_partial;
		f.err = err;
		f.n_head = static_cast<int>(n_head);
		f.n_kv_head = static_cast<int>(n_kv_head);
		f.rope_dims = static_cast<int>(rope_dims);
		f.d = static_cast<int>(d);
		f.spin_limit = spin_limit;
#define LITENN_BLOCK_LAUNCH(U0, U1, UO, TWO) launch_attn_block_variant<U0, U1, UO>(plan, stream)
		LITENN_BLOCK_INSTANCE(LITENN_BLOCK_LAUNCH)
#undef LITENN_BLOCK_LAUNCH
#undef LITENN_BLOCK_INSTANCE
		return true;
	}

	void launch_dequantize(int fmt, const void* wq, size_t rows, size_t k, float* dst, hipStream_t stream)
	{
		dequantize_kernel<<<dim3(rows), dim3(256), 0, stream>>>(fmt, static_cast<const uint8_t*>(wq), dst, rows,
		                                                         static_cast<int>(k), row_bytes(fmt, k));
	}

	void launch_get_rows_q(int fmt, const void* table, size_t rows, size_t k, const int32_t* ids, size_t n_ids,
	                       float* out, int* err_flag, hipStream_t stream)
	{
		get_rows_q_kernel<<<dim3(n_ids), dim3(k >= 4096 ? 1024 : 256), 0, stream>>>(fmt, static_cast<const uint8_t*>(table),
		                                                          static_cast<int>(rows), static_cast<int>(k),
		                                                          row_bytes(fmt, k), ids, out, err_flag);
	}
} // namespace litenn_hip

extern "C" int litenn_hip_gemv_last_launch(char* out, size_t capacity)
{
	using namespace litenn_hip;
	if (!out || capacity == 0)
	{
		return fail("describe the last GEMV launch", "destination is null or empty");
	}
	const StreamLaunchRecord& r = t_last_stream_launch;
	if (!r.kernel)
	{
		std::snprintf(out, capacity, "none");
		return 0;
	}
	char name[160];
	if (std::strcmp(r.unit0, r.unit1) == 0)
	{
		std::snprintf(name, sizeof name, "%s<%s, %d, %s, %d>", r.kernel, r.unit0, r.xp, r.whole ? "true" : "false",
		              r.instance_threads);
	}
	else
	{
		std::snprintf(name, sizeof name, "%s<%s, %s, %d>", r.kernel, r.unit0, r.unit1, r.xp);
	}
	std::snprintf(out, capacity, "%s grid %d x %d threads, %zu B LDS, runs of %d and %d rows", name, r.blocks, r.threads,
	              r.lds, r.rows, r.rows - r.run_diff);
	return 0;
}

#ifdef LITENN_GEMV_TRACE
// Timeline build only: copies the stamps of the last streaming launch to the host
// ([wavefront][slot] of 100 MHz clock ticks, 0 where a slot was not reached) and clears them.
extern "C" int litenn_hip_gemv_trace_read(unsigned long long* dst, size_t entries)
{
	using namespace litenn_hip;
	constexpr size_t total = static_cast<size_t>(kTraceWaves) * kTraceSlots;
	if (!dst || entries > total)
	{
		return fail("read the GEMV timeline", "destination is null or asks for more than 4096 x 16 entries");
	}
	LITENN_HIP_TRY("read the GEMV timeline", hipDeviceSynchronize());
	LITENN_HIP_TRY("read the GEMV timeline",
	               hipMemcpyFromSymbol(dst, HIP_SYMBOL(g_trace), entries * sizeof(unsigned long long)));
	void* dev = nullptr;
	LITENN_HIP_TRY("read the GEMV timeline", hipGetSymbolAddress(&dev, HIP_SYMBOL(g_trace)));
	LITENN_HIP_TRY("read the GEMV timeline", hipMemset(dev, 0, total * sizeof(unsigned long long)));
	return 0;
}

// Timeline build only: the decoder-block kernel's stamps ([wavefront][8 points]) of its last launch
extern "C" int litenn_hip_block_trace_read(unsigned long long* dst, size_t entries)
{
	using namespace litenn_hip;
	constexpr size_t total = static_cast<size_t>(kTraceWaves) * kBlockTraceSlots;
	if (!dst || entries > total)
	{
		return fail("read the block timeline", "destination is null or asks for more than 4096 x 8 entries");
	}
	LITENN_HIP_TRY("read the block timeline", hipDeviceSynchronize());
	LITENN_HIP_TRY("read the block timeline",
	               hipMemcpyFromSymbol(dst, HIP_SYMBOL(g_block_trace), entries * sizeof(unsigned long long)));
	return 0;
}

// Timeline build only: 1 makes the streaming kernel fetch its rows and read them from LDS without
// multiplying them (results are then meaningless), which times the row traffic alone; 0 restores it.
extern "C" int litenn_hip_gemv_trace_skip_arithmetic(int skip)
{
	using namespace litenn_hip;
	const int value = skip ? 1 : 0;
	LITENN_HIP_TRY("set the GEMV timeline switch", hipDeviceSynchronize());
	LITENN_HIP_TRY("set the GEMV timeline switch",
	               hipMemcpyToSymbol(HIP_SYMBOL(g_trace_skip_arithmetic), &value, sizeof(value)));
	return 0;
}
#endif
