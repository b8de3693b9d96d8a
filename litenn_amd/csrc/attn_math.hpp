// litenn-hip: the arithmetic of one new row's attention step that more than one kernel shares: the
// separately rounded RoPE rotation, the cache type's rounding of the new key and value, the merge
// weight of partial softmax triples, and the device-scope accesses through which workgroups hand
// values to each other inside one launch.
#pragma once

#include "common.hpp"

#if defined(__HIPCC__)
namespace litenn_hip
{
	// f32 rotation with separately rounded products (RoPE.h:93-111), so the four multiplies
	// round like the reference's Multiply nodes.  The pragma is what keeps them apart: the
	// compiler contracts a * c - b * s into a fused multiply-add by default.
	__device__ __forceinline__ void rotate(float a, float b, float c, float s, float& o0, float& o1)
	{
#pragma clang fp contract(off)
		const float ac = a * c, bs = b * s, as = a * s, bc = b * c;
		o0 = ac - bs;
		o1 = as + bc;
	}

	__device__ __forceinline__ void device_store(float* p, float v)
	{
		__hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
	}
	__device__ __forceinline__ float device_load(const float* p)
	{
		return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
	}

	__device__ __forceinline__ float softmax_weight(float m, float m_all)
	{
		return m == -INFINITY ? 0.0f : expf(m - m_all);
	}

	template <typename KV>
	__device__ __forceinline__ float through_cache(float v);
	template <>
	__device__ __forceinline__ float through_cache<float>(float v) { return v; }
	template <>
	__device__ __forceinline__ float through_cache<uint16_t>(float v)
	{
		return f16_bits_to_f32(f32_to_f16_bits_litenn(v));
	}

	// The new row's key / value as the cache will hold them: rounded through the cache type once,
	// used from registers and stored from the same values.
	template <typename KV>
	__device__ __forceinline__ void round_through_cache(float (&v)[8])
	{
#pragma unroll
		for (int e = 0; e < 8; ++e)
		{
			v[e] = through_cache<KV>(v[e]);
		}
	}
	// values already representable in the cache type: the hardware conversion is exact for them
	__device__ __forceinline__ void store8_exact(float* dst, const float (&v)[8])
	{
		reinterpret_cast<float4*>(dst)[0] = make_float4(v[0], v[1], v[2], v[3]);
		reinterpret_cast<float4*>(dst)[1] = make_float4(v[4], v[5], v[6], v[7]);
	}
	__device__ __forceinline__ void store8_exact(uint16_t* dst, const float (&v)[8])
	{
		typedef _Float16 half2v __attribute__((ext_vector_type(2)));
		typedef float float2v __attribute__((ext_vector_type(2)));
		uint32_t w[4];
#pragma unroll
		for (int i = 0; i < 4; ++i)
		{
			const float2v f = { v[2 * i], v[2 * i + 1] };
			w[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(f, half2v));
		}
		*reinterpret_cast<uint4*>(dst) = make_uint4(w[0], w[1], w[2], w[3]);
	}

	__device__ __forceinline__ void store8(float* dst, const float (&v)[8])
	{
		reinterpret_cast<float4*>(dst)[0] = make_float4(v[0], v[1], v[2], v[3]);
		reinterpret_cast<float4*>(dst)[1] = make_float4(v[4], v[5], v[6], v[7]);
	}
	__device__ __forceinline__ void store8(uint16_t* dst, const float (&v)[8])
	{
		uint32_t w[4];
#pragma unroll
		for (int i = 0; i < 4; ++i)
		{
			w[i] = static_cast<uint32_t>(f32_to_f16_bits_litenn(v[2 * i])) |
			       (static_cast<uint32_t>(f32_to_f16_bits_litenn(v[2 * i + 1])) << 16);
		}
		*reinterpret_cast<uint4*>(dst) = make_uint4(w[0], w[1], w[2], w[3]);
	}

	// the four interleaved pairs a lane owns, rotated by the angles of its position
	__device__ __forceinline__ void rotate8(float (&v)[8], const float4& c, const float4& sn)
	{
		const float cs[4] = { c.x, c.y, c.z, c.w }, ss[4] = { sn.x, sn.y, sn.z, sn.w };
#pragma unroll
		for (int i = 0; i < 4; ++i)
		{
			float o0, o1;
			rotate(v[2 * i], v[2 * i + 1], cs[i], ss[i], o0, o1);
			v[2 * i] = o0;
			v[2 * i + 1] = o1;
		}
	}

} // namespace litenn_hip
#endif
