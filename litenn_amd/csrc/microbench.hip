// litenn-hip: measurement kernels of lib/liblitenn_hip_trace.so (not part of the product library).
// They give the streaming GEMV's time something to be read against on the same card, stream and
// graph: what a launch costs when the kernel does nothing, and how fast the same bytes arrive when
// the kernel does nothing but read them.  A third kernel issues the matrix-core GEMM's instruction
// mix (MFMAs, LDS fragment reads, plain arithmetic) from registers and LDS only, so that the issue
// rate of that mix can be read beside the GEMM's.
#include "common.hpp"

namespace litenn_hip
{
	typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

	namespace
	{
		__global__ __launch_bounds__(512) void mb_empty_kernel() {}

		// Every workgroup reads a contiguous share of the buffer with 128-bit loads, `depth` of them
		// in flight per lane, and folds what it read into one value that is stored only if it
		// equals a sentinel (so the loads cannot be dropped and nothing is written).
		// ONCE: the loads carry the non-temporal bit, like the weight rows of the streaming GEMV.
		template <bool ONCE>
		__device__ __forceinline__ u32x4 mb_load(const u32x4* p)
		{
			if constexpr (ONCE)
			{
				return __builtin_nontemporal_load(p);
			}
			else
			{
				return *p;
			}
		}

		template <int DEPTH, bool ONCE>
		__global__ __launch_bounds__(512) void mb_read_kernel(const u32x4* __restrict__ src, size_t pieces,
		                                                       unsigned* __restrict__ sink)
		{
			const size_t per_block = (pieces + gridDim.x - 1) / gridDim.x;
			const size_t begin = static_cast<size_t>(blockIdx.x) * per_block;
			const size_t end = begin + per_block < pieces ? begin + per_block : pieces;
			unsigned acc = 0;
			size_t i = begin + threadIdx.x;
			for (; i + static_cast<size_t>(DEPTH - 1) * blockDim.x < end; i += static_cast<size_t>(DEPTH) * blockDim.x)
			{
				u32x4 v[DEPTH];
#pragma unroll
				for (int j = 0; j < DEPTH; ++j)
				{
					v[j] = mb_load<ONCE>(src + i + static_cast<size_t>(j) * blockDim.x);
				}
#pragma unroll
				for (int j = 0; j < DEPTH; ++j)
				{
					acc ^= v[j].x ^ v[j].y ^ v[j].z ^ v[j].w;
				}
			}
			for (; i < end; i += blockDim.x)
			{
				const u32x4 v = mb_load<ONCE>(src + i);
				acc ^= v.x ^ v.y ^ v.z ^ v.w;
			}
			if (acc == 0x9E3779B9u)
			{
				sink[0] = acc;
			}
		}

		typedef _Float16 mb_half8 __attribute__((ext_vector_type(8)));
		typedef float mb_floatx4 __attribute__((ext_vector_type(4)));

		// One "group" is what the GEMM's inner loop does per activation fragment: two
		// v_mfma_f32_16x16x32_f16 (two weight groups), READS ds_read_b128 and VALU independent
		// f32 multiply-adds.  Eight groups are a step; every SYNC steps the workgroup meets at a
		// barrier (0 = never).  Each wavefront reports the cycles its walk took; with a closing
		// barrier the slowest wavefront's figure is the workgroup's.
		template <bool MFMA, int READS, int VALU, int SYNC>
		__global__ __launch_bounds__(512) void mb_mix_kernel(unsigned long long* __restrict__ cycles, int steps, float seed)
		{
			extern __shared__ __attribute__((aligned(16))) uint8_t mb_lds[];
			const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
			for (int i = threadIdx.x; i < 32768 / 4; i += blockDim.x)
			{
				reinterpret_cast<unsigned*>(mb_lds)[i] = i * 2654435761u;
			}
			__syncthreads();
			mb_floatx4 acc[16];
#pragma unroll
			for (int i = 0; i < 16; ++i)
			{
				acc[i] = mb_floatx4{ seed, 0.0f, 0.0f, 0.0f };
			}
			mb_half8 a0, a1;
#pragma unroll
			for (int i = 0; i < 8; ++i)
			{
				a0[i] = static_cast<_Float16>(seed + i);
				a1[i] = static_cast<_Float16>(seed - i);
			}
			u32x4 b[8];
#pragma unroll
			for (int i = 0; i < 8; ++i)
			{
				b[i] = u32x4{ static_cast<unsigned>(i), 1u, 2u, 3u };
			}
			float v0 = seed, v1 = seed * 2, v2 = seed * 3, v3 = seed * 5, v4 = seed * 7;
			const uint8_t* base = mb_lds + lane * 16 + (wave & 3) * 1024;
			__syncthreads();
			const unsigned long long t0 = __builtin_readcyclecounter();
			for (int it = 0; it < steps; ++it)
			{
#pragma unroll
				for (int t = 0; t < 8; ++t)
				{
					if (MFMA)
					{
						const mb_half8 bt = __builtin_bit_cast(mb_half8, b[t]);
						acc[2 * t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, bt, acc[2 * t], 0, 0, 0);
						acc[2 * t + 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, bt, acc[2 * t + 1], 0, 0, 0);
					}
#pragma unroll
					for (int r = 0; r < READS; ++r)
					{
						b[t] = *reinterpret_cast<const u32x4*>(base + ((t + r) & 7) * 4096);
					}
#pragma unroll
					for (int r = 0; r < VALU; ++r)
					{
						if (r % 5 == 0) v0 = __builtin_fmaf(v0, v1, v2);
						if (r % 5 == 1) v1 = __builtin_fmaf(v1, v2, v3);
						if (r % 5 == 2) v2 = __builtin_fmaf(v2, v3, v4);
						if (r % 5 == 3) v3 = __builtin_fmaf(v3, v4, v0);
						if (r % 5 == 4) v4 = __builtin_fmaf(v4, v0, v1);
					}
					if (MFMA)
					{
						__builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
						if (READS) __builtin_amdgcn_sched_group_barrier(0x100, READS, 0);
						if (VALU) __builtin_amdgcn_sched_group_barrier(0x002, VALU, 0);
					}
				}
				__builtin_amdgcn_sched_barrier(0);
				if (SYNC > 0 && (it % SYNC) == SYNC - 1)
				{
					__syncthreads();
				}
			}
			__syncthreads();
			const unsigned long long t1 = __builtin_readcyclecounter();
			float s = v0 + v1 + v2 + v3 + v4;
#pragma unroll
			for (int i = 0; i < 16; ++i)
			{
				s += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
			}
#pragma unroll
			for (int i = 0; i < 8; ++i)
			{
				s += static_cast<float>(b[i].x ^ b[i].y ^ b[i].z ^ b[i].w);
			}
			if (s == 1.2345f)
			{
				cycles[4096] = 1; // keeps the arithmetic alive; never taken in practice
			}
			if (lane == 0)
			{
				cycles[blockIdx.x * 8 + wave] = t1 - t0;
			}
		}

		template <bool MFMA, int READS, int VALU>
		int launch_mix(unsigned long long* cycles, int blocks, int threads, int steps, int sync, hipStream_t st)
		{
			// 96 KB of LDS keeps one workgroup per CU, like the GEMM's
			if (sync == 0)
			{
				allow_dynamic_lds(reinterpret_cast<const void*>(&mb_mix_kernel<MFMA, READS, VALU, 0>), 160 * 1024);
				mb_mix_kernel<MFMA, READS, VALU, 0><<<blocks, threads, 96 * 1024, st>>>(cycles, steps, 1.0f);
			}
			else
			{
				allow_dynamic_lds(reinterpret_cast<const void*>(&mb_mix_kernel<MFMA, READS, VALU, 4>), 160 * 1024);
				mb_mix_kernel<MFMA, READS, VALU, 4><<<blocks, threads, 96 * 1024, st>>>(cycles, steps, 1.0f);
			}
			return 0;
		}
	} // namespace
} // namespace litenn_hip

// One launch of the kernel that does nothing: `blocks` workgroups of `threads` threads (the GEMV
// launches 256 of 512) that each reserve `lds_bytes` of LDS.
extern "C" int litenn_hip_mb_empty(int blocks, int threads, size_t lds_bytes, void* stream)
{
	using namespace litenn_hip;
	if (blocks < 1 || threads < 64 || threads > 512 || lds_bytes > 160 * 1024)
	{
		return fail("launch the empty kernel", "geometry out of range");
	}
	allow_dynamic_lds(reinterpret_cast<const void*>(&mb_empty_kernel), 160 * 1024);
	mb_empty_kernel<<<dim3(blocks), dim3(threads), lds_bytes, static_cast<hipStream_t>(stream)>>>();
	LITENN_HIP_TRY("launch the empty kernel", hipGetLastError());
	return 0;
}

// One launch that reads `bytes` (a multiple of 16) at `src` once: `blocks` workgroups of 512
// threads, `depth` (1, 2, 4 or 8) 128-bit loads in flight per lane, with the non-temporal bit when
// `nontemporal` is non-zero.  `sink` is 4 bytes of device memory that is never written in practice.
extern "C" int litenn_hip_mb_read_policy(const void* src, size_t bytes, int blocks, int depth, int nontemporal,
                                         void* sink, void* stream)
{
	using namespace litenn_hip;
	if (!src || !sink || bytes % 16 != 0 || blocks < 1)
	{
		return fail("launch the read kernel", "null buffer, byte count not a multiple of 16, or no workgroups");
	}
	const u32x4* p = static_cast<const u32x4*>(src);
	unsigned* s = static_cast<unsigned*>(sink);
	hipStream_t st = static_cast<hipStream_t>(stream);
#define LITENN_MB_READ(D)                                                                                           \
	case D:                                                                                                          \
		if (nontemporal)                                                                                             \
		{                                                                                                            \
			mb_read_kernel<D, true><<<dim3(blocks), dim3(512), 0, st>>>(p, bytes / 16, s);                           \
		}                                                                                                            \
		else                                                                                                         \
		{                                                                                                            \
			mb_read_kernel<D, false><<<dim3(blocks), dim3(512), 0, st>>>(p, bytes / 16, s);                          \
		}                                                                                                            \
		break;
	switch (depth)
	{
		LITENN_MB_READ(1)
		LITENN_MB_READ(2)
		LITENN_MB_READ(4)
		LITENN_MB_READ(8)
	default: return fail("launch the read kernel", "depth must be 1, 2, 4 or 8");
	}
#undef LITENN_MB_READ
	LITENN_HIP_TRY("launch the read kernel", hipGetLastError());
	return 0;
}

extern "C" int litenn_hip_mb_read(const void* src, size_t bytes, int blocks, int depth, void* sink, void* stream)
{
	return litenn_hip_mb_read_policy(src, bytes, blocks, depth, 0, sink, stream);
}

// The GEMM's instruction mix without its memory traffic: `blocks` workgroups of `threads` (256 or
// 512: one or two wavefronts per SIMD) walk `steps` steps of eight groups of [2 MFMA if mfma,
// `reads` (0 or 1) ds_read_b128, `valu` (0, 3, 5 or 8) multiply-adds], with a workgroup barrier
// every four steps when `sync` is non-zero and one after the walk.  cycles[block * 8 + wavefront]
// receives each wavefront's cycle count (shader clock); `cycles` holds at least 4097 entries and
// blocks * 8 of them.
extern "C" int litenn_hip_mb_mix(int mfma, int reads, int valu, int sync, void* cycles, int blocks, int threads, int steps,
                                 void* stream)
{
	using namespace litenn_hip;
	if (!cycles || blocks < 1 || blocks > 512 || (threads != 256 && threads != 512) || steps < 1)
	{
		return fail("launch the instruction-mix kernel", "null buffer or geometry out of range");
	}
	unsigned long long* c = static_cast<unsigned long long*>(cycles);
	hipStream_t st = static_cast<hipStream_t>(stream);
	int rc = 1;
#define LITENN_MIX(M, R, V)                                                                                        \
	if ((mfma != 0) == M && reads == R && valu == V)                                                                \
	{                                                                                                               \
		rc = launch_mix<M, R, V>(c, blocks, threads, steps, sync, st);                                              \
	}
	LITENN_MIX(true, 0, 0)
	LITENN_MIX(true, 1, 0)
	LITENN_MIX(true, 0, 3)
	LITENN_MIX(true, 0, 5)
	LITENN_MIX(true, 0, 8)
	LITENN_MIX(true, 1, 3)
	LITENN_MIX(true, 1, 5)
	LITENN_MIX(true, 1, 8)
	LITENN_MIX(false, 1, 0)
	LITENN_MIX(false, 0, 5)
#undef LITENN_MIX
	if (rc != 0)
	{
		return fail("launch the instruction-mix kernel", "this combination of mfma, reads and valu is not built");
	}
	LITENN_HIP_TRY("launch the instruction-mix kernel", hipGetLastError());
	return 0;
}
