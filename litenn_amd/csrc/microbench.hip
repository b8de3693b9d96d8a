// litenn-hip: measurement kernels of lib/liblitenn_hip_trace.so (not part of the product library).
// They give the streaming GEMV's time something to be read against on the same card, stream and
// graph: what a launch costs when the kernel does nothing, and how fast the same bytes arrive when
// the kernel does nothing but read them.
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
		template <int DEPTH>
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
					v[j] = src[i + static_cast<size_t>(j) * blockDim.x];
				}
#pragma unroll
				for (int j = 0; j < DEPTH; ++j)
				{
					acc ^= v[j].x ^ v[j].y ^ v[j].z ^ v[j].w;
				}
			}
			for (; i < end; i += blockDim.x)
			{
				const u32x4 v = src[i];
				acc ^= v.x ^ v.y ^ v.z ^ v.w;
			}
			if (acc == 0x9E3779B9u)
			{
				sink[0] = acc;
			}
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
// threads, `depth` (1, 2, 4 or 8) 128-bit loads in flight per lane.  `sink` is 4 bytes of device
// memory that is never written in practice.
extern "C" int litenn_hip_mb_read(const void* src, size_t bytes, int blocks, int depth, void* sink, void* stream)
{
	using namespace litenn_hip;
	if (!src || !sink || bytes % 16 != 0 || blocks < 1)
	{
		return fail("launch the read kernel", "null buffer, byte count not a multiple of 16, or no workgroups");
	}
	const u32x4* p = static_cast<const u32x4*>(src);
	unsigned* s = static_cast<unsigned*>(sink);
	hipStream_t st = static_cast<hipStream_t>(stream);
	switch (depth)
	{
	case 1: mb_read_kernel<1><<<dim3(blocks), dim3(512), 0, st>>>(p, bytes / 16, s); break;
	case 2: mb_read_kernel<2><<<dim3(blocks), dim3(512), 0, st>>>(p, bytes / 16, s); break;
	case 4: mb_read_kernel<4><<<dim3(blocks), dim3(512), 0, st>>>(p, bytes / 16, s); break;
	case 8: mb_read_kernel<8><<<dim3(blocks), dim3(512), 0, st>>>(p, bytes / 16, s); break;
	default: return fail("launch the read kernel", "depth must be 1, 2, 4 or 8");
	}
	LITENN_HIP_TRY("launch the read kernel", hipGetLastError());
	return 0;
}
