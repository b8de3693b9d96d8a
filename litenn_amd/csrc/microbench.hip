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

		// ---- exchange among the workgroups of one XCD -----------------------------------------
		// The card's 256 CUs sit in 8 XCDs of 32, each with an L2 of its own; what one CU stores is
		// visible to the other CUs of its XCD once it has reached that L2, without crossing the
		// fabric that joins the XCDs.  This kernel measures what a phase boundary inside one launch
		// costs when only the workgroups of one XCD have to meet: every workgroup reads the XCD it
		// runs on (XCC_ID), takes a slot among that XCD's workgroups from a ticket counter, and then
		// walks `phases` phases; in each it publishes one value and needs the values all slots of its
		// XCD published in the phase before.
		//   MODE 0: store, wait for the L2's acknowledgement, add one to the XCD's counter (an atomic
		//           executed in the L2); one lane polls the counter with an atomic add of zero, then
		//           the values are loaded past the CU's own L1 (sc0).
		//   MODE 1: every value carries the number of its phase; 32 lanes poll the 32 slots
		//           themselves with sc0 loads until each shows the phase wanted.
		//   MODE 2: like 1 with device-scope accesses (sc1 on loads and stores), the form an
		//           exchange across XCDs needs; here still among the workgroups of one XCD.
		//   MODE 3: one flag word per workgroup: the value is stored with an ordinary store to an address
		//           of its own per phase (never in any CU's L1), acknowledged by the L2, then the flag is
		//           stored; 32 lanes poll the 32 flags with atomic ORs of zero (executed in the L2) and
		//           then load the values with ordinary loads.
		//   MODE 4: like 3 with the flags polled by device-scope loads.
		// Every wait is bounded by `spin_limit` polls; a wait that runs out sets err[0] and the
		// workgroup walks the remaining phases without waiting, so the grid always drains.
		// Layout of `mem` (unsigned, zeroed by the host): [0,8) tickets per XCD, [16,24) arrival
		// counters per XCD, then from word 64 on, per XCD, 2 x 64 words: two parities of 32 slots of
		// {value, phase tag}.
		__device__ __forceinline__ unsigned mb_xcc_id()
		{
			// HW_REG_XCC_ID (register 20), bits [3:0]
			return __builtin_amdgcn_s_getreg(20 | (0 << 6) | (3 << 11));
		}

		__device__ __forceinline__ unsigned mb_l2_atomic_add(unsigned* p, unsigned v)
		{
			unsigned old;
			asm volatile("global_atomic_add %0, %1, %2, off sc0\n\ts_waitcnt vmcnt(0)" : "=v"(old) : "v"(p), "v"(v) : "memory");
			return old;
		}

		template <bool DEVICE_SCOPE>
		__device__ __forceinline__ unsigned long long mb_load_past_l1(const unsigned long long* p)
		{
			unsigned long long v;
			if constexpr (DEVICE_SCOPE)
			{
				asm volatile("global_load_dwordx2 %0, %1, off sc0 sc1\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory");
			}
			else
			{
				asm volatile("global_load_dwordx2 %0, %1, off sc0\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory");
			}
			return v;
		}

		template <bool DEVICE_SCOPE>
		__device__ __forceinline__ void mb_store_to_l2(unsigned long long* p, unsigned long long v)
		{
			if constexpr (DEVICE_SCOPE)
			{
				asm volatile("global_store_dwordx2 %0, %1, off sc0 sc1\n\ts_waitcnt vmcnt(0)" : : "v"(p), "v"(v) : "memory");
			}
			else
			{
				asm volatile("global_store_dwordx2 %0, %1, off\n\ts_waitcnt vmcnt(0)" : : "v"(p), "v"(v) : "memory");
			}
		}

		template <int MODE>
		__global__ __launch_bounds__(512) void mb_xcd_exchange_kernel(unsigned* __restrict__ mem, int phases, int spin_limit,
		                                                               int expected_per_xcd, int* __restrict__ err,
		                                                               unsigned* __restrict__ result,
		                                                               unsigned long long* __restrict__ stamps)
		{
			__shared__ unsigned s_value;
			__shared__ int s_slot;
			__shared__ volatile int s_dead;
			const int tid = threadIdx.x;
			const unsigned xcc = mb_xcc_id() & 7u;
			constexpr bool kDevice = MODE == 2;

			if (tid == 0)
			{
				s_slot = static_cast<int>(mb_l2_atomic_add(mem + xcc, 1u));
				s_dead = 0;
				s_value = 1u;
			}
			__syncthreads();
			const int slot = s_slot;
			if (slot >= 32)
			{
				// more workgroups on this XCD than the exchange has slots: not the placement measured
				if (tid == 0)
				{
					atomicExch(err, 2);
				}
				return;
			}
			if constexpr (MODE >= 3)
			{
				// mem: [64, 64 + 8 * 32) flags; fresh[phase][xcc][32] values (8 bytes each) behind them
				unsigned* flags = mem + 64 + xcc * 32;
				unsigned long long* fresh = reinterpret_cast<unsigned long long*>(mem + 2048);
				for (int p = 0; p < phases; ++p)
				{
					unsigned long long* row = fresh + (static_cast<size_t>(p) * 8 + xcc) * 32;
					if (tid == 0)
					{
						mb_store_to_l2<false>(row + slot, s_value); // waits for the L2's acknowledgement
						asm volatile("global_store_dword %0, %1, off" : : "v"(flags + slot), "v"(static_cast<unsigned>(p + 1)) : "memory");
						if (stamps && blockIdx.x == 0)
						{
							stamps[p] = __builtin_amdgcn_s_memrealtime();
						}
					}
					if (tid < 64)
					{
						unsigned mine = 0;
						if (tid < expected_per_xcd)
						{
							int spins = 0;
							for (;;)
							{
								unsigned seen;
								if (MODE == 3)
								{
									seen = mb_l2_atomic_add(flags + tid, 0u);
								}
								else
								{
									asm volatile("global_load_dword %0, %1, off sc0 sc1\n\ts_waitcnt vmcnt(0)" : "=v"(seen) : "v"(flags + tid) : "memory");
								}
								if (seen == static_cast<unsigned>(p + 1) || s_dead)
								{
									break;
								}
								if (++spins > spin_limit)
								{
									s_dead = 1;
									atomicExch(err, 1);
									break;
								}
							}
							unsigned long long got;
							asm volatile("global_load_dwordx2 %0, %1, off\n\ts_waitcnt vmcnt(0)" : "=v"(got) : "v"(row + tid) : "memory");
							mine = static_cast<unsigned>(got);
						}
						for (int o = 32; o; o >>= 1)
						{
							mine += __shfl_xor(mine, o);
						}
						if (tid == 0)
						{
							s_value = mine + 1u;
						}
					}
					__syncthreads();
				}
				if (tid == 0)
				{
					result[blockIdx.x * 2] = s_value;
					result[blockIdx.x * 2 + 1] = xcc * 64u + static_cast<unsigned>(slot);
				}
				return;
			}
			unsigned long long* values = reinterpret_cast<unsigned long long*>(mem + 64 + xcc * 128);
			unsigned* counter = mem + 16 + xcc;
			for (int p = 0; p < phases; ++p)
			{
				// publish this workgroup's value of phase p
				if (tid == 0)
				{
					const unsigned long long v = (static_cast<unsigned long long>(p + 1) << 32) | s_value;
					mb_store_to_l2<kDevice>(values + (p & 1) * 32 + slot, v);
					if (MODE == 0)
					{
						mb_l2_atomic_add(counter, 1u);
					}
					if (stamps && blockIdx.x == 0)
					{
						stamps[p] = __builtin_amdgcn_s_memrealtime();
					}
				}
				// the first wavefront collects the values of all slots of this XCD
				if (tid < 64)
				{
					if (MODE == 0)
					{
						if (tid == 0 && !s_dead)
						{
							const unsigned want = static_cast<unsigned>(expected_per_xcd) * static_cast<unsigned>(p + 1);
							int spins = 0;
							while (mb_l2_atomic_add(counter, 0u) < want)
							{
								if (++spins > spin_limit)
								{
									s_dead = 1;
									atomicExch(err, 1);
									break;
								}
							}
						}
						__builtin_amdgcn_wave_barrier();
					}
					unsigned mine = 0;
					if (tid < expected_per_xcd)
					{
						const unsigned long long* src = values + (p & 1) * 32 + tid;
						unsigned long long got = mb_load_past_l1<kDevice>(src);
						if (MODE != 0)
						{
							int spins = 0;
							while (static_cast<unsigned>(got >> 32) != static_cast<unsigned>(p + 1) && !s_dead)
							{
								if (++spins > spin_limit)
								{
									s_dead = 1;
									atomicExch(err, 1);
									break;
								}
								got = mb_load_past_l1<kDevice>(src);
							}
						}
						mine = static_cast<unsigned>(got);
					}
					// the next value: the sum of the XCD's values plus one
					for (int o = 32; o; o >>= 1)
					{
						mine += __shfl_xor(mine, o);
					}
					if (tid == 0)
					{
						s_value = mine + 1u;
					}
				}
				__syncthreads();
			}
			if (tid == 0)
			{
				result[blockIdx.x * 2] = s_value;
				result[blockIdx.x * 2 + 1] = xcc * 64u + static_cast<unsigned>(slot);
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

// The exchange among the workgroups of one XCD (see mb_xcd_exchange_kernel): `blocks` workgroups of
// 512 threads with 90 KB of LDS each (one per CU), `phases` phases, each wait bounded by
// `spin_limit` polls.  mode 0: counter in the L2; 1: values that carry their phase, polled past the
// L1; 2: the same with device-scope accesses; 3: flags polled by atomics in the L2, values by ordinary
// stores and loads at fresh addresses; 4: like 3 with the flags polled by device-scope loads.  `mem` is
// 8 KB (modes 3 and 4: 8 KB + phases * 2 KB) of device memory that this call clears;
// result (2 x blocks words) receives each workgroup's final value and 64 * XCD + slot; err (one int,
// cleared by this call) is 0 when no wait ran out, 1 when one did, 2 when an XCD received more than
// 32 workgroups; stamps (phases entries, or null) receives workgroup 0's 100 MHz clock per phase.
extern "C" int litenn_hip_mb_xcd_exchange(int mode, int blocks, int phases, int spin_limit, int expected_per_xcd, void* mem,
                                          void* err, void* result, void* stamps, void* stream)
{
	using namespace litenn_hip;
	if (!mem || !err || !result || blocks < 1 || blocks > 256 || phases < 1 || spin_limit < 1 || expected_per_xcd < 1 ||
	    expected_per_xcd > 32 || mode < 0 || mode > 4 || (mode >= 3 && phases > 4000))
	{
		return fail("launch the XCD exchange kernel", "null buffer or arguments out of range");
	}
	hipStream_t st = static_cast<hipStream_t>(stream);
	LITENN_HIP_TRY("launch the XCD exchange kernel",
	               hipMemsetAsync(mem, 0, 8192 + (mode >= 3 ? static_cast<size_t>(phases) * 2048 : 0), st));
	LITENN_HIP_TRY("launch the XCD exchange kernel", hipMemsetAsync(err, 0, sizeof(int), st));
	unsigned* m = static_cast<unsigned*>(mem);
	int* e = static_cast<int*>(err);
	unsigned* r = static_cast<unsigned*>(result);
	unsigned long long* t = static_cast<unsigned long long*>(stamps);
	const size_t lds = 90 * 1024;
	switch (mode)
	{
	case 0:
		allow_dynamic_lds(reinterpret_cast<const void*>(&mb_xcd_exchange_kernel<0>), 128 * 1024);
		mb_xcd_exchange_kernel<0><<<dim3(blocks), dim3(512), lds, st>>>(m, phases, spin_limit, expected_per_xcd, e, r, t);
		break;
	case 1:
		allow_dynamic_lds(reinterpret_cast<const void*>(&mb_xcd_exchange_kernel<1>), 128 * 1024);
		mb_xcd_exchange_kernel<1><<<dim3(blocks), dim3(512), lds, st>>>(m, phases, spin_limit, expected_per_xcd, e, r, t);
		break;
	case 2:
		allow_dynamic_lds(reinterpret_cast<const void*>(&mb_xcd_exchange_kernel<2>), 128 * 1024);
		mb_xcd_exchange_kernel<2><<<dim3(blocks), dim3(512), lds, st>>>(m, phases, spin_limit, expected_per_xcd, e, r, t);
		break;
	case 3:
		allow_dynamic_lds(reinterpret_cast<const void*>(&mb_xcd_exchange_kernel<3>), 128 * 1024);
		mb_xcd_exchange_kernel<3><<<dim3(blocks), dim3(512), lds, st>>>(m, phases, spin_limit, expected_per_xcd, e, r, t);
		break;
	default:
		allow_dynamic_lds(reinterpret_cast<const void*>(&mb_xcd_exchange_kernel<4>), 128 * 1024);
		mb_xcd_exchange_kernel<4><<<dim3(blocks), dim3(512), lds, st>>>(m, phases, spin_limit, expected_per_xcd, e, r, t);
		break;
	}
	LITENN_HIP_TRY("launch the XCD exchange kernel", hipGetLastError());
	return 0;
}
