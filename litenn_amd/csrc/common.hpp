// Shared host/device helpers of the gfx950 backend.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <mutex>
#include <set>
#include <string>
#include <utility>

#include "../../include/litenn_hip.h"

namespace litenn_hip
{
	// integer tuning knob from the environment
	inline int env_int(const char* name, int fallback)
	{
		const char* v = getenv(name);
		return (v && *v) ? atoi(v) : fallback;
	}

	// Lets `kernel` be launched with up to `bytes` of dynamic LDS.  The attribute belongs to the
	// kernel's instance on one device, so it is set once per (device, kernel), for the device that
	// is current at the launch.
	inline void allow_dynamic_lds(const void* kernel, size_t bytes)
	{
		static std::mutex mutex;
		static std::set<std::pair<int, const void*>> done;
		int dev = 0;
		if (hipGetDevice(&dev) != hipSuccess)
		{
			return; // the launch that follows reports the error
		}
		std::lock_guard<std::mutex> lock(mutex);
		if (done.insert({ dev, kernel }).second)
		{
			(void)hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(bytes));
		}
	}

	// ---- error reporting: status code + thread-local message ---------------
	void set_error(const std::string& message);
	int fail(const char* action, const std::string& message);
	int fail_hip(const char* action, hipError_t err);

#define LITENN_HIP_TRY(action, expr)                                                                                   \
	do                                                                                                                 \
	{                                                                                                                  \
		const hipError_t litenn_err_ = (expr);                                                                         \
		if (litenn_err_ != hipSuccess)                                                                                 \
		{                                                                                                              \
			return ::litenn_hip::fail_hip(action, litenn_err_);                                                        \
		}                                                                                                              \
	} while (0)

	// Selects `dev` for the lifetime of the guard and restores the caller's device.
	class DeviceGuard
	{
	public:
		explicit DeviceGuard(int dev);
		~DeviceGuard();
		bool ok() const { return ok_; }
		hipError_t error() const { return err_; }

	private:
		int previous_ = -1;
		bool ok_ = false;
		hipError_t err_ = hipSuccess;
	};

	inline hipStream_t stream_of(const litenn_hip_exec* opts)
	{
		return opts ? static_cast<hipStream_t>(opts->stream) : nullptr;
	}

	// Applies the synchronize flag of the execution options and reports launch errors.
	int finish(const char* action, const litenn_hip_exec* opts);

	size_t dtype_size(int dtype);
	int block_elements(int fmt);
	int block_bytes(int fmt);
	// bytes of one row of k elements, 0 when k is not a whole number of blocks
	size_t row_bytes(int fmt, size_t k);

	constexpr int kWave = 64;
} // namespace litenn_hip

// ---- device-side helpers ---------------------------------------------------
#if defined(__HIPCC__)
namespace litenn_hip
{
	__device__ __forceinline__ float f16_bits_to_f32(uint32_t bits)
	{
		return __half2float(__ushort_as_half(static_cast<unsigned short>(bits & 0xffffu)));
	}

	// LiteNN's Float32 -> Float16 conversion (src/LiteNN/DType.h:63-110): nearest, ties UP in
	// magnitude (only the first dropped bit is examined), subnormals and overflow handled the
	// same way.  Not IEEE round-to-nearest-even, so the hardware converter is not used.
	__device__ __forceinline__ uint16_t f32_to_f16_bits_litenn(float value)
	{
		const uint32_t bits = __float_as_uint(value);
		// Values that land on normal halves (all of them, in practice) take the hardware converter:
		// round-to-nearest-even differs from the rule above only on an exact tie whose lower
		// neighbour is even, where one is added (a carry into the exponent, up to infinity, is
		// what the reference's sum does too).  One wavefront-uniform branch; any lane outside the
		// range sends the wavefront through the general form below.
		{
			const uint32_t e = (bits >> 23) & 0xffu;
			const bool plain = e >= 113u && e <= 142u;
			if (__builtin_amdgcn_ballot_w64(!plain) == 0)
			{
				const _Float16 h = static_cast<_Float16>(value);
				const uint32_t hb = __builtin_bit_cast(uint16_t, h);
				return static_cast<uint16_t>(hb + ((bits & 0x3fffu) == 0x1000u ? 1u : 0u));
			}
		}
		// branch-free: every range is computed and the result selected, so a wave converting a
		// handful of values does not serialise through divergent paths
		const uint32_t sign = (bits >> 16) & 0x8000u;
		const uint32_t mag = bits & 0x7fffffffu;
		const uint32_t exp_field = mag >> 23; // biased by 127
		// normal halves (exponent -14 .. 15): adding the first dropped bit carries into the
		// exponent exactly as the reference's explicit mantissa-overflow branch does, and
		// saturates at infinity (0x7c00)
		const uint32_t normal = ((mag + 0x1000u) >> 13) - 0x1c000u;
		// subnormal halves (exponent -24 .. -15): shift = -exponent - 1 in [14, 23]
		const uint32_t mantissa = (mag & 0x7fffffu) | 0x800000u;
		const uint32_t shift = 126u - exp_field;
		const uint32_t subnormal = ((mantissa >> ((shift - 1u) & 31u)) + 1u) >> 1;
		uint32_t half = normal;
		half = exp_field < 113u ? subnormal : half;
		half = exp_field < 103u ? 0u : half;         // below 2^-24 (and f32 zero/subnormals): zero
		half = mag >= 0x47800000u ? 0x7c00u : half; // exponent above 15, infinity
		half = mag > 0x7f800000u ? 0x7e00u : half;  // NaN
		return static_cast<uint16_t>(sign | half);
	}

	template <int Ctrl, int RowMask = 0xF, int BankMask = 0xF>
	__device__ __forceinline__ float dpp_f32(float v)
	{
		return __int_as_float(
		    __builtin_amdgcn_update_dpp(0, __float_as_int(v), Ctrl, RowMask, BankMask, false));
	}

	// Sum over the 64 lanes of a wavefront with DPP only (no LDS traffic); the total is
	// returned in every lane.
	__device__ __forceinline__ float wave_sum(float v)
	{
		v += dpp_f32<0xB1>(v);  // quad_perm [1,0,3,2]
		v += dpp_f32<0x4E>(v);  // quad_perm [2,3,0,1]
		v += dpp_f32<0x141>(v); // row_half_mirror
		v += dpp_f32<0x140>(v); // row_mirror: every lane holds its 16-lane row total
		v += dpp_f32<0x142, 0xA>(v); // row_bcast15 into rows 1 and 3
		v += dpp_f32<0x143, 0xC>(v); // row_bcast31 into rows 2 and 3: lane 63 holds the total
		return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
	}

	// Sum within aligned groups of 16 lanes; every lane of the group holds the result.
	__device__ __forceinline__ float row16_sum(float v)
	{
		v += dpp_f32<0xB1>(v);
		v += dpp_f32<0x4E>(v);
		v += dpp_f32<0x141>(v);
		v += dpp_f32<0x140>(v);
		return v;
	}

	__device__ __forceinline__ float wave_max(float v)
	{
		for (int off = 32; off > 0; off >>= 1)
		{
			v = fmaxf(v, __shfl_xor(v, off, 64));
		}
		return v;
	}
} // namespace litenn_hip
#endif
