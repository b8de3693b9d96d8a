// C ABI: error state, device management, memory, dtype conversion, and the quantised
// extension entry points.  Host-side validation lives here so that no kernel is ever
// launched on operands whose shapes it does not expect.
#include "common.hpp"

#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <vector>

namespace litenn_hip
{
	// launchers defined in gemv.hip / gemm.hip / glue.hip
	int launch_gemv(int fmt, const void* wq, size_t n, size_t k, const float* x, size_t m, float* y,
	                const float* residual, hipStream_t stream);
	size_t gemm_scratch_halves(size_t m, size_t k);
	bool launch_gemm(int fmt, const void* wq, size_t n, size_t k, const float* x, size_t m, float* y,
	                 const float* residual, void* scratch_halves, float* partial, size_t partial_floats,
	                 hipStream_t stream);
	bool launch_linear_group(int fmt, int count, const void* const* w, float* const* y, const size_t* n, size_t k,
	                         const float* x, const float* residual, const float* norm_w, double eps, bool silu_mul,
	                         float* scratch_x, float* scratch_gate, float* scratch_up, hipStream_t stream);
	void launch_dequantize(int fmt, const void* wq, size_t rows, size_t k, float* dst, hipStream_t stream);
	void launch_get_rows_q(int fmt, const void* table, size_t rows, size_t k, const int32_t* ids, size_t n_ids,
	                       float* out, int* err_flag, hipStream_t stream);
	void launch_rmsnorm(const float* x, const float* w, double eps, size_t m, size_t d, float* y, hipStream_t s);
	void launch_rope_table(float* cos_t, float* sin_t, size_t positions, size_t half, double base, double freq_scale,
	                       size_t pos_offset, hipStream_t s);
	void launch_rope(const float* x, float* y, size_t m, size_t n_heads, size_t head_dim, size_t rope_dims,
	                 const float* cos_t, const float* sin_t, hipStream_t s);
	void launch_kv_append(void* cache, int cache_dtype, size_t past_elems, const float* cur, size_t count,
	                      hipStream_t s);
	size_t attn_splits(size_t m, size_t max_len, size_t n_head);
	size_t attn_partial_floats(size_t m, size_t n_head, size_t head_dim, size_t splits);
	bool launch_attn_tile(const float* q, const void* kcache, const void* vcache, int cache_dtype, size_t m,
	                      const int* past_dev, size_t past_host, size_t n_head, size_t n_kv_head, size_t head_dim,
	                      float* out, hipStream_t s);
	void launch_attn_decode(const float* q, const void* kcache, const void* vcache, int cache_dtype, size_t m,
	                        const int* past_dev, size_t past_host, size_t n_head, size_t n_kv_head, size_t head_dim,
	                        float* out, size_t splits, float* partial, int* counters, hipStream_t s);
	bool attn_static_fits(size_t m, size_t n_head, size_t head_dim, size_t splits);
	size_t attn_static_scratch_bytes();
	hipError_t launch_attn_decode_static(const float* q, const void* kcache, const void* vcache, int cache_dtype,
	                                     size_t m, size_t past_host, size_t n_head, size_t n_kv_head, size_t head_dim,
	                                     float* out, size_t splits, hipStream_t s);
	void launch_attn_ext(const float* q, const void* kcache, const void* vcache, int cache_dtype, size_t m, size_t keys,
	                     size_t n_head, size_t n_kv_head, size_t head_dim, double scale, double max_bias,
	                     double logit_softcap, const float* mask, const float* sinks, bool causal, size_t key_offset,
	                     size_t query_offset, float* out, hipStream_t s);
	void launch_silu_mul(const float* gate, const float* up, float* y, size_t n, hipStream_t s);
	void launch_zero_ints(int* p, size_t n, hipStream_t s);
	void launch_argmax(const float* x, size_t rows, size_t n, int32_t* out, hipStream_t s);

	// ---- error state -----------------------------------------------------------------------
	static thread_local std::string g_error;

	void set_error(const std::string& message) { g_error = message; }

	int fail(const char* action, const std::string& message)
	{
		// same text shape as the reference's ThrowCUDAError (Device/CUDA.cpp:89-95)
		g_error = std::string(action) + " failed: " + message;
		return 1;
	}

	int fail_hip(const char* action, hipError_t err)
	{
		(void)hipGetLastError(); // clear the sticky launch error so the next call starts clean
		return fail(action, hipGetErrorString(err));
	}

	DeviceGuard::DeviceGuard(int dev)
	{
		int count = 0;
		err_ = hipGetDeviceCount(&count);
		if (err_ != hipSuccess)
		{
			return;
		}
		if (dev < 0 || dev >= count)
		{
			err_ = hipErrorInvalidDevice;
			return;
		}
		err_ = hipGetDevice(&previous_);
		if (err_ != hipSuccess)
		{
			return;
		}
		if (previous_ != dev)
		{
			err_ = hipSetDevice(dev);
			if (err_ != hipSuccess)
			{
				return;
			}
		}
		else
		{
			previous_ = -1; // nothing to restore
		}
		ok_ = true;
	}

	DeviceGuard::~DeviceGuard()
	{
		if (ok_ && previous_ >= 0)
		{
			(void)hipSetDevice(previous_);
		}
	}

	int finish(const char* action, const litenn_hip_exec* opts)
	{
		LITENN_HIP_TRY(action, hipGetLastError());
		if (!opts || opts->synchronize)
		{
			LITENN_HIP_TRY(action, hipStreamSynchronize(stream_of(opts)));
		}
		return 0;
	}

	// Device memory a call needs beyond its operands, in stream order: it comes from a memory pool of
	// the library's own (one per device, created on first use) through hipMallocFromPoolAsync, and
	// hipFreeAsync returns it once the work queued before has run, so such a call neither waits for the
	// stream nor stalls the device the way hipMalloc / hipFree do.  The pool keeps up to
	// kScratchPoolKeepBytes of what was returned for the next call and hands the rest back to the
	// device at the next synchronisation; the device's default pool, which other users of
	// hipMallocAsync in the process share, is left as it is.  A stream that is being captured gets no
	// allocation (the caller passes a workspace there).  Where the stream-ordered allocator is not
	// available the memory comes from hipMalloc and the call drains the stream before freeing it;
	// `blocking()` tells the caller which it was.
	constexpr unsigned long long kScratchPoolKeepBytes = 256ull << 20;
	class StreamScratch
	{
	public:
		explicit StreamScratch(hipStream_t s) : stream_(s) {}
		StreamScratch(const StreamScratch&) = delete;
		StreamScratch& operator=(const StreamScratch&) = delete;
		~StreamScratch()
		{
			if (!ptr_)
			{
				return;
			}
			if (async_)
			{
				(void)hipFreeAsync(ptr_, stream_);
			}
			else
			{
				(void)hipStreamSynchronize(stream_);
				(void)hipFree(ptr_);
			}
		}
		hipError_t allocate(size_t bytes)
		{
			static const bool use_pool = env_int("LITENN_HIP_STREAM_ORDERED_SCRATCH", 1) != 0;
			hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
			if (stream_ && hipStreamIsCapturing(stream_, &capture) == hipSuccess && capture != hipStreamCaptureStatusNone)
			{
				// neither an allocation node in the caller's graph nor a hipMalloc under capture
				return hipErrorStreamCaptureUnsupported;
			}
			(void)hipGetLastError();
			hipMemPool_t pool = use_pool ? scratch_pool() : nullptr;
			if (pool)
			{
				if (hipMallocFromPoolAsync(&ptr_, bytes ? bytes : 1, pool, stream_) == hipSuccess)
				{
					async_ = true;
					return hipSuccess;
				}
				(void)hipGetLastError();
				ptr_ = nullptr;
			}
			async_ = false;
			return hipMalloc(&ptr_, bytes ? bytes : 1);
		}
		void* get() const { return ptr_; }
		bool blocking() const { return ptr_ && !async_; }

	private:
		// the library's pool of the current device, created on first use; null where the device has no
		// stream-ordered allocator
		static hipMemPool_t scratch_pool()
		{
			static std::mutex mutex;
			static std::map<int, hipMemPool_t> pools; // a null entry: refused once, not tried again
			int dev = 0;
			if (hipGetDevice(&dev) != hipSuccess)
			{
				return nullptr;
			}
			std::lock_guard<std::mutex> lock(mutex);
			const auto found = pools.find(dev);
			if (found != pools.end())
			{
				return found->second;
			}
			int supported = 0;
			hipMemPool_t pool = nullptr;
			hipMemPoolProps props{};
			props.allocType = hipMemAllocationTypePinned;
			props.handleTypes = hipMemHandleTypeNone;
			props.location.type = hipMemLocationTypeDevice;
			props.location.id = dev;
			unsigned long long keep = kScratchPoolKeepBytes;
			if (hipDeviceGetAttribute(&supported, hipDeviceAttributeMemoryPoolsSupported, dev) != hipSuccess || !supported ||
			    hipMemPoolCreate(&pool, &props) != hipSuccess)
			{
				(void)hipGetLastError();
				pool = nullptr;
			}
			else if (hipMemPoolSetAttribute(pool, hipMemPoolAttrReleaseThreshold, &keep) != hipSuccess)
			{
				(void)hipGetLastError();
				(void)hipMemPoolDestroy(pool);
				pool = nullptr;
			}
			pools[dev] = pool;
			return pool;
		}
		void* ptr_ = nullptr;
		hipStream_t stream_ = nullptr;
		bool async_ = false;
	};

	// like finish(), for a call that holds a StreamScratch: a scratch that came from hipMalloc is freed
	// by draining the stream, so the launch error is collected first and the drain reported
	int finish_with(const StreamScratch& scratch, const char* action, const litenn_hip_exec* opts)
	{
		LITENN_HIP_TRY(action, hipGetLastError());
		if (scratch.blocking() || !opts || opts->synchronize)
		{
			LITENN_HIP_TRY(action, hipStreamSynchronize(stream_of(opts)));
		}
		return 0;
	}

	size_t dtype_size(int dtype)
	{
		switch (dtype)
		{
		case LITENN_F32:
		case LITENN_I32:
			return 4;
		case LITENN_F64:
		case LITENN_I64:
			return 8;
		case LITENN_F16:
		case LITENN_BF16:
			return 2;
		case LITENN_BOOL:
		case LITENN_F8E4M3:
		case LITENN_F8E5M2:
		case LITENN_I8:
		case LITENN_U8:
			return 1;
		default:
			return 0;
		}
	}

	int block_elements(int fmt)
	{
		switch (fmt)
		{
		case LITENN_FMT_Q4_0:
		case LITENN_FMT_Q4_1:
		case LITENN_FMT_Q5_0:
		case LITENN_FMT_Q5_1:
		case LITENN_FMT_Q8_0:
			return 32;
		case LITENN_FMT_Q2_K:
		case LITENN_FMT_Q3_K:
		case LITENN_FMT_Q4_K:
		case LITENN_FMT_Q5_K:
		case LITENN_FMT_Q6_K:
			return 256;
		case LITENN_FMT_F16:
		case LITENN_FMT_F32:
			return 1;
		default:
			return 0;
		}
	}

	int block_bytes(int fmt)
	{
		switch (fmt)
		{
		case LITENN_FMT_Q4_0:
			return 18;
		case LITENN_FMT_Q4_1:
			return 20;
		case LITENN_FMT_Q5_0:
			return 22;
		case LITENN_FMT_Q5_1:
			return 24;
		case LITENN_FMT_Q8_0:
			return 34;
		case LITENN_FMT_Q2_K:
			return 84;
		case LITENN_FMT_Q3_K:
			return 110;
		case LITENN_FMT_Q4_K:
			return 144;
		case LITENN_FMT_Q5_K:
			return 176;
		case LITENN_FMT_Q6_K:
			return 210;
		case LITENN_FMT_F16:
			return 2;
		case LITENN_FMT_F32:
			return 4;
		default:
			return 0;
		}
	}

	size_t row_bytes(int fmt, size_t k)
	{
		const int be = block_elements(fmt);
		if (be == 0 || k % static_cast<size_t>(be) != 0)
		{
			return 0;
		}
		return k / static_cast<size_t>(be) * static_cast<size_t>(block_bytes(fmt));
	}

	// ---- dtype conversion --------------------------------------------------------------------
	namespace
	{
		struct F16 { uint16_t bits; };
		struct BF16 { uint16_t bits; };
		// Float8E4M3 (4 exponent bits, bias 7) and Float8E5M2 (5, bias 15), both with the top
		// exponent reserved for infinity and NaN as LiteNN defines them (DType.h:290-344)
		template <int EBITS, int MBITS, int BIAS>
		struct F8 { uint8_t bits; };
		using F8E4M3 = F8<4, 3, 7>;
		using F8E5M2 = F8<5, 2, 15>;

		// Float8BitsToFloat32 (DType.h:203-229): every value is exact in Float32
		template <int EBITS, int MBITS, int BIAS>
		__device__ __forceinline__ float f8_bits_to_f32(uint8_t bits)
		{
			const uint32_t exp_mask = (1u << EBITS) - 1u;
			const uint32_t e = (bits >> MBITS) & exp_mask, mant = bits & ((1u << MBITS) - 1u);
			const float sign = (bits & 0x80u) ? -1.0f : 1.0f;
			if (e == 0)
			{
				return sign * ldexpf(static_cast<float>(mant), 1 - BIAS - MBITS); // zero keeps its sign
			}
			if (e == exp_mask)
			{
				return mant == 0 ? sign * INFINITY : __uint_as_float(0x7fc00000u);
			}
			return sign * ldexpf(static_cast<float>((1u << MBITS) | mant), static_cast<int>(e) - BIAS - MBITS);
		}

		// Float32ToFloat8Bits (DType.h:148-201), step for step: the magnitude is brought into [1, 2)
		// (exact), the mantissa is (uint32)(x * 2^MBITS + 0.5f) with the Float32 addition's own
		// rounding, a mantissa that rounds up to 2^MBITS carries into the exponent, the top exponent is
		// infinity (NaN goes there too, with its sign bit), stored exponents <= 0 are subnormal with the
		// mantissa clamped to its field.
		template <int EBITS, int MBITS, int BIAS>
		__device__ __forceinline__ uint8_t f32_to_f8_bits(float value)
		{
			const uint32_t raw = __float_as_uint(value);
			const uint32_t sign = (raw >> 24) & 0x80u;
			const uint32_t mag = raw & 0x7fffffffu;
			const uint32_t max_exp = (1u << EBITS) - 1u;
			if (mag == 0)
			{
				return static_cast<uint8_t>(sign);
			}
			if (mag >= 0x7f800000u)
			{
				return static_cast<uint8_t>(sign | (max_exp << MBITS));
			}
			if (mag < 0x00800000u)
			{
				return static_cast<uint8_t>(sign); // a Float32 subnormal is far below half the smallest step
			}
			const int exponent = static_cast<int>(mag >> 23) - 127;
			const float m = __uint_as_float((mag & 0x007fffffu) | 0x3f800000u); // in [1, 2)
			const int stored = exponent + BIAS;
			const float scale = static_cast<float>(1u << MBITS);
			if (stored >= static_cast<int>(max_exp))
			{
				return static_cast<uint8_t>(sign | (max_exp << MBITS));
			}
			if (stored <= 0)
			{
				const float sub = ldexpf(m, stored - 1); // exact here: the product below is compared with 1/2
				const uint32_t q = static_cast<uint32_t>(__fadd_rn(__fmul_rn(sub, scale), 0.5f));
				return static_cast<uint8_t>(sign | min(q, (1u << MBITS) - 1u));
			}
			uint32_t q = static_cast<uint32_t>(__fadd_rn(__fmul_rn(__fsub_rn(m, 1.0f), scale), 0.5f));
			uint32_t e = static_cast<uint32_t>(stored);
			if (q == (1u << MBITS))
			{
				q = 0;
				e = min(e + 1u, max_exp);
			}
			return static_cast<uint8_t>(sign | (e << MBITS) | q);
		}

		template <typename T>
		__device__ __forceinline__ double load_as_double(const T* p, size_t i) { return static_cast<double>(p[i]); }
		template <>
		__device__ __forceinline__ double load_as_double<F16>(const F16* p, size_t i)
		{
			return static_cast<double>(f16_bits_to_f32(p[i].bits));
		}
		template <>
		__device__ __forceinline__ double load_as_double<BF16>(const BF16* p, size_t i)
		{
			return static_cast<double>(__uint_as_float(static_cast<uint32_t>(p[i].bits) << 16));
		}

		template <>
		__device__ __forceinline__ double load_as_double<F8E4M3>(const F8E4M3* p, size_t i)
		{
			return static_cast<double>(f8_bits_to_f32<4, 3, 7>(p[i].bits));
		}
		template <>
		__device__ __forceinline__ double load_as_double<F8E5M2>(const F8E5M2* p, size_t i)
		{
			return static_cast<double>(f8_bits_to_f32<5, 2, 15>(p[i].bits));
		}

		template <typename S>
		struct IsInt { static constexpr bool value = false; };
		template <> struct IsInt<int32_t> { static constexpr bool value = true; };
		template <> struct IsInt<int64_t> { static constexpr bool value = true; };
		template <> struct IsInt<int8_t> { static constexpr bool value = true; };
		template <> struct IsInt<uint8_t> { static constexpr bool value = true; };
		template <> struct IsInt<bool> { static constexpr bool value = true; };

		// The float a Float16 / BFloat16 constructor receives: integers convert to float in one
		// rounding (a detour through double would round an Int64 beyond 2^53 twice).
		template <typename S>
		__device__ __forceinline__ float load_as_float(const S* p, size_t i)
		{
			if constexpr (IsInt<S>::value)
			{
				return static_cast<float>(p[i]);
			}
			else
			{
				return static_cast<float>(load_as_double<S>(p, i));
			}
		}

		// static_cast<Dst>(src) for every pair, with LiteNN's own Float16 / BFloat16 constructors
		// (via float; DType.h:63-110, :136-141).
		template <typename S, typename D>
		__device__ __forceinline__ void convert_one(const S* src, D* dst, size_t i)
		{
			if constexpr (IsInt<S>::value)
			{
				dst[i] = static_cast<D>(src[i]);
			}
			else
			{
				dst[i] = static_cast<D>(load_as_double<S>(src, i));
			}
		}
		template <typename S>
		__device__ __forceinline__ void convert_one(const S* src, F16* dst, size_t i)
		{
			dst[i].bits = f32_to_f16_bits_litenn(load_as_float<S>(src, i));
		}
		template <typename S>
		__device__ __forceinline__ void convert_one(const S* src, BF16* dst, size_t i)
		{
			const uint32_t bits = __float_as_uint(load_as_float<S>(src, i));
			const uint32_t lsb = (bits >> 16) & 1u;
			dst[i].bits = static_cast<uint16_t>((bits + 0x7fffu + lsb) >> 16);
		}

		template <typename S, int EBITS, int MBITS, int BIAS>
		__device__ __forceinline__ void convert_one(const S* src, F8<EBITS, MBITS, BIAS>* dst, size_t i)
		{
			dst[i].bits = f32_to_f8_bits<EBITS, MBITS, BIAS>(load_as_float<S>(src, i));
		}

		template <typename S, typename D>
		__global__ void convert_kernel(const S* __restrict__ src, D* __restrict__ dst, size_t n)
		{
			const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
			if (i < n)
			{
				convert_one(src, dst, i);
			}
		}

		template <typename S>
		bool convert_from(const void* src, int dst_dtype, void* dst, size_t n, hipStream_t s)
		{
			const dim3 grid((n + 255) / 256), block(256);
			const S* sp = static_cast<const S*>(src);
			switch (dst_dtype)
			{
			case LITENN_F32: convert_kernel<S, float><<<grid, block, 0, s>>>(sp, static_cast<float*>(dst), n); return true;
			case LITENN_F64: convert_kernel<S, double><<<grid, block, 0, s>>>(sp, static_cast<double*>(dst), n); return true;
			case LITENN_I32: convert_kernel<S, int32_t><<<grid, block, 0, s>>>(sp, static_cast<int32_t*>(dst), n); return true;
			case LITENN_I64: convert_kernel<S, int64_t><<<grid, block, 0, s>>>(sp, static_cast<int64_t*>(dst), n); return true;
			case LITENN_BOOL: convert_kernel<S, bool><<<grid, block, 0, s>>>(sp, static_cast<bool*>(dst), n); return true;
			case LITENN_F16: convert_kernel<S, F16><<<grid, block, 0, s>>>(sp, static_cast<F16*>(dst), n); return true;
			case LITENN_BF16: convert_kernel<S, BF16><<<grid, block, 0, s>>>(sp, static_cast<BF16*>(dst), n); return true;
			case LITENN_F8E4M3: convert_kernel<S, F8E4M3><<<grid, block, 0, s>>>(sp, static_cast<F8E4M3*>(dst), n); return true;
			case LITENN_F8E5M2: convert_kernel<S, F8E5M2><<<grid, block, 0, s>>>(sp, static_cast<F8E5M2*>(dst), n); return true;
			case LITENN_I8: convert_kernel<S, int8_t><<<grid, block, 0, s>>>(sp, static_cast<int8_t*>(dst), n); return true;
			case LITENN_U8: convert_kernel<S, uint8_t><<<grid, block, 0, s>>>(sp, static_cast<uint8_t*>(dst), n); return true;
			default: return false;
			}
		}
	} // namespace

	// device -> device conversion; false when a dtype is not executed by this backend (fp8)
	bool launch_convert(int src_dtype, const void* src, size_t n, int dst_dtype, void* dst, hipStream_t s)
	{
		if (n == 0)
		{
			return true;
		}
		switch (src_dtype)
		{
		case LITENN_F32: return convert_from<float>(src, dst_dtype, dst, n, s);
		case LITENN_F64: return convert_from<double>(src, dst_dtype, dst, n, s);
		case LITENN_I32: return convert_from<int32_t>(src, dst_dtype, dst, n, s);
		case LITENN_I64: return convert_from<int64_t>(src, dst_dtype, dst, n, s);
		case LITENN_BOOL: return convert_from<bool>(src, dst_dtype, dst, n, s);
		case LITENN_F16: return convert_from<F16>(src, dst_dtype, dst, n, s);
		case LITENN_BF16: return convert_from<BF16>(src, dst_dtype, dst, n, s);
		case LITENN_F8E4M3: return convert_from<F8E4M3>(src, dst_dtype, dst, n, s);
		case LITENN_F8E5M2: return convert_from<F8E5M2>(src, dst_dtype, dst, n, s);
		case LITENN_I8: return convert_from<int8_t>(src, dst_dtype, dst, n, s);
		case LITENN_U8: return convert_from<uint8_t>(src, dst_dtype, dst, n, s);
		default: return false;
		}
	}
} // namespace litenn_hip

using namespace litenn_hip;

#define GUARD(action, dev)                                                                                             \
	DeviceGuard guard_(dev);                                                                                           \
	if (!guard_.ok())                                                                                                  \
	{                                                                                                                  \
		return fail_hip(action, guard_.error());                                                                       \
	}

extern "C" const char* litenn_hip_last_error(void)
{
	return g_error.c_str();
}

extern "C" int litenn_hip_device_count(void)
{
	int count = 0;
	if (hipGetDeviceCount(&count) != hipSuccess)
	{
		(void)hipGetLastError();
		return 0;
	}
	return count;
}

extern "C" int litenn_hip_device_info(int dev, char* buf, size_t buf_len)
{
	GUARD("HIP device query", dev);
	hipDeviceProp_t prop;
	LITENN_HIP_TRY("HIP device query", hipGetDeviceProperties(&prop, dev));
	if (buf && buf_len)
	{
		snprintf(buf, buf_len, "HIP device %d: %s (%s, %d CUs, %.1f GiB)", dev, prop.name, prop.gcnArchName,
		         prop.multiProcessorCount, static_cast<double>(prop.totalGlobalMem) / (1024.0 * 1024.0 * 1024.0));
	}
	return 0;
}

extern "C" int litenn_hip_alloc(int dev, int dtype, size_t n, void** out)
{
	const size_t es = dtype_size(dtype);
	if (!out || es == 0)
	{
		return fail("HIP allocate", "bad dtype or null output pointer");
	}
	if (n > SIZE_MAX / es)
	{
		return fail("HIP allocate", "element count overflows the byte size");
	}
	GUARD("HIP allocate", dev);
	*out = nullptr;
	// zero-element tensors still get a distinct, freeable pointer
	LITENN_HIP_TRY("HIP allocate", hipMalloc(out, n * es ? n * es : 1));
	return 0;
}

extern "C" int litenn_hip_free(int dev, void* ptr, int dtype, size_t n)
{
	(void)dtype;
	(void)n;
	if (!ptr)
	{
		return 0;
	}
	GUARD("HIP deallocate", dev);
	LITENN_HIP_TRY("HIP deallocate", hipFree(ptr));
	return 0;
}

extern "C" int litenn_hip_zero(int dev, void* ptr, int dtype, size_t n)
{
	const size_t es = dtype_size(dtype);
	if (es == 0)
	{
		return fail("HIP zero fill", "bad dtype");
	}
	if (n == 0)
	{
		return 0;
	}
	if (!ptr)
	{
		return fail("HIP zero fill", "null operand");
	}
	GUARD("HIP zero fill", dev);
	LITENN_HIP_TRY("HIP zero fill", hipMemset(ptr, 0, n * es));
	return 0;
}

extern "C" int litenn_hip_convert(int dev, int src_dtype, const void* src, size_t n, int dst_dtype, void* dst,
                                  const litenn_hip_exec* opts)
{
	if (dtype_size(src_dtype) == 0 || dtype_size(dst_dtype) == 0)
	{
		return fail("HIP convert", "bad dtype");
	}
	if (n && (!src || !dst))
	{
		return fail("HIP convert", "null operand");
	}
	GUARD("HIP convert", dev);
	if (src_dtype == dst_dtype)
	{
		if (n)
		{
			LITENN_HIP_TRY("HIP convert", hipMemcpyAsync(dst, src, n * dtype_size(src_dtype), hipMemcpyDeviceToDevice,
			                                             stream_of(opts)));
		}
	}
	else if (!launch_convert(src_dtype, src, n, dst_dtype, dst, stream_of(opts)))
	{
		return fail("HIP convert", "dtype pair is not supported on the device");
	}
	return finish("HIP convert", opts);
}

extern "C" int litenn_hip_copy_to_host(int dev, int src_dtype, const void* src, size_t n, int dst_dtype, void* dst,
                                       const litenn_hip_exec* opts)
{
	if (dtype_size(src_dtype) == 0 || dtype_size(dst_dtype) == 0)
	{
		return fail("HIP copy to host", "bad dtype");
	}
	if (n == 0)
	{
		return 0;
	}
	if (!src || !dst)
	{
		return fail("HIP copy to host", "null operand");
	}
	GUARD("HIP copy to host", dev);
	hipStream_t s = stream_of(opts);
	if (src_dtype == dst_dtype)
	{
		LITENN_HIP_TRY("HIP copy to host", hipMemcpyAsync(dst, src, n * dtype_size(src_dtype), hipMemcpyDeviceToHost, s));
		return finish("HIP copy to host", opts);
	}
	// convert on the device, then one copy; the staging buffer forces a synchronous finish
	void* tmp = nullptr;
	LITENN_HIP_TRY("HIP copy to host", hipMalloc(&tmp, n * dtype_size(dst_dtype)));
	int rc = 0;
	if (!launch_convert(src_dtype, src, n, dst_dtype, tmp, s))
	{
		rc = fail("HIP copy to host", "dtype pair is not supported on the device");
	}
	else
	{
		const hipError_t e = hipMemcpyAsync(dst, tmp, n * dtype_size(dst_dtype), hipMemcpyDeviceToHost, s);
		const hipError_t e2 = hipStreamSynchronize(s);
		if (e != hipSuccess || e2 != hipSuccess)
		{
			rc = fail_hip("HIP copy to host", e != hipSuccess ? e : e2);
		}
	}
	(void)hipFree(tmp);
	return rc;
}

extern "C" int litenn_hip_copy_from_host(int dev, int dst_dtype, void* dst, int src_dtype, const void* src, size_t n,
                                         const litenn_hip_exec* opts)
{
	if (dtype_size(src_dtype) == 0 || dtype_size(dst_dtype) == 0)
	{
		return fail("HIP copy from host", "bad dtype");
	}
	if (n == 0)
	{
		return 0;
	}
	if (!src || !dst)
	{
		return fail("HIP copy from host", "null operand");
	}
	GUARD("HIP copy from host", dev);
	hipStream_t s = stream_of(opts);
	if (src_dtype == dst_dtype)
	{
		LITENN_HIP_TRY("HIP copy from host",
		               hipMemcpyAsync(dst, src, n * dtype_size(src_dtype), hipMemcpyHostToDevice, s));
		return finish("HIP copy from host", opts);
	}
	void* tmp = nullptr;
	LITENN_HIP_TRY("HIP copy from host", hipMalloc(&tmp, n * dtype_size(src_dtype)));
	int rc = 0;
	const hipError_t e = hipMemcpyAsync(tmp, src, n * dtype_size(src_dtype), hipMemcpyHostToDevice, s);
	if (e != hipSuccess)
	{
		rc = fail_hip("HIP copy from host", e);
	}
	else if (!launch_convert(src_dtype, tmp, n, dst_dtype, dst, s))
	{
		rc = fail("HIP copy from host", "dtype pair is not supported on the device");
	}
	const hipError_t e2 = hipStreamSynchronize(s);
	if (rc == 0 && e2 != hipSuccess)
	{
		rc = fail_hip("HIP copy from host", e2);
	}
	(void)hipFree(tmp);
	return rc;
}

// ---- group 2: quantised extensions ------------------------------------------------------------

static bool is_weight_format(int fmt)
{
	return block_elements(fmt) != 0;
}

// From this many activation rows on a quantised matmul goes to the matrix cores: one padded 16-row
// tile costs about as much as three single-row GEMVs (Q4_K 14336 x 4096: 14.6 us against 8.2 each).
static constexpr size_t kMatrixCoreMinRows = 4;

extern "C" size_t litenn_hip_mul_mat_q_workspace_bytes(size_t m, size_t k)
{
	return m >= kMatrixCoreMinRows ? 2 * gemm_scratch_halves(m, k) : 0;
}

extern "C" int litenn_hip_mul_mat_q(int dev, int fmt, const void* wq, size_t n, size_t k, const void* x, int x_dtype,
                                    size_t m, void* y, const void* residual, unsigned flags,
                                    const litenn_hip_exec* opts)
{
	return litenn_hip_mul_mat_q_ws(dev, fmt, wq, n, k, x, x_dtype, m, y, residual, flags, nullptr, 0, opts);
}

extern "C" int litenn_hip_mul_mat_q_ws(int dev, int fmt, const void* wq, size_t n, size_t k, const void* x,
                                       int x_dtype, size_t m, void* y, const void* residual, unsigned flags,
                                       void* workspace, size_t workspace_bytes, const litenn_hip_exec* opts)
{
	const char* action = "HIP quantized matmul";
	if (!is_weight_format(fmt))
	{
		return fail(action, "unsupported block format");
	}
	if (x_dtype != LITENN_F32 && x_dtype != LITENN_F16 && x_dtype != LITENN_BF16)
	{
		return fail(action, "activations must be Float32, Float16 or BFloat16");
	}
	if (row_bytes(fmt, k) == 0)
	{
		return fail(action, "row width is incompatible with the block size of the format");
	}
	if (n > 0x7fffffffu || k > 0x7fffffffu || m > 0x7fffffffu)
	{
		return fail(action, "dimension exceeds 2^31-1");
	}
	if (n == 0 || m == 0)
	{
		return 0;
	}
	if (k == 0)
	{
		return fail(action, "inner dimension must be positive");
	}
	if (!wq || !x || !y)
	{
		return fail(action, "null operand");
	}
	GUARD(action, dev);
	hipStream_t s = stream_of(opts);
	// 16-bit activations are widened (exactly) into a Float32 copy that this call owns (stream-ordered
	// scratch: returned to the pool once the work queued here has run)
	StreamScratch widened(s);
	const float* xf = static_cast<const float*>(x);
	if (x_dtype != LITENN_F32)
	{
		LITENN_HIP_TRY(action, widened.allocate(sizeof(float) * m * k));
		if (!launch_convert(x_dtype, x, m * k, LITENN_F32, widened.get(), s))
		{
			return fail(action, "activation dtype is not supported on the device");
		}
		xf = static_cast<const float*>(widened.get());
	}
	float* yf = static_cast<float*>(y);
	const float* rf = static_cast<const float*>(residual);
	const bool quant = fmt != LITENN_FMT_F16 && fmt != LITENN_FMT_F32;
	if (m >= kMatrixCoreMinRows && !(flags & LITENN_HIP_MATMUL_PRECISE) && quant && k % 256 == 0)
	{
		// the matrix-core path rounds the activations to fp16 into a workspace
		const size_t need = 2 * gemm_scratch_halves(m, k);
		// room for more m x n products behind it lets K be walked in parts
		const size_t need16 = (need + 15) & ~size_t{ 15 };
		// (three more products, so that K can be walked in four ranges, while a product is at most 16 MB:
		// larger products belong to launches that fill the card without ranges)
		const bool small_product = m * n <= (size_t{ 4 } << 20);
		const size_t with_partial = need16 + sizeof(float) * m * n * (small_product ? 3 : 1);
		if (workspace)
		{
			if (workspace_bytes < need)
			{
				return fail(action, "workspace is smaller than litenn_hip_mul_mat_q_workspace_bytes(m, k)");
			}
			const bool roomy = workspace_bytes >= need16 + sizeof(float) * m * n;
			float* partial = roomy ? reinterpret_cast<float*>(static_cast<char*>(workspace) + need16) : nullptr;
			const size_t partial_floats = roomy ? (workspace_bytes - need16) / sizeof(float) : 0;
			if (!launch_gemm(fmt, wq, n, k, xf, m, yf, rf, workspace, partial, partial_floats, s))
			{
				launch_gemv(fmt, wq, n, k, xf, m, yf, rf, s);
			}
			return finish_with(widened, action, opts);
		}
		// none given: this call takes one in stream order and returns it the same way
		StreamScratch scratch(s);
		const bool splits = (k >= 8192 && m >= 128) || small_product;
		LITENN_HIP_TRY(action, scratch.allocate(splits ? with_partial : need));
		float* partial = splits ? reinterpret_cast<float*>(static_cast<char*>(scratch.get()) + need16) : nullptr;
		if (!launch_gemm(fmt, wq, n, k, xf, m, yf, rf, scratch.get(), partial,
		                 splits ? (with_partial - need16) / sizeof(float) : 0, s))
		{
			launch_gemv(fmt, wq, n, k, xf, m, yf, rf, s);
		}
		if (scratch.blocking() || widened.blocking())
		{
			const hipError_t launched = hipGetLastError();
			const hipError_t drained = hipStreamSynchronize(s);
			if (launched != hipSuccess || drained != hipSuccess)
			{
				return fail_hip(action, launched != hipSuccess ? launched : drained);
			}
			return 0;
		}
		return finish(action, opts);
	}
	launch_gemv(fmt, wq, n, k, xf, m, yf, rf, s);
	return finish_with(widened, action, opts);
}

extern "C" int litenn_hip_linear_group(int dev, int fmt, size_t count, const void* const* wq, const size_t* n, size_t k,
                                       const void* x, void* const* y, const void* residual, const void* norm_w,
                                       double eps, unsigned flags, const litenn_hip_exec* opts)
{
	const char* action = "HIP linear group";
	const bool silu = (flags & LITENN_HIP_GROUP_SILU_MUL) != 0;
	if (!is_weight_format(fmt))
	{
		return fail(action, "unsupported block format");
	}
	if (count < 1 || count > 3 || !wq || !n || !y || !x)
	{
		return fail(action, "a group holds one to three matrices");
	}
	if (row_bytes(fmt, k) == 0 || k == 0)
	{
		return fail(action, "row width is incompatible with the block size of the format");
	}
	if (silu && (count != 2 || n[0] != n[1]))
	{
		return fail(action, "SwiGLU needs exactly two matrices of equal height");
	}
	if (residual && count != 1)
	{
		return fail(action, "a residual goes with a single matrix");
	}
	if (norm_w && !(eps > 0.0))
	{
		return fail(action, "RMSNorm epsilon must be greater than zero");
	}
	float* ys[3] = { nullptr, nullptr, nullptr };
	for (size_t i = 0; i < count; ++i)
	{
		if (n[i] == 0 || n[i] > 0x3fffffffu || k > 0x7fffffffu || !wq[i] || (!y[i] && !(silu && i == 1)))
		{
			return fail(action, "bad matrix in the group");
		}
		ys[i] = static_cast<float*>(y[i]);
	}
	GUARD(action, dev);
	hipStream_t s = stream_of(opts);
	// the single-launch form needs no memory of its own; the composed form takes its scratch from the
	// library's pool and returns it in stream order
	StreamScratch scratch_mem(s);
	if (!launch_linear_group(fmt, static_cast<int>(count), wq, ys, n, k, static_cast<const float*>(x),
	                         static_cast<const float*>(residual), static_cast<const float*>(norm_w), eps, silu, nullptr,
	                         nullptr, nullptr, s))
	{
		const size_t scratch_floats = k + 2 * n[0];
		LITENN_HIP_TRY(action, scratch_mem.allocate(sizeof(float) * scratch_floats));
		float* scratch = static_cast<float*>(scratch_mem.get());
		launch_linear_group(fmt, static_cast<int>(count), wq, ys, n, k, static_cast<const float*>(x),
		                    static_cast<const float*>(residual), static_cast<const float*>(norm_w), eps, silu, scratch,
		                    scratch + k, scratch + k + n[0], s);
	}
	return finish_with(scratch_mem, action, opts);
}

extern "C" int litenn_hip_dequantize(int dev, int fmt, const void* wq, size_t rows, size_t k, void* dst,
                                     const litenn_hip_exec* opts)
{
	const char* action = "HIP dequantize";
	if (!is_weight_format(fmt) || row_bytes(fmt, k) == 0)
	{
		return fail(action, "unsupported block format or row width");
	}
	if (rows == 0 || k == 0)
	{
		return 0;
	}
	if (k > 0x7fffffffu || rows > 0x7fffffffu)
	{
		return fail(action, "dimension exceeds 2^31-1");
	}
	if (!wq || !dst)
	{
		return fail(action, "null operand");
	}
	GUARD(action, dev);
	launch_dequantize(fmt, wq, rows, k, static_cast<float*>(dst), stream_of(opts));
	return finish(action, opts);
}

extern "C" int litenn_hip_get_rows_q(int dev, int fmt, const void* table, size_t rows, size_t k, const void* ids,
                                     size_t n_ids, void* out, const litenn_hip_exec* opts)
{
	const char* action = "HIP GetRows";
	if (!is_weight_format(fmt) || row_bytes(fmt, k) == 0)
	{
		return fail(action, "unsupported block format or row width");
	}
	if (n_ids == 0)
	{
		return 0;
	}
	if (k > 0x7fffffffu || rows > 0x7fffffffu || n_ids > 0x7fffffffu)
	{
		return fail(action, "dimension exceeds 2^31-1");
	}
	if (!table || !ids || !out)
	{
		return fail(action, "null operand");
	}
	GUARD(action, dev);
	hipStream_t s = stream_of(opts);
	// the range check runs on the device; its flag is read back, which makes this call blocking
	int* flag = nullptr;
	LITENN_HIP_TRY(action, hipMalloc(reinterpret_cast<void**>(&flag), sizeof(int)));
	int host_flag = 0;
	hipError_t e = hipMemcpyAsync(flag, &host_flag, sizeof(int), hipMemcpyHostToDevice, s);
	if (e == hipSuccess)
	{
		launch_get_rows_q(fmt, table, rows, k, static_cast<const int32_t*>(ids), n_ids, static_cast<float*>(out), flag,
		                  s);
		e = hipGetLastError();
	}
	if (e == hipSuccess)
	{
		e = hipMemcpyAsync(&host_flag, flag, sizeof(int), hipMemcpyDeviceToHost, s);
	}
	if (e == hipSuccess)
	{
		e = hipStreamSynchronize(s);
	}
	(void)hipFree(flag);
	if (e != hipSuccess)
	{
		return fail_hip(action, e);
	}
	if (host_flag)
	{
		return fail(action, "GetRows index out of range");
	}
	return 0;
}

extern "C" int litenn_hip_rmsnorm(int dev, const void* x, const void* w, double eps, size_t m, size_t d, void* y,
                                  const litenn_hip_exec* opts)
{
	const char* action = "HIP RMSNorm";
	if (m == 0 || d == 0)
	{
		return 0;
	}
	if (d > 0x7fffffffu || m > 0x7fffffffu)
	{
		return fail(action, "dimension exceeds 2^31-1");
	}
	if (!x || !y) // w may be null: a norm without a weight
	{
		return fail(action, "null operand");
	}
	GUARD(action, dev);
	launch_rmsnorm(static_cast<const float*>(x), static_cast<const float*>(w), eps, m, d, static_cast<float*>(y),
	               stream_of(opts));
	return finish(action, opts);
}

extern "C" int litenn_hip_rope_interleaved(int dev, const void* x, void* y, size_t m, size_t n_heads, size_t head_dim,
                                           size_t rope_dims, double base, double freq_scale, size_t pos_offset,
                                           const litenn_hip_exec* opts)
{
	const char* action = "HIP RoPE";
	if (head_dim % 2 != 0)
	{
		return fail(action, "RoPE featureSize must be even");
	}
	if (rope_dims > head_dim || rope_dims % 2 != 0)
	{
		return fail(action, "rope dimension count must be even and no larger than headDim");
	}
	if (!(base > 0.0) || !(freq_scale > 0.0))
	{
		return fail(action, "RoPE base and frequencyScale must be finite and greater than zero");
	}
	if (m == 0 || n_heads == 0 || head_dim == 0)
	{
		return 0;
	}
	if (m * n_heads * head_dim > 0x7fffffffu)
	{
		return fail(action, "tensor too large");
	}
	if (!x || !y)
	{
		return fail(action, "null operand");
	}
	GUARD(action, dev);
	hipStream_t s = stream_of(opts);
	const size_t half = rope_dims / 2;
	float* tables = nullptr;
	if (half)
	{
		LITENN_HIP_TRY(action, hipMalloc(reinterpret_cast<void**>(&tables), sizeof(float) * 2 * m * half));
		launch_rope_table(tables, tables + m * half, m, half, base, freq_scale, pos_offset, s);
	}
	launch_rope(static_cast<const float*>(x), static_cast<float*>(y), m, n_heads, head_dim, rope_dims, tables,
	            tables ? tables + m * half : nullptr, s);
	// the angle tables are private to this call, so it always completes before returning
	hipError_t e = hipGetLastError();
	if (e == hipSuccess)
	{
		e = hipStreamSynchronize(s);
	}
	if (tables)
	{
		(void)hipFree(tables);
	}
	if (e != hipSuccess)
	{
		return fail_hip(action, e);
	}
	return 0;
}

extern "C" int litenn_hip_kv_append(int dev, void* cache, int cache_dtype, size_t past, const void* cur, size_t m,
                                    size_t width, const litenn_hip_exec* opts)
{
	const char* action = "HIP KV append";
	if (cache_dtype != LITENN_F16 && cache_dtype != LITENN_F32)
	{
		return fail(action, "cache dtype must be Float16 or Float32");
	}
	if (m == 0 || width == 0)
	{
		return 0;
	}
	if (!cache || !cur)
	{
		return fail(action, "null operand");
	}
	GUARD(action, dev);
	launch_kv_append(cache, cache_dtype, past * width, static_cast<const float*>(cur), m * width, stream_of(opts));
	return finish(action, opts);
}

// Operand checks shared by the attention entry points; returns 0, a failure status, or -1 when
// there is nothing to do (m == 0).
static int attn_check(const char* action, const void* q, const void* kcache, const void* vcache, int cache_dtype,
                      size_t m, size_t past, size_t n_head, size_t n_kv_head, size_t head_dim, const void* out)
{
	if (cache_dtype != LITENN_F16 && cache_dtype != LITENN_F32)
	{
		return fail(action, "cache dtype must be Float16 or Float32");
	}
	if (n_head == 0 || n_kv_head == 0 || n_head % n_kv_head != 0)
	{
		return fail(action, "head count must be a positive multiple of the KV head count");
	}
	if (head_dim == 0 || head_dim > 256)
	{
		return fail(action, "head dimension must be in [1, 256]");
	}
	if (m == 0)
	{
		return -1;
	}
	if (past + m > (size_t{ 1 } << 30))
	{
		return fail(action, "key length exceeds 2^30 positions");
	}
	if (m > 65535 || n_head > 65535)
	{
		return fail(action, "too many query rows or heads");
	}
	if (!q || !kcache || !vcache || !out)
	{
		return fail(action, "null operand");
	}
	return 0;
}

static int attn_rows_impl(int dev, const void* q, const void* kcache, const void* vcache, int cache_dtype, size_t m,
                          size_t past, size_t n_head, size_t n_kv_head, size_t head_dim, void* out, bool matrix_cores,
                          const litenn_hip_exec* opts)
{
	const char* action = "HIP attention";
	if (const int rc = attn_check(action, q, kcache, vcache, cache_dtype, m, past, n_head, n_kv_head, head_dim, out))
	{
		return rc < 0 ? 0 : rc;
	}
	GUARD(action, dev);
	if (matrix_cores && m >= 16 &&
	    launch_attn_tile(static_cast<const float*>(q), kcache, vcache, cache_dtype, m, nullptr, past, n_head, n_kv_head,
	                     head_dim, static_cast<float*>(out), stream_of(opts)))
	{
		return finish(action, opts);
	}
	// a single row against a long cache is cut into chunks that meet in scratch memory, which this
	// call takes and returns in stream order
	const size_t splits = attn_splits(m, past + m, n_head);
	StreamScratch scratch(stream_of(opts));
	float* partial = nullptr;
	int* counters = nullptr;
	if (splits > 1)
	{
		const size_t bytes = sizeof(float) * attn_partial_floats(m, n_head, head_dim, splits);
		LITENN_HIP_TRY(action, scratch.allocate(bytes + sizeof(int) * m * n_head));
		partial = static_cast<float*>(scratch.get());
		counters = reinterpret_cast<int*>(reinterpret_cast<char*>(partial) + bytes);
		launch_zero_ints(counters, m * n_head, stream_of(opts));
	}
	launch_attn_decode(static_cast<const float*>(q), kcache, vcache, cache_dtype, m, nullptr, past, n_head, n_kv_head,
	                   head_dim, static_cast<float*>(out), splits, partial, counters, stream_of(opts));
	return finish_with(scratch, action, opts);
}

extern "C" int litenn_hip_attn_decode(int dev, const void* q, const void* kcache, const void* vcache, int cache_dtype,
                                      size_t m, size_t past, size_t n_head, size_t n_kv_head, size_t head_dim,
                                      void* out, const litenn_hip_exec* opts)
{
	return attn_rows_impl(dev, q, kcache, vcache, cache_dtype, m, past, n_head, n_kv_head, head_dim, out, false, opts);
}

extern "C" int litenn_hip_attn_decode_noalloc(int dev, const void* q, const void* kcache, const void* vcache,
                                              int cache_dtype, size_t m, size_t past, size_t n_head, size_t n_kv_head,
                                              size_t head_dim, void* out, const litenn_hip_exec* opts)
{
	const char* action = "HIP attention (no allocation)";
	if (const int rc = attn_check(action, q, kcache, vcache, cache_dtype, m, past, n_head, n_kv_head, head_dim, out))
	{
		return rc < 0 ? 0 : rc;
	}
	const size_t splits = attn_splits(m, past + m, n_head);
	if (!attn_static_fits(m, n_head, head_dim, splits))
	{
		return fail(action, "a single row cut into key chunks needs more than the static scratch of " +
		                        std::to_string(attn_static_scratch_bytes()) +
		                        " bytes: heads * chunks * (head_dim + 2) must not exceed 262144 floats");
	}
	GUARD(action, dev);
	LITENN_HIP_TRY(action, launch_attn_decode_static(static_cast<const float*>(q), kcache, vcache, cache_dtype, m, past,
	                                                 n_head, n_kv_head, head_dim, static_cast<float*>(out), splits,
	                                                 stream_of(opts)));
	return finish(action, opts);
}

extern "C" int litenn_hip_attn_rows(int dev, const void* q, const void* kcache, const void* vcache, int cache_dtype,
                                    size_t m, size_t past, size_t n_head, size_t n_kv_head, size_t head_dim, void* out,
                                    unsigned flags, const litenn_hip_exec* opts)
{
	return attn_rows_impl(dev, q, kcache, vcache, cache_dtype, m, past, n_head, n_kv_head, head_dim, out,
	                      !(flags & LITENN_HIP_MATMUL_PRECISE), opts);
}

extern "C" int litenn_hip_flash_attn_ext(int dev, const void* q, const void* k, const void* v, int kv_dtype, size_t m,
                                        size_t keys, size_t n_head, size_t n_kv_head, size_t head_dim,
                                        const litenn_hip_attn_ext_opts* o, void* out, const litenn_hip_exec* opts)
{
	const char* action = "HIP FlashAttnExt";
	static const litenn_hip_attn_ext_opts plain = { 1.0, 0.0, 0.0, nullptr, nullptr, 0, 0, 0 };
	if (!o)
	{
		o = &plain;
	}
	if (keys == 0)
	{
		return fail(action, "no keys");
	}
	if (const int rc = attn_check(action, q, k, v, kv_dtype, m, 0, n_head, n_kv_head, head_dim, out))
	{
		return rc < 0 ? 0 : rc;
	}
	if (keys > (size_t{ 1 } << 30))
	{
		return fail(action, "key length exceeds 2^30 positions");
	}
	if (o->max_bias > 0.0 && !o->mask)
	{
		// the reference's text (src/LiteNN/Layer/FlashAttnExt.h:163-166)
		return fail(action, "FlashAttnExt maxBias requires an explicit additive mask");
	}
	if (!(o->scale == o->scale) || !(o->logit_softcap == o->logit_softcap) || !(o->max_bias == o->max_bias))
	{
		return fail(action, "scale, logit softcap and max bias must be numbers");
	}
	if (o->key_position_offset > (size_t{ 1 } << 40) || o->query_position_offset > (size_t{ 1 } << 40))
	{
		return fail(action, "position offsets exceed 2^40");
	}
	if (o->causal && o->key_position_offset > o->query_position_offset)
	{
		// such a row would take its weights from masked scores alone; the lowering never asks for it
		return fail(action, "the causal mask hides every key from the first query row");
	}
	GUARD(action, dev);
	launch_attn_ext(static_cast<const float*>(q), k, v, kv_dtype, m, keys, n_head, n_kv_head, head_dim, o->scale,
	                o->max_bias, o->logit_softcap, static_cast<const float*>(o->mask), static_cast<const float*>(o->sinks),
	                o->causal != 0, o->key_position_offset, o->query_position_offset, static_cast<float*>(out),
	                stream_of(opts));
	return finish(action, opts);
}

extern "C" int litenn_hip_silu_mul(int dev, const void* gate, const void* up, void* y, size_t n,
                                   const litenn_hip_exec* opts)
{
	const char* action = "HIP SiLU";
	if (n == 0)
	{
		return 0;
	}
	if (!gate || !up || !y)
	{
		return fail(action, "null operand");
	}
	GUARD(action, dev);
	launch_silu_mul(static_cast<const float*>(gate), static_cast<const float*>(up), static_cast<float*>(y), n,
	                stream_of(opts));
	return finish(action, opts);
}

extern "C" int litenn_hip_argmax(int dev, const void* x, size_t rows, size_t n, void* out_index,
                                 const litenn_hip_exec* opts)
{
	const char* action = "HIP argmax";
	if (rows == 0)
	{
		return 0;
	}
	if (n == 0 || n > 0x7fffffffu)
	{
		return fail(action, "row length must be in [1, 2^31-1]");
	}
	if (!x || !out_index)
	{
		return fail(action, "null operand");
	}
	GUARD(action, dev);
	launch_argmax(static_cast<const float*>(x), rows, n, static_cast<int32_t*>(out_index), stream_of(opts));
	return finish(action, opts);
}
