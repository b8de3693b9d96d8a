// Device versions of the generic DeviceTraits primitives (unary, binary with broadcast, reduce,
// concat, slice, get_rows, permute) so a graph lowered by the reference can run without the
// device -> host -> device round trips its CUDA backend takes for everything but MatMul
// (src/LiteNN/Device/CUDA.cpp:1894-2019).  Semantics follow DeviceTraits<CPU>
// (src/LiteNN/Device.h:393-966).  None of this is on the bandwidth-critical path; the kernels are
// simple, one element per thread, and keep the reference's evaluation order where it changes
// results (MatMul accumulates k-ascending with separately rounded multiply and add; reductions
// run sequentially along the reduced axis).
#include "common.hpp"

#include <type_traits>
#include <vector>

namespace litenn_hip
{
	namespace
	{
		constexpr int kMaxRank = 8;
		struct Dims
		{
			size_t v[kMaxRank];
		};

		// ---------------- unary ---------------------------------------------------------------
		template <typename T>
		__device__ __forceinline__ T unary_apply(int op, T a)
		{
			switch (op)
			{
			case LITENN_UN_NEGATE: return -a;
			case LITENN_UN_ABS: return a < T(0) ? -a : a;
			case LITENN_UN_SQRT: return static_cast<T>(sqrt(static_cast<double>(a)));
			case LITENN_UN_EXP: return static_cast<T>(exp(static_cast<double>(a)));
			case LITENN_UN_LOG: return static_cast<T>(log(static_cast<double>(a)));
			case LITENN_UN_SIN: return static_cast<T>(sin(static_cast<double>(a)));
			case LITENN_UN_COS: return static_cast<T>(cos(static_cast<double>(a)));
			case LITENN_UN_TAN: return static_cast<T>(tan(static_cast<double>(a)));
			case LITENN_UN_ARCSIN: return static_cast<T>(asin(static_cast<double>(a)));
			case LITENN_UN_ARCCOS: return static_cast<T>(acos(static_cast<double>(a)));
			case LITENN_UN_ARCTAN: return static_cast<T>(atan(static_cast<double>(a)));
			case LITENN_UN_ERF: return static_cast<T>(erf(static_cast<double>(a)));
			default: return a;
			}
		}
		// f32 uses the f32 library routines, like std::exp(float) etc. on the host
		template <>
		__device__ __forceinline__ float unary_apply<float>(int op, float a)
		{
			switch (op)
			{
			case LITENN_UN_NEGATE: return -a;
			case LITENN_UN_ABS: return fabsf(a);
			case LITENN_UN_SQRT: return sqrtf(a);
			case LITENN_UN_EXP: return expf(a);
			case LITENN_UN_LOG: return logf(a);
			case LITENN_UN_SIN: return sinf(a);
			case LITENN_UN_COS: return cosf(a);
			case LITENN_UN_TAN: return tanf(a);
			case LITENN_UN_ARCSIN: return asinf(a);
			case LITENN_UN_ARCCOS: return acosf(a);
			case LITENN_UN_ARCTAN: return atanf(a);
			case LITENN_UN_ERF: return erff(a);
			default: return a;
			}
		}

		template <typename T>
		__global__ void unary_kernel(int op, const T* __restrict__ src, T* __restrict__ dst, size_t n)
		{
			const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
			if (i < n)
			{
				dst[i] = unary_apply<T>(op, src[i]);
			}
		}

		__global__ void logical_not_kernel(const bool* __restrict__ src, bool* __restrict__ dst, size_t n)
		{
			const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
			if (i < n)
			{
				dst[i] = !src[i];
			}
		}

		// ---------------- permute / transpose (any element size) -------------------------------
		template <typename T>
		__global__ void permute_kernel(const T* __restrict__ src, T* __restrict__ dst, size_t total, int rank,
		                               Dims dst_shape, Dims src_stride_of_dst_axis)
		{
			const size_t linear = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
			if (linear >= total)
			{
				return;
			}
			size_t rem = linear, off = 0;
			for (int d = rank - 1; d >= 0; --d)
			{
				const size_t c = rem % dst_shape.v[d];
				rem /= dst_shape.v[d];
				off += c * src_stride_of_dst_axis.v[d];
			}
			dst[linear] = src[off];
		}

		// ---------------- binary with broadcast ------------------------------------------------
		template <typename T>
		__device__ __forceinline__ T binary_apply(int op, T a, T b)
		{
			switch (op)
			{
			case LITENN_BIN_ADD: return a + b;
			case LITENN_BIN_SUBTRACT: return a - b;
			case LITENN_BIN_MULTIPLY: return a * b;
			case LITENN_BIN_DIVIDE: return a / b;
			case LITENN_BIN_POW: {
				const double p = pow(static_cast<double>(a), static_cast<double>(b));
				if constexpr (std::is_integral<T>::value)
				{
					// std::pow(int, int) on the host returns the exact integer for a non-negative
					// exponent (while it fits a double); the device routine may land one unit in
					// the last place below it, which the cast would turn into the next integer down
					return static_cast<T>(b >= T(0) ? rint(p) : p);
				}
				return static_cast<T>(p);
			}
			case LITENN_BIN_MAX: return a < b ? b : a; // std::max(a, b)
			case LITENN_BIN_MIN: return b < a ? b : a; // std::min(a, b)
			default: return a;
			}
		}
		template <>
		__device__ __forceinline__ float binary_apply<float>(int op, float a, float b)
		{
			switch (op)
			{
			case LITENN_BIN_ADD: return __fadd_rn(a, b);
			case LITENN_BIN_SUBTRACT: return __fsub_rn(a, b);
			case LITENN_BIN_MULTIPLY: return __fmul_rn(a, b);
			case LITENN_BIN_DIVIDE: return __fdiv_rn(a, b);
			case LITENN_BIN_POW: return powf(a, b);
			case LITENN_BIN_MAX: return a < b ? b : a;
			case LITENN_BIN_MIN: return b < a ? b : a;
			default: return a;
			}
		}

		// strides are in elements over the RESULT's axes, 0 where the operand broadcasts
		template <typename T, typename R, bool Compare>
		__global__ void binary_kernel(int op, const T* __restrict__ a, const T* __restrict__ b, R* __restrict__ dst,
		                              size_t total, int rank, Dims shape, Dims sa, Dims sb)
		{
			const size_t linear = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
			if (linear >= total)
			{
				return;
			}
			size_t rem = linear, oa = 0, ob = 0;
			for (int d = rank - 1; d >= 0; --d)
			{
				const size_t c = rem % shape.v[d];
				rem /= shape.v[d];
				oa += c * sa.v[d];
				ob += c * sb.v[d];
			}
			if constexpr (Compare)
			{
				const T x = a[oa], y = b[ob];
				dst[linear] = op == LITENN_BIN_LESS ? (x < y) : op == LITENN_BIN_GREATER ? (x > y) : (x == y);
			}
			else
			{
				dst[linear] = binary_apply<T>(op, a[oa], b[ob]);
			}
		}

		// ---------------- MatMul: bit-for-bit the i-k-j loop of Device.h:645-658 --------------
		// One thread per output element; k ascends; multiply and add round separately, so the
		// result equals the host loop exactly.  A and B tiles are staged through LDS.
		// The compiler contracts a * b + c into a fused multiply-add by default, also through the
		// *_rn intrinsics (they are plain operators here); the pragma keeps the two roundings of
		// the host loop (x86-64 without FMA).
		template <typename T>
		__device__ __forceinline__ T mul_then_add(T acc, T a, T b)
		{
#pragma clang fp contract(off)
			const T product = a * b;
			return acc + product;
		}

		template <typename T>
		__global__ __launch_bounds__(256) void matmul_kernel(const T* __restrict__ a, const T* __restrict__ b,
		                                                      T* __restrict__ c, int m, int k, int n)
		{
			__shared__ T ta[16][17];
			__shared__ T tb[16][17];
			const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
			const int row = blockIdx.y * 16 + ty, col = blockIdx.x * 16 + tx;
			T acc = T(0);
			for (int k0 = 0; k0 < k; k0 += 16)
			{
				ta[ty][tx] = (row < m && k0 + tx < k) ? a[static_cast<size_t>(row) * k + k0 + tx] : T(0);
				tb[ty][tx] = (k0 + ty < k && col < n) ? b[static_cast<size_t>(k0 + ty) * n + col] : T(0);
				__syncthreads();
				const int kn = min(16, k - k0);
				for (int kk = 0; kk < kn; ++kk)
				{
					acc = mul_then_add<T>(acc, ta[ty][kk], tb[kk][tx]);
				}
				__syncthreads();
			}
			if (row < m && col < n)
			{
				c[static_cast<size_t>(row) * n + col] = acc;
			}
		}

		// ---------------- reduce along one axis, sequential like Device.h:727-756 -------------
		template <typename T>
		__global__ void reduce_kernel(int op, const T* __restrict__ src, T* __restrict__ dst, size_t outer,
		                              size_t reduce_dim, size_t inner)
		{
			const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
			if (idx >= outer * inner)
			{
				return;
			}
			const size_t o = idx / inner, j = idx % inner;
			T acc = src[(o * reduce_dim) * inner + j];
			for (size_t r = 1; r < reduce_dim; ++r)
			{
				const T val = src[(o * reduce_dim + r) * inner + j];
				if (op == LITENN_RED_MAX)
				{
					if (val > acc)
					{
						acc = val;
					}
				}
				else
				{
					acc = acc + val;
				}
			}
			if (op == LITENN_RED_MEAN)
			{
				acc = acc / static_cast<T>(reduce_dim);
			}
			dst[idx] = acc;
		}

		// ---------------- strided block copy: concat, slice, get_rows -------------------------
		// copies `count` chunks of `chunk` bytes: src + i*src_stride -> dst + i*dst_stride
		__global__ void chunk_copy_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, size_t count,
		                                  size_t chunk, size_t src_stride, size_t dst_stride)
		{
			const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
			if (idx >= count * chunk)
			{
				return;
			}
			const size_t i = idx / chunk, b = idx % chunk;
			dst[i * dst_stride + b] = src[i * src_stride + b];
		}

		template <typename I>
		__global__ void get_rows_kernel(const uint8_t* __restrict__ data, size_t rows, size_t row_bytes,
		                                const I* __restrict__ idx, size_t n_idx, uint8_t* __restrict__ dst,
		                                int* err_flag)
		{
			const size_t i = blockIdx.x;
			const I raw = idx[i];
			if (raw < 0 || static_cast<size_t>(raw) >= rows)
			{
				if (threadIdx.x == 0)
				{
					*err_flag = 1;
				}
				return;
			}
			for (size_t b = threadIdx.x; b < row_bytes; b += blockDim.x)
			{
				dst[i * row_bytes + b] = data[static_cast<size_t>(raw) * row_bytes + b];
			}
		}

		size_t product(const size_t* shape, size_t from, size_t to)
		{
			size_t p = 1;
			for (size_t i = from; i < to; ++i)
			{
				p *= shape[i];
			}
			return p;
		}

		dim3 grid_for(size_t n) { return dim3(static_cast<unsigned>((n + 255) / 256)); }

		template <typename F>
		bool dispatch_numeric(int dtype, F&& f)
		{
			switch (dtype)
			{
			case LITENN_F32: f(float{}); return true;
			case LITENN_F64: f(double{}); return true;
			case LITENN_I32: f(int32_t{}); return true;
			case LITENN_I64: f(int64_t{}); return true;
			case LITENN_I8: f(int8_t{}); return true;
			case LITENN_U8: f(uint8_t{}); return true;
			default: return false;
			}
		}

		template <typename F>
		bool dispatch_size(size_t es, F&& f)
		{
			switch (es)
			{
			case 1: f(uint8_t{}); return true;
			case 2: f(uint16_t{}); return true;
			case 4: f(uint32_t{}); return true;
			case 8: f(uint64_t{}); return true;
			default: return false;
			}
		}
	} // namespace
} // namespace litenn_hip

using namespace litenn_hip;

#define GUARD(action, dev)                                                                                             \
	DeviceGuard guard_(dev);                                                                                           \
	if (!guard_.ok())                                                                                                  \
	{                                                                                                                  \
		return fail_hip(action, guard_.error());                                                                       \
	}

extern "C" int litenn_hip_permute(int dev, void* dst, int dtype, const size_t* src_shape, size_t rank, const void* src,
                                  const size_t* perm, const litenn_hip_exec* opts)
{
	const char* action = "HIP permute";
	if ((rank && (!src_shape || !perm)))
	{
		return fail(action, "null shape");
	}
	const size_t es = dtype_size(dtype);
	if (es == 0)
	{
		return fail(action, "bad dtype");
	}
	if (rank > static_cast<size_t>(kMaxRank))
	{
		return fail(action, "rank exceeds 8");
	}
	std::vector<bool> seen(rank, false);
	for (size_t d = 0; d < rank; ++d)
	{
		if (perm[d] >= rank || seen[perm[d]])
		{
			return fail(action, "Permute permutation must be a valid permutation of [0, rank)");
		}
		seen[perm[d]] = true;
	}
	const size_t total = product(src_shape, 0, rank);
	if (total == 0)
	{
		return 0;
	}
	if (!dst || !src || !perm)
	{
		return fail(action, "null operand");
	}
	GUARD(action, dev);
	hipStream_t s = stream_of(opts);
	if (rank == 0)
	{
		LITENN_HIP_TRY(action, hipMemcpyAsync(dst, src, es, hipMemcpyDeviceToDevice, s));
		return finish(action, opts);
	}
	size_t src_strides[kMaxRank];
	src_strides[rank - 1] = 1;
	for (size_t d = rank - 1; d > 0; --d)
	{
		src_strides[d - 1] = src_strides[d] * src_shape[d];
	}
	Dims dshape{}, dstride{};
	for (size_t d = 0; d < rank; ++d)
	{
		dshape.v[d] = src_shape[perm[d]];
		dstride.v[d] = src_strides[perm[d]];
	}
	dispatch_size(es, [&](auto tag) {
		using T = decltype(tag);
		permute_kernel<T><<<grid_for(total), 256, 0, s>>>(static_cast<const T*>(src), static_cast<T*>(dst), total,
		                                                   static_cast<int>(rank), dshape, dstride);
	});
	return finish(action, opts);
}

extern "C" int litenn_hip_unary(int dev, int op, void* dst, int dtype, const size_t* shape, size_t rank,
                                const void* src, const litenn_hip_exec* opts)
{
	const char* action = "HIP unary op";
	if ((rank && !shape))
	{
		return fail(action, "null shape");
	}
	if (dtype_size(dtype) == 0)
	{
		return fail(action, "bad dtype");
	}
	if (op == LITENN_UN_TRANSPOSE)
	{
		if (rank != 2)
		{
			return fail(action, "Transpose only supports 2D tensors");
		}
		const size_t perm[2] = { 1, 0 };
		return litenn_hip_permute(dev, dst, dtype, shape, 2, src, perm, opts);
	}
	const size_t n = product(shape, 0, rank);
	if (op == LITENN_UN_LOGICAL_NEGATION)
	{
		if (dtype != LITENN_BOOL)
		{
			return fail(action, "LogicalNegation only supports boolean tensors");
		}
		if (n == 0)
		{
			return 0;
		}
		if (!dst || !src)
		{
			return fail(action, "null operand");
		}
		GUARD(action, dev);
		logical_not_kernel<<<grid_for(n), 256, 0, stream_of(opts)>>>(static_cast<const bool*>(src),
		                                                              static_cast<bool*>(dst), n);
		return finish(action, opts);
	}
	if (dtype == LITENN_BOOL)
	{
		return fail(action, "Default UnaryOp does not support boolean tensors");
	}
	if (op < 0 || op > LITENN_UN_ERF)
	{
		return fail(action, "unknown unary op");
	}
	if (n == 0)
	{
		return 0;
	}
	if (!dst || !src)
	{
		return fail(action, "null operand");
	}
	GUARD(action, dev);
	hipStream_t s = stream_of(opts);
	const bool ok = dispatch_numeric(dtype, [&](auto tag) {
		using T = decltype(tag);
		unary_kernel<T><<<grid_for(n), 256, 0, s>>>(op, static_cast<const T*>(src), static_cast<T*>(dst), n);
	});
	if (!ok)
	{
		return fail(action, "dtype is not supported on the device");
	}
	return finish(action, opts);
}

extern "C" int litenn_hip_binary(int dev, int op, void* dst, int dtype1, const size_t* shape1, size_t rank1,
                                 const void* src1, int dtype2, const size_t* shape2, size_t rank2, const void* src2,
                                 const litenn_hip_exec* opts)
{
	const char* action = "HIP binary op";
	if (((rank1 && !shape1) || (rank2 && !shape2)))
	{
		return fail(action, "null shape");
	}
	if (dtype1 != dtype2)
	{
		return fail(action, op == LITENN_BIN_MATMUL ? "MatMul requires both inputs to have the same data type"
		                                             : "Default BinaryOp requires both inputs to have the same data type");
	}
	if (op < 0 || op > LITENN_BIN_EQUAL)
	{
		return fail(action, "unknown binary op");
	}
	if (op == LITENN_BIN_MATMUL)
	{
		if (rank1 != 2 || rank2 != 2)
		{
			return fail(action, "MatMul only supports 2D tensors");
		}
		if (shape1[1] != shape2[0])
		{
			return fail(action, "MatMul requires the inner dimensions of the two inputs to match");
		}
		const size_t m = shape1[0], k = shape1[1], n = shape2[1];
		if (m > 0x7fffffffu || k > 0x7fffffffu || n > 0x7fffffffu)
		{
			return fail(action, "dimension exceeds 2^31-1");
		}
		if (dtype1 != LITENN_F32 && dtype1 != LITENN_F64)
		{
			return fail(action, "MatMul dtype is not supported on the device");
		}
		if (m == 0 || n == 0)
		{
			return 0;
		}
		if (!dst || !src1 || !src2)
		{
			return fail(action, "null operand");
		}
		GUARD(action, dev);
		hipStream_t s = stream_of(opts);
		const dim3 grid(static_cast<unsigned>((n + 15) / 16), static_cast<unsigned>((m + 15) / 16));
		if (dtype1 == LITENN_F32)
		{
			matmul_kernel<float><<<grid, 256, 0, s>>>(static_cast<const float*>(src1), static_cast<const float*>(src2),
			                                           static_cast<float*>(dst), static_cast<int>(m),
			                                           static_cast<int>(k), static_cast<int>(n));
		}
		else
		{
			matmul_kernel<double><<<grid, 256, 0, s>>>(static_cast<const double*>(src1),
			                                            static_cast<const double*>(src2), static_cast<double*>(dst),
			                                            static_cast<int>(m), static_cast<int>(k), static_cast<int>(n));
		}
		return finish(action, opts);
	}
	if (dtype1 == LITENN_BOOL)
	{
		return fail(action, "Default BinaryOp does not support boolean tensors");
	}
	// Result shape: DefaultBinaryOpTraits::ResultShape (Operators.h:173-188).  Executed cases: equal
	// ranks (extent 1 broadcasts), and a rank-1 operand against a higher-rank one, which the CPU
	// loop applies along the LAST axis (Device.h:566-578).
	const size_t rank = rank1 > rank2 ? rank1 : rank2;
	if (rank > static_cast<size_t>(kMaxRank) || rank == 0)
	{
		return fail(action, "rank must be in [1, 8]");
	}
	Dims shape{}, sa{}, sb{};
	auto strides_for = [&](const size_t* sh, size_t r, Dims& out) -> bool {
		for (size_t d = 0; d < rank; ++d)
		{
			out.v[d] = 0;
		}
		if (r == rank)
		{
			size_t stride = 1;
			for (size_t d = rank; d-- > 0;)
			{
				if (sh[d] != 1 && sh[d] != shape.v[d])
				{
					return false;
				}
				out.v[d] = sh[d] == 1 ? 0 : stride;
				stride *= sh[d];
			}
			return true;
		}
		if (r == 1)
		{
			if (sh[0] != 1 && sh[0] != shape.v[rank - 1])
			{
				return false;
			}
			out.v[rank - 1] = sh[0] == 1 ? 0 : 1;
			return true;
		}
		return false;
	};
	for (size_t d = 0; d < rank; ++d)
	{
		const size_t d1 = rank1 == rank ? shape1[d] : 1, d2 = rank2 == rank ? shape2[d] : 1;
		shape.v[d] = d1 > d2 ? d1 : d2;
	}
	if (!strides_for(shape1, rank1, sa) || !strides_for(shape2, rank2, sb))
	{
		return fail(action, "BinaryOp requires input shapes to be compatible for broadcasting");
	}
	size_t total = 1;
	for (size_t d = 0; d < rank; ++d)
	{
		total *= shape.v[d];
	}
	if (total == 0)
	{
		return 0;
	}
	if (!dst || !src1 || !src2)
	{
		return fail(action, "null operand");
	}
	GUARD(action, dev);
	hipStream_t s = stream_of(opts);
	const bool compare = op >= LITENN_BIN_LESS;
	const bool ok = dispatch_numeric(dtype1, [&](auto tag) {
		using T = decltype(tag);
		if (compare)
		{
			binary_kernel<T, bool, true><<<grid_for(total), 256, 0, s>>>(op, static_cast<const T*>(src1),
			                                                              static_cast<const T*>(src2),
			                                                              static_cast<bool*>(dst), total,
			                                                              static_cast<int>(rank), shape, sa, sb);
		}
		else
		{
			binary_kernel<T, T, false><<<grid_for(total), 256, 0, s>>>(op, static_cast<const T*>(src1),
			                                                            static_cast<const T*>(src2),
			                                                            static_cast<T*>(dst), total,
			                                                            static_cast<int>(rank), shape, sa, sb);
		}
	});
	if (!ok)
	{
		return fail(action, "dtype is not supported on the device");
	}
	return finish(action, opts);
}

extern "C" int litenn_hip_reduce(int dev, int op, void* dst, int dtype, const size_t* shape, size_t rank,
                                 const void* src, size_t axis, const litenn_hip_exec* opts)
{
	const char* action = "HIP reduce op";
	if ((rank && !shape))
	{
		return fail(action, "null shape");
	}
	if (axis >= rank)
	{
		return fail(action, "ReduceOp axis out of range");
	}
	if (dtype == LITENN_BOOL)
	{
		return fail(action, "ReduceOp does not support boolean tensors");
	}
	if (op < 0 || op > LITENN_RED_MAX)
	{
		return fail(action, "unknown reduce op");
	}
	const size_t outer = product(shape, 0, axis), rd = shape[axis], inner = product(shape, axis + 1, rank);
	if (outer * inner == 0)
	{
		return 0;
	}
	if (rd == 0)
	{
		return fail(action, "cannot reduce over an empty axis");
	}
	if (!dst || !src)
	{
		return fail(action, "null operand");
	}
	GUARD(action, dev);
	hipStream_t s = stream_of(opts);
	const bool ok = dispatch_numeric(dtype, [&](auto tag) {
		using T = decltype(tag);
		reduce_kernel<T><<<grid_for(outer * inner), 256, 0, s>>>(op, static_cast<const T*>(src), static_cast<T*>(dst),
		                                                          outer, rd, inner);
	});
	if (!ok)
	{
		return fail(action, "dtype is not supported on the device");
	}
	return finish(action, opts);
}

extern "C" int litenn_hip_concat(int dev, void* dst, int dtype, const void* const* srcs, const size_t* shapes,
                                 size_t rank, size_t input_count, size_t axis, const litenn_hip_exec* opts)
{
	const char* action = "HIP concat";
	if ((rank && input_count && !shapes) || !srcs)
	{
		return fail(action, "null shape");
	}
	const size_t es = dtype_size(dtype);
	if (es == 0)
	{
		return fail(action, "bad dtype");
	}
	if (input_count == 0 || axis >= rank)
	{
		return fail(action, "concat needs at least one input and an axis inside the rank");
	}
	for (size_t i = 1; i < input_count; ++i)
	{
		for (size_t d = 0; d < rank; ++d)
		{
			if (d != axis && shapes[i * rank + d] != shapes[d])
			{
				return fail(action, "concat inputs must agree on every axis but the concatenated one");
			}
		}
	}
	const size_t outer = product(shapes, 0, axis), inner = product(shapes, axis + 1, rank);
	size_t total_axis = 0;
	for (size_t i = 0; i < input_count; ++i)
	{
		total_axis += shapes[i * rank + axis];
	}
	if (!dst)
	{
		return fail(action, "null operand");
	}
	for (size_t i = 0; i < input_count; ++i)
	{
		if (!srcs[i] && outer * inner * shapes[i * rank + axis] != 0)
		{
			return fail(action, "null operand");
		}
	}
	GUARD(action, dev);
	hipStream_t s = stream_of(opts);
	size_t axis_off = 0;
	for (size_t i = 0; i < input_count; ++i)
	{
		const size_t chunk = shapes[i * rank + axis] * inner * es;
		if (chunk && outer)
		{
			chunk_copy_kernel<<<grid_for(outer * chunk), 256, 0, s>>>(
			    static_cast<const uint8_t*>(srcs[i]), static_cast<uint8_t*>(dst) + axis_off * inner * es, outer, chunk,
			    chunk, total_axis * inner * es);
		}
		axis_off += shapes[i * rank + axis];
	}
	return finish(action, opts);
}

extern "C" int litenn_hip_slice(int dev, void* dst, int dtype, const size_t* src_shape, size_t rank, const void* src,
                                size_t axis, size_t start, size_t length, const litenn_hip_exec* opts)
{
	const char* action = "HIP slice";
	if ((rank && !src_shape))
	{
		return fail(action, "null shape");
	}
	const size_t es = dtype_size(dtype);
	if (es == 0)
	{
		return fail(action, "bad dtype");
	}
	if (axis >= rank || start + length > src_shape[axis])
	{
		return fail(action, "slice range out of bounds");
	}
	const size_t outer = product(src_shape, 0, axis), inner = product(src_shape, axis + 1, rank);
	const size_t chunk = length * inner * es;
	if (outer * chunk == 0)
	{
		return 0;
	}
	if (!dst || !src)
	{
		return fail(action, "null operand");
	}
	GUARD(action, dev);
	chunk_copy_kernel<<<grid_for(outer * chunk), 256, 0, stream_of(opts)>>>(
	    static_cast<const uint8_t*>(src) + start * inner * es, static_cast<uint8_t*>(dst), outer, chunk,
	    src_shape[axis] * inner * es, chunk);
	return finish(action, opts);
}

extern "C" int litenn_hip_get_rows(int dev, void* dst, int dtype, const size_t* data_shape, size_t data_rank,
                                   const void* data, int index_dtype, const size_t* index_shape, size_t index_rank,
                                   const void* indices, const litenn_hip_exec* opts)
{
	const char* action = "HIP GetRows";
	if (((data_rank && !data_shape) || (index_rank && !index_shape)))
	{
		return fail(action, "null shape");
	}
	const size_t es = dtype_size(dtype);
	if (es == 0)
	{
		return fail(action, "bad dtype");
	}
	if (data_rank == 0)
	{
		return fail(action, "GetRows requires a rank >= 1 data tensor");
	}
	if (index_dtype != LITENN_I32 && index_dtype != LITENN_I64)
	{
		return fail(action, "GetRows indices must have dtype Int32 or Int64");
	}
	const size_t rows = data_shape[0], rb = product(data_shape, 1, data_rank) * es;
	const size_t n_idx = product(index_shape, 0, index_rank);
	if (n_idx == 0)
	{
		return 0;
	}
	if (n_idx > 0x7fffffffu)
	{
		return fail(action, "index count exceeds 2^31-1");
	}
	if (!dst || !data || !indices)
	{
		return fail(action, "null operand");
	}
	GUARD(action, dev);
	hipStream_t s = stream_of(opts);
	int* flag = nullptr;
	LITENN_HIP_TRY(action, hipMalloc(reinterpret_cast<void**>(&flag), sizeof(int)));
	int host_flag = 0;
	hipError_t e = hipMemcpyAsync(flag, &host_flag, sizeof(int), hipMemcpyHostToDevice, s);
	if (e == hipSuccess)
	{
		if (index_dtype == LITENN_I32)
		{
			get_rows_kernel<int32_t><<<dim3(static_cast<unsigned>(n_idx)), 256, 0, s>>>(
			    static_cast<const uint8_t*>(data), rows, rb, static_cast<const int32_t*>(indices), n_idx,
			    static_cast<uint8_t*>(dst), flag);
		}
		else
		{
			get_rows_kernel<int64_t><<<dim3(static_cast<unsigned>(n_idx)), 256, 0, s>>>(
			    static_cast<const uint8_t*>(data), rows, rb, static_cast<const int64_t*>(indices), n_idx,
			    static_cast<uint8_t*>(dst), flag);
		}
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
