// LiteNN::HIP -- the device tag and DeviceTraits<HIP> specialisation over the C ABI of
// litenn_hip.h, written the way src/LiteNN/Device/CUDA.h:16-25,98-165 declares the CUDA backend
// (same member names, argument order and error behaviour as the Device concept,
// src/LiteNN/Device.h:17-69).
//
// LiteNN's own headers need a C++26 reflection compiler.  When they are on the include path
// (LITENN_DEVICE_H is defined by <LiteNN/Device.h>) this header specialises the reference's
// DeviceTraits; otherwise it brings the small vocabulary the traits speak (DataType, the operator
// enums, ShapeView) with the reference's positional values, so that the backend can be built and
// tested with an ordinary C++20 compiler.
#ifndef LITENN_DEVICE_HIP_H
#define LITENN_DEVICE_HIP_H

#include <cstddef>
#include <cstdint>
#include <initializer_list>
#include <stdexcept>
#include <string>
#include <string_view>
#include <vector>

#include "../../litenn_hip.h"

#ifndef LITENN_DEVICE_H
namespace LiteNN
{
	// src/LiteNN/DType.h:17-30
	enum class DataType
	{
		Float32, Float64, Int32, Int64, Bool, Float16, BFloat16, Float8E4M3, Float8E5M2, Int8, UInt8,
	};
	// src/LiteNN/Operators.h:12-51,237-242
	enum class UnaryOp
	{
		Negate, Abs, Sqrt, Exp, Log, Sin, Cos, Tan, Arcsin, Arccos, Arctan, Transpose, LogicalNegation, Erf,
	};
	enum class BinaryOp
	{
		Add, Subtract, Multiply, Divide, MatMul, Pow, Max, Min, Less, Greater, Equal,
	};
	enum class ReduceOp
	{
		Sum, Mean, Max,
	};
	// src/LiteNN/Quantization.h:31-62 (the members this backend executes)
	enum class QuantizedBlockFormat
	{
		Q4_0 = 1, Q4_1 = 2, Q5_0 = 3, Q5_1 = 4, Q8_0 = 5, Q2_K = 7, Q3_K = 8, Q4_K = 9, Q5_K = 10, Q6_K = 11, F16 = 25, F32 = 27,
	};

	// the view of a shape the traits take (src/LiteNN/Device.h uses ShapeView the same way)
	class ShapeView
	{
	public:
		ShapeView(const std::size_t* data, std::size_t count) : data_(data), count_(count) {}
		ShapeView(const std::vector<std::size_t>& v) : data_(v.data()), count_(v.size()) {}
		// a braced list lives until the end of the call it is an argument of, which is all a view needs
#if defined(__GNUC__) && !defined(__clang__)
#pragma GCC diagnostic push
#pragma GCC diagnostic ignored "-Winit-list-lifetime"
#endif
		ShapeView(std::initializer_list<std::size_t> v) : data_(v.begin()), count_(v.size()) {}
#if defined(__GNUC__) && !defined(__clang__)
#pragma GCC diagnostic pop
#endif
		std::size_t NumDim() const { return count_; }
		std::size_t operator[](std::size_t i) const { return data_[i]; }
		const std::size_t* begin() const { return data_; }
		const std::size_t* end() const { return data_ + count_; }

	private:
		const std::size_t* data_;
		std::size_t count_;
	};

	template <typename D>
	struct DeviceTraits;
} // namespace LiteNN
#endif

namespace LiteNN
{
	struct HIP
	{
		int deviceIndex = 0;
		mutable std::string infoCache;

		bool operator==(const HIP& other) const
		{
			return deviceIndex == other.deviceIndex;
		}
	};

	// CUDADeviceCount / IsCUDADeviceAvailable, src/LiteNN/Device/CUDA.h:27-28
	inline int HIPDeviceCount() noexcept
	{
		return litenn_hip_device_count();
	}
	inline bool IsHIPDeviceAvailable(int deviceIndex = 0) noexcept
	{
		return deviceIndex >= 0 && deviceIndex < litenn_hip_device_count();
	}

	// CUDAExecutionOptions, src/LiteNN/Device/CUDA.h:70-74
	struct HIPExecutionOptions
	{
		void* stream{};
		bool synchronize{ true };
	};

	namespace Detail
	{
		// the reference throws std::runtime_error("<action> failed: <message>")
		// (src/LiteNN/Device/CUDA.cpp:89-95); the library formats its message that way
		inline void HIPCheck(int status)
		{
			if (status != 0)
			{
				throw std::runtime_error(litenn_hip_last_error());
			}
		}
		inline std::vector<std::size_t> Extents(ShapeView shape)
		{
			return std::vector<std::size_t>(shape.begin(), shape.end());
		}
		inline litenn_hip_exec Exec(const HIPExecutionOptions& o)
		{
			return litenn_hip_exec{ o.stream, o.synchronize ? 1 : 0 };
		}
	} // namespace Detail

	template <>
	struct DeviceTraits<HIP>
	{
		static std::string_view Name()
		{
			return "HIP";
		}
		static std::string_view Info(const HIP& device)
		{
			char buf[256] = {};
			Detail::HIPCheck(litenn_hip_device_info(device.deviceIndex, buf, sizeof buf));
			device.infoCache = buf;
			return device.infoCache;
		}

		// size is an element count; the storage is uninitialised (src/LiteNN/Device.h:28-34)
		static void* Allocate(HIP& device, DataType type, std::size_t size)
		{
			void* ptr = nullptr;
			Detail::HIPCheck(litenn_hip_alloc(device.deviceIndex, static_cast<int>(type), size, &ptr));
			return ptr;
		}
		static void Deallocate(HIP& device, void* ptr, DataType type, std::size_t size)
		{
			Detail::HIPCheck(litenn_hip_free(device.deviceIndex, ptr, static_cast<int>(type), size));
		}
		static void ZeroFill(HIP& device, void* ptr, DataType type, std::size_t size)
		{
			Detail::HIPCheck(litenn_hip_zero(device.deviceIndex, ptr, static_cast<int>(type), size));
		}
		static void CopyToCPU(const HIP& device, DataType srcType, const void* src, std::size_t size, DataType dstType,
		                      void* dst)
		{
			Detail::HIPCheck(litenn_hip_copy_to_host(device.deviceIndex, static_cast<int>(srcType), src, size,
			                                         static_cast<int>(dstType), dst, nullptr));
		}
		static void CopyFromCPU(HIP& device, DataType dstType, void* dst, DataType srcType, const void* src,
		                        std::size_t size)
		{
			Detail::HIPCheck(litenn_hip_copy_from_host(device.deviceIndex, static_cast<int>(dstType), dst,
			                                           static_cast<int>(srcType), src, size, nullptr));
		}
		static void ConvertTo(const HIP& device, DataType srcType, const void* src, std::size_t size, DataType dstType,
		                      void* dst)
		{
			Detail::HIPCheck(litenn_hip_convert(device.deviceIndex, static_cast<int>(srcType), src, size,
			                                    static_cast<int>(dstType), dst, nullptr));
		}

		static void DoUnaryOp(HIP& device, UnaryOp op, void* dst, DataType type, ShapeView shape, const void* src)
		{
			const auto e = Detail::Extents(shape);
			Detail::HIPCheck(litenn_hip_unary(device.deviceIndex, static_cast<int>(op), dst, static_cast<int>(type),
			                                  e.data(), e.size(), src, nullptr));
		}
		static void DoBinaryOp(HIP& device, BinaryOp op, void* dst, DataType type1, ShapeView shape1, const void* src1,
		                       DataType type2, ShapeView shape2, const void* src2)
		{
			const auto e1 = Detail::Extents(shape1), e2 = Detail::Extents(shape2);
			Detail::HIPCheck(litenn_hip_binary(device.deviceIndex, static_cast<int>(op), dst, static_cast<int>(type1),
			                                   e1.data(), e1.size(), src1, static_cast<int>(type2), e2.data(), e2.size(),
			                                   src2, nullptr));
		}
		static void DoReduceOp(HIP& device, ReduceOp op, void* dst, DataType type, ShapeView shape, const void* src,
		                       std::size_t axis)
		{
			const auto e = Detail::Extents(shape);
			Detail::HIPCheck(litenn_hip_reduce(device.deviceIndex, static_cast<int>(op), dst, static_cast<int>(type),
			                                   e.data(), e.size(), src, axis, nullptr));
		}
		static void DoConcatOp(HIP& device, void* dst, DataType type, const void* const* srcPtrs,
		                       const ShapeView* srcShapes, std::size_t inputCount, std::size_t axis)
		{
			const std::size_t rank = inputCount ? srcShapes[0].NumDim() : 0;
			std::vector<std::size_t> flat;
			for (std::size_t i = 0; i < inputCount; ++i)
			{
				flat.insert(flat.end(), srcShapes[i].begin(), srcShapes[i].end());
			}
			Detail::HIPCheck(litenn_hip_concat(device.deviceIndex, dst, static_cast<int>(type), srcPtrs, flat.data(), rank,
			                                   inputCount, axis, nullptr));
		}
		static void DoSliceOp(HIP& device, void* dst, DataType type, ShapeView shape, const void* src, std::size_t axis,
		                      std::size_t start, std::size_t length)
		{
			const auto e = Detail::Extents(shape);
			Detail::HIPCheck(litenn_hip_slice(device.deviceIndex, dst, static_cast<int>(type), e.data(), e.size(), src,
			                                  axis, start, length, nullptr));
		}
		static void DoGetRowsOp(HIP& device, void* dst, DataType type, ShapeView dataShape, const void* data,
		                        DataType indexType, ShapeView indexShape, const void* indices)
		{
			const auto e = Detail::Extents(dataShape), ie = Detail::Extents(indexShape);
			Detail::HIPCheck(litenn_hip_get_rows(device.deviceIndex, dst, static_cast<int>(type), e.data(), e.size(), data,
			                                     static_cast<int>(indexType), ie.data(), ie.size(), indices, nullptr));
		}
		static void DoPermuteOp(HIP& device, void* dst, DataType type, ShapeView shape, const void* src,
		                        ShapeView permutation)
		{
			const auto e = Detail::Extents(shape), p = Detail::Extents(permutation);
			Detail::HIPCheck(litenn_hip_permute(device.deviceIndex, dst, static_cast<int>(type), e.data(), e.size(), src,
			                                    p.data(), nullptr));
		}

		// ---- extensions: the quantised path (no counterpart in the reference's traits) ----------

		// y[m, n] = x[m, k] . deq(wq)[n, k]^T (+ residual); wq is the raw GGUF payload the importer keeps
		// (tools/gguf/GGUFImporter.cpp:487-489), i.e. what AddLinear computes after the lowering's
		// dequantise + transpose (tools/gguf/LLaMABuilder.cpp:144-150,225-230)
		static void DoQuantizedMatMul(HIP& device, QuantizedBlockFormat format, const void* wq, std::size_t n,
		                              std::size_t k, const void* x, std::size_t m, void* y,
		                              const void* residual = nullptr, bool preciseActivations = false,
		                              const HIPExecutionOptions& options = {})
		{
			const litenn_hip_exec e = Detail::Exec(options);
			Detail::HIPCheck(litenn_hip_mul_mat_q(device.deviceIndex, static_cast<int>(format), wq, n, k, x,
			                                      static_cast<int>(DataType::Float32), m, y, residual,
			                                      preciseActivations ? LITENN_HIP_MATMUL_PRECISE : 0u, &e));
		}
		static void DoDequantize(HIP& device, QuantizedBlockFormat format, const void* wq, std::size_t rows,
		                         std::size_t k, void* dst)
		{
			Detail::HIPCheck(
			    litenn_hip_dequantize(device.deviceIndex, static_cast<int>(format), wq, rows, k, dst, nullptr));
		}
		static void DoRMSNorm(HIP& device, const void* x, const void* weight, double epsilon, std::size_t rows,
		                      std::size_t width, void* y)
		{
			Detail::HIPCheck(litenn_hip_rmsnorm(device.deviceIndex, x, weight, epsilon, rows, width, y, nullptr));
		}
	};
} // namespace LiteNN

#endif
