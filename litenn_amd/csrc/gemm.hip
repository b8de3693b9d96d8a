// placeholder replaced below
#include "common.hpp"
namespace litenn_hip
{
	int launch_gemv(int fmt, const void* wq, size_t n, size_t k, const float* x, size_t m, float* y,
	                const float* residual, hipStream_t stream);
	int launch_gemm(int fmt, const void* wq, size_t n, size_t k, const float* x, size_t m, float* y,
	                const float* residual, hipStream_t stream)
	{
		return launch_gemv(fmt, wq, n, k, x, m, y, residual, stream);
	}
}
