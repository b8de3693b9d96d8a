// Exercises LiteNN::DeviceTraits<LiteNN::HIP> (include/LiteNN/Device/HIP.h) the way the reference's
// device tests exercise DeviceTraits<CUDA> (tests/CUDADeviceTest.cpp:69-125): allocate, copy,
// element-wise ops, MatMul, reduce, error text -- plus the quantised matmul on the reference's own
// 18-byte Q4_0 payload fixture (tests/GGUFImporterTest.cpp:173-178).
//
// Exit status: 0 = every check passed (or no device: only the device-free checks ran),
// 1 = a check failed.  Prints one line per check.
#include <LiteNN/Device/HIP.h>

#include <cmath>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

using namespace LiteNN;
using Traits = DeviceTraits<HIP>;

static int g_failed = 0;

static void Check(bool ok, const char* what)
{
	std::printf("%s %s\n", ok ? "ok  " : "FAIL", what);
	if (!ok)
	{
		++g_failed;
	}
}

template <typename T>
static void* Upload(HIP& dev, DataType type, const std::vector<T>& host)
{
	void* p = Traits::Allocate(dev, type, host.size());
	Traits::CopyFromCPU(dev, type, p, type, host.data(), host.size());
	return p;
}

static std::vector<float> Download(HIP& dev, const void* p, std::size_t n)
{
	std::vector<float> host(n);
	Traits::CopyToCPU(dev, DataType::Float32, p, n, DataType::Float32, host.data());
	return host;
}

int main()
{
	HIP dev{ 0 };
	Check(Traits::Name() == "HIP", "Name() is HIP");
	Check(HIPDeviceCount() >= 0, "HIPDeviceCount() never fails");

	// argument validation is reported as an exception carrying the library's message, device or not
	try
	{
		Traits::DoQuantizedMatMul(dev, static_cast<QuantizedBlockFormat>(6), nullptr, 4, 32, nullptr, 1, nullptr); // Q8_1: no dequantizer
		Check(false, "unsupported block format throws");
	}
	catch (const std::runtime_error& e)
	{
		Check(std::strstr(e.what(), "HIP quantized matmul failed: unsupported block format") != nullptr,
		      "unsupported block format throws '<action> failed: <message>'");
	}

	if (!IsHIPDeviceAvailable(0))
	{
		try
		{
			(void)Traits::Allocate(dev, DataType::Float32, 16);
			Check(false, "Allocate without a device throws");
		}
		catch (const std::runtime_error& e)
		{
			Check(std::strstr(e.what(), "HIP allocate failed") != nullptr, "Allocate without a device throws");
		}
		std::printf("no HIP device: device checks skipped\n");
		return g_failed ? 1 : 0;
	}

	std::printf("%s\n", std::string(Traits::Info(dev)).c_str());

	// tests/CUDADeviceTest.cpp:108-125: [[1,2,3],[4,5,6]] . transpose = [[14,32],[32,77]]
	{
		const std::vector<float> a = { 1, 2, 3, 4, 5, 6 };
		void* da = Upload(dev, DataType::Float32, a);
		void* dt = Traits::Allocate(dev, DataType::Float32, 6);
		void* dc = Traits::Allocate(dev, DataType::Float32, 4);
		Traits::DoUnaryOp(dev, UnaryOp::Transpose, dt, DataType::Float32, { 2, 3 }, da);
		Traits::DoBinaryOp(dev, BinaryOp::MatMul, dc, DataType::Float32, { 2, 3 }, da, DataType::Float32, { 3, 2 }, dt);
		const auto c = Download(dev, dc, 4);
		Check(c == std::vector<float>({ 14, 32, 32, 77 }), "MatMul reference vector");

		void* dn = Traits::Allocate(dev, DataType::Float32, 6);
		Traits::DoUnaryOp(dev, UnaryOp::Negate, dn, DataType::Float32, { 2, 3 }, da);
		Check(Download(dev, dn, 6) == std::vector<float>({ -1, -2, -3, -4, -5, -6 }), "Negate");

		void* ds = Traits::Allocate(dev, DataType::Float32, 2);
		Traits::DoReduceOp(dev, ReduceOp::Sum, ds, DataType::Float32, { 2, 3 }, da, 1);
		Check(Download(dev, ds, 2) == std::vector<float>({ 6, 15 }), "Reduce Sum over the last axis");

		Traits::ZeroFill(dev, dn, DataType::Float32, 6);
		Check(Download(dev, dn, 6) == std::vector<float>(6, 0.0f), "ZeroFill");

		// dtype-changing copy: f32 -> f64 on the way back
		std::vector<double> wide(6);
		Traits::CopyToCPU(dev, DataType::Float32, da, 6, DataType::Float64, wide.data());
		Check(wide == std::vector<double>({ 1, 2, 3, 4, 5, 6 }), "CopyToCPU widens Float32 to Float64");

		Traits::Deallocate(dev, da, DataType::Float32, 6);
		Traits::Deallocate(dev, dt, DataType::Float32, 6);
		Traits::Deallocate(dev, dc, DataType::Float32, 4);
		Traits::Deallocate(dev, dn, DataType::Float32, 6);
		Traits::Deallocate(dev, ds, DataType::Float32, 2);
	}

	// the reference's Q4_0 payload fixture: d = fp16 0x0010 = 2^-20, then 16 nibble bytes
	{
		const std::vector<uint8_t> block = { 0x10, 0x00, 0x22, 0x44, 0x66, 0x88, 0xaa, 0xcc, 0xee, 0x11, 0x33,
			                                 0x55, 0x77, 0x99, 0xbb, 0xdd, 0xff, 0x7f };
		std::vector<float> x(32);
		for (int i = 0; i < 32; ++i)
		{
			x[i] = 0.25f * static_cast<float>(i + 1);
		}
		const double d = std::ldexp(1.0, -20);
		double want = 0.0;
		std::vector<float> deq(32);
		for (int j = 0; j < 16; ++j)
		{
			deq[j] = static_cast<float>(((block[2 + j] & 15) - 8) * d);
			deq[j + 16] = static_cast<float>(((block[2 + j] >> 4) - 8) * d);
		}
		for (int i = 0; i < 32; ++i)
		{
			want += static_cast<double>(deq[i]) * x[i];
		}
		void* dw = Upload(dev, DataType::UInt8, block);
		void* dx = Upload(dev, DataType::Float32, x);
		void* dy = Traits::Allocate(dev, DataType::Float32, 1);
		Traits::DoQuantizedMatMul(dev, QuantizedBlockFormat::Q4_0, dw, 1, 32, dx, 1, dy);
		const float got = Download(dev, dy, 1)[0];
		Check(std::fabs(got - want) <= 1e-6 * std::fabs(want), "Q4_0 fixture block . x (closed form)");

		void* dd = Traits::Allocate(dev, DataType::Float32, 32);
		Traits::DoDequantize(dev, QuantizedBlockFormat::Q4_0, dw, 1, 32, dd);
		Check(Download(dev, dd, 32) == deq, "Q4_0 fixture block dequantised (closed form, exact)");

		Traits::Deallocate(dev, dw, DataType::UInt8, block.size());
		Traits::Deallocate(dev, dx, DataType::Float32, 32);
		Traits::Deallocate(dev, dy, DataType::Float32, 1);
		Traits::Deallocate(dev, dd, DataType::Float32, 32);
	}

	// RMSNorm closed form: x = [3, 4], w = [1, 2], eps = 0 -> x / sqrt(12.5) * w
	{
		void* dx = Upload(dev, DataType::Float32, std::vector<float>{ 3, 4 });
		void* dw = Upload(dev, DataType::Float32, std::vector<float>{ 1, 2 });
		void* dy = Traits::Allocate(dev, DataType::Float32, 2);
		Traits::DoRMSNorm(dev, dx, dw, 0.0, 1, 2, dy);
		const auto y = Download(dev, dy, 2);
		const double r = 1.0 / std::sqrt(12.5);
		Check(std::fabs(y[0] - 3 * r) < 1e-6 && std::fabs(y[1] - 8 * r) < 1e-6, "RMSNorm closed form");
		Traits::Deallocate(dev, dx, DataType::Float32, 2);
		Traits::Deallocate(dev, dw, DataType::Float32, 2);
		Traits::Deallocate(dev, dy, DataType::Float32, 2);
	}

	std::printf(g_failed ? "%d check(s) FAILED\n" : "all checks passed\n", g_failed);
	return g_failed ? 1 : 0;
}
