/*
 * litenn_oracle.c -- CPU restatement of LiteNN's CPU path for GGUF-quantised
 * LLaMA inference.  TEST INFRASTRUCTURE ONLY: see litenn_oracle.h.
 *
 * Build with -ffp-contract=off and without -ffast-math: every multiply and add
 * below is meant to round separately, as the reference's scalar f32 loops do
 * on a baseline x86-64 build.
 */
#include "litenn_oracle.h"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

static __thread char g_err[256];

const char* oracle_last_error(void)
{
	return g_err;
}

static int fail(const char* msg)
{
	snprintf(g_err, sizeof g_err, "%s", msg);
	return -1;
}

void oracle_set_threads(int n)
{
#ifdef _OPENMP
	if (n > 0)
	{
		omp_set_num_threads(n);
	}
#else
	(void)n;
#endif
}

/* ---------------------------------------------------------------------- */
/* Float16, src/LiteNN/DType.h:63-134                                      */
/* ---------------------------------------------------------------------- */

static inline uint32_t f32_bits(float v)
{
	uint32_t b;
	memcpy(&b, &v, 4);
	return b;
}

static inline float bits_f32(uint32_t b)
{
	float v;
	memcpy(&v, &b, 4);
	return v;
}

/* DType.h:112-134.  The reference builds the value with ldexp of an exactly
 * representable fraction, so the result is the exact IEEE binary16 value. */
float oracle_f16_to_f32(uint16_t bits)
{
	const float sign = (bits & 0x8000u) ? -1.0f : 1.0f;
	const int exponent = (int)((bits >> 10) & 0x1fu);
	const uint32_t mantissa = (uint32_t)(bits & 0x03ffu);
	if (exponent == 0)
	{
		if (mantissa == 0)
		{
			return sign * 0.0f;
		}
		return sign * ldexpf((float)mantissa / 1024.0f, -14);
	}
	if (exponent == 0x1f)
	{
		if (mantissa == 0)
		{
			return sign * INFINITY;
		}
		return NAN;
	}
	return sign * ldexpf(1.0f + (float)mantissa / 1024.0f, exponent - 15);
}

/* DType.h:63-110.  Rounds to nearest with ties going UP in magnitude (it tests
 * only the first dropped bit), unlike IEEE round-to-nearest-even. */
uint16_t oracle_f32_to_f16(float value)
{
	const uint32_t bits = f32_bits(value);
	const uint16_t sign = (uint16_t)((bits >> 16) & 0x8000u);
	const int exponent = (int)((bits >> 23) & 0xffu) - 127;
	uint32_t mantissa = bits & 0x7fffffu;

	if ((bits & 0x7fffffffu) == 0)
	{
		return sign;
	}
	if (((bits >> 23) & 0xffu) == 0xffu)
	{
		return (uint16_t)(sign | 0x7c00u | (mantissa ? 0x0200u : 0u));
	}
	if (exponent > 15)
	{
		return (uint16_t)(sign | 0x7c00u);
	}
	if (exponent < -14)
	{
		if (exponent < -24)
		{
			return sign;
		}
		mantissa |= 0x800000u;
		const uint32_t shift = (uint32_t)(-exponent - 14 + 13);
		uint16_t half_mantissa = (uint16_t)(mantissa >> shift);
		const uint32_t round_bit = 1u << (shift - 1);
		if ((mantissa & round_bit) != 0)
		{
			++half_mantissa;
		}
		return (uint16_t)(sign | half_mantissa);
	}

	uint16_t half_exponent = (uint16_t)((exponent + 15) << 10);
	uint16_t half_mantissa = (uint16_t)(mantissa >> 13);
	if ((mantissa & 0x1000u) != 0)
	{
		++half_mantissa;
		if ((half_mantissa & 0x0400u) != 0)
		{
			half_mantissa = 0;
			half_exponent = (uint16_t)(half_exponent + 0x0400u);
			if (half_exponent >= 0x7c00u)
			{
				half_exponent = 0x7c00u;
			}
		}
	}
	return (uint16_t)(sign | half_exponent | half_mantissa);
}

void oracle_f16_to_f32_array(const uint16_t* src, float* dst, size_t n)
{
	for (size_t i = 0; i < n; ++i)
	{
		dst[i] = oracle_f16_to_f32(src[i]);
	}
}

void oracle_f32_to_f16_array(const float* src, uint16_t* dst, size_t n)
{
	for (size_t i = 0; i < n; ++i)
	{
		dst[i] = oracle_f32_to_f16(src[i]);
	}
}

/* ---------------------------------------------------------------------- */
/* Block formats, src/LiteNN/Quantization.h:186-217                        */
/* ---------------------------------------------------------------------- */

int oracle_block_elements(int fmt)
{
	switch (fmt)
	{
	case ORACLE_FMT_Q4_0:
	case ORACLE_FMT_Q4_1:
	case ORACLE_FMT_Q5_0:
	case ORACLE_FMT_Q5_1:
	case ORACLE_FMT_Q8_0:
		return 32;
	case ORACLE_FMT_Q2_K:
	case ORACLE_FMT_Q3_K:
	case ORACLE_FMT_Q4_K:
	case ORACLE_FMT_Q5_K:
	case ORACLE_FMT_Q6_K:
		return 256;
	case ORACLE_FMT_F16:
	case ORACLE_FMT_F32:
		return 1;
	default:
		return 0;
	}
}

int oracle_block_bytes(int fmt)
{
	switch (fmt)
	{
	case ORACLE_FMT_Q4_0:
		return 18;
	case ORACLE_FMT_Q4_1:
		return 20;
	case ORACLE_FMT_Q5_0:
		return 22;
	case ORACLE_FMT_Q5_1:
		return 24;
	case ORACLE_FMT_Q8_0:
		return 34;
	case ORACLE_FMT_Q2_K:
		return 84;
	case ORACLE_FMT_Q3_K:
		return 110;
	case ORACLE_FMT_Q4_K:
		return 144;
	case ORACLE_FMT_Q5_K:
		return 176;
	case ORACLE_FMT_Q6_K:
		return 210;
	case ORACLE_FMT_F16:
		return 2;
	case ORACLE_FMT_F32:
		return 4;
	default:
		return 0;
	}
}

size_t oracle_row_bytes(int fmt, size_t k)
{
	const int be = oracle_block_elements(fmt);
	if (be == 0 || k % (size_t)be != 0)
	{
		return 0;
	}
	return k / (size_t)be * (size_t)oracle_block_bytes(fmt);
}

static inline uint16_t load_u16(const uint8_t* p)
{
	return (uint16_t)(p[0] | ((uint16_t)p[1] << 8));
}

/* ggml block_q4_0 { fp16 d; u8 qs[16]; }: dequantize_row_q4_0 */
static void dequant_q4_0(const uint8_t* src, float* y, size_t k)
{
	const size_t nb = k / 32;
	for (size_t i = 0; i < nb; ++i)
	{
		const uint8_t* b = src + i * 18;
		const float d = oracle_f16_to_f32(load_u16(b));
		const uint8_t* qs = b + 2;
		for (int j = 0; j < 16; ++j)
		{
			const int x0 = (qs[j] & 0x0F) - 8;
			const int x1 = (qs[j] >> 4) - 8;
			y[i * 32 + j] = (float)x0 * d;
			y[i * 32 + j + 16] = (float)x1 * d;
		}
	}
}

/* ggml block_q4_1 { fp16 d; fp16 m; u8 qs[16]; }: dequantize_row_q4_1 */
static void dequant_q4_1(const uint8_t* src, float* y, size_t k)
{
	const size_t nb = k / 32;
	for (size_t i = 0; i < nb; ++i)
	{
		const uint8_t* b = src + i * 20;
		const float d = oracle_f16_to_f32(load_u16(b));
		const float m = oracle_f16_to_f32(load_u16(b + 2));
		const uint8_t* qs = b + 4;
		for (int j = 0; j < 16; ++j)
		{
			const int x0 = qs[j] & 0x0F;
			const int x1 = qs[j] >> 4;
			y[i * 32 + j] = (float)x0 * d + m;
			y[i * 32 + j + 16] = (float)x1 * d + m;
		}
	}
}

/* the fifth bits of a 32-element block: bit j of the little-endian u32 qh belongs to element j */
static inline uint32_t load_u32(const uint8_t* p)
{
	return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
}

/* ggml block_q5_0 { fp16 d; u8 qh[4]; u8 qs[16]; }: dequantize_row_q5_0 */
static void dequant_q5_0(const uint8_t* src, float* y, size_t k)
{
	const size_t nb = k / 32;
	for (size_t i = 0; i < nb; ++i)
	{
		const uint8_t* b = src + i * 22;
		const float d = oracle_f16_to_f32(load_u16(b));
		const uint32_t qh = load_u32(b + 2);
		const uint8_t* qs = b + 6;
		for (int j = 0; j < 16; ++j)
		{
			const uint8_t xh_0 = (uint8_t)(((qh >> (j + 0)) << 4) & 0x10);
			const uint8_t xh_1 = (uint8_t)((qh >> (j + 12)) & 0x10);
			const int x0 = ((qs[j] & 0x0F) | xh_0) - 16;
			const int x1 = ((qs[j] >> 4) | xh_1) - 16;
			y[i * 32 + j] = (float)x0 * d;
			y[i * 32 + j + 16] = (float)x1 * d;
		}
	}
}

/* ggml block_q5_1 { fp16 d; fp16 m; u8 qh[4]; u8 qs[16]; }: dequantize_row_q5_1 */
static void dequant_q5_1(const uint8_t* src, float* y, size_t k)
{
	const size_t nb = k / 32;
	for (size_t i = 0; i < nb; ++i)
	{
		const uint8_t* b = src + i * 24;
		const float d = oracle_f16_to_f32(load_u16(b));
		const float m = oracle_f16_to_f32(load_u16(b + 2));
		const uint32_t qh = load_u32(b + 4);
		const uint8_t* qs = b + 8;
		for (int j = 0; j < 16; ++j)
		{
			const uint8_t xh_0 = (uint8_t)(((qh >> (j + 0)) << 4) & 0x10);
			const uint8_t xh_1 = (uint8_t)((qh >> (j + 12)) & 0x10);
			const int x0 = (qs[j] & 0x0F) | xh_0;
			const int x1 = (qs[j] >> 4) | xh_1;
			y[i * 32 + j] = (float)x0 * d + m;
			y[i * 32 + j + 16] = (float)x1 * d + m;
		}
	}
}

/* ggml block_q8_0 { fp16 d; i8 qs[32]; }: dequantize_row_q8_0 */
static void dequant_q8_0(const uint8_t* src, float* y, size_t k)
{
	const size_t nb = k / 32;
	for (size_t i = 0; i < nb; ++i)
	{
		const uint8_t* b = src + i * 34;
		const float d = oracle_f16_to_f32(load_u16(b));
		const int8_t* qs = (const int8_t*)(b + 2);
		for (int j = 0; j < 32; ++j)
		{
			y[i * 32 + j] = (float)qs[j] * d;
		}
	}
}

/* ggml get_scale_min_k4 */
static inline void scale_min_k4(int j, const uint8_t* q, uint8_t* sc, uint8_t* mn)
{
	if (j < 4)
	{
		*sc = q[j] & 63;
		*mn = q[j + 4] & 63;
	}
	else
	{
		*sc = (uint8_t)((q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4));
		*mn = (uint8_t)((q[j + 4] >> 4) | ((q[j - 0] >> 6) << 4));
	}
}

/* ggml block_q2_K { u8 scales[16]; u8 qs[64]; fp16 d; fp16 dmin; }: dequantize_row_q2_K */
static void dequant_q2_k(const uint8_t* src, float* y, size_t k)
{
	const size_t nb = k / 256;
	for (size_t i = 0; i < nb; ++i)
	{
		const uint8_t* b = src + i * 84;
		const uint8_t* scales = b;
		const uint8_t* q = b + 16;
		const float d = oracle_f16_to_f32(load_u16(b + 80));
		const float dmin = oracle_f16_to_f32(load_u16(b + 82));
		int is = 0;
		for (int n = 0; n < 256; n += 128)
		{
			int shift = 0;
			for (int j = 0; j < 4; ++j)
			{
				uint8_t sc = scales[is++];
				float dl = d * (float)(sc & 0xF), ml = dmin * (float)(sc >> 4);
				for (int l = 0; l < 16; ++l)
				{
					*y++ = dl * (float)((int8_t)((q[l] >> shift) & 3)) - ml;
				}
				sc = scales[is++];
				dl = d * (float)(sc & 0xF);
				ml = dmin * (float)(sc >> 4);
				for (int l = 0; l < 16; ++l)
				{
					*y++ = dl * (float)((int8_t)((q[l + 16] >> shift) & 3)) - ml;
				}
				shift += 2;
			}
			q += 32;
		}
	}
}

/* ggml block_q3_K { u8 hmask[32]; u8 qs[64]; u8 scales[12]; fp16 d; }: dequantize_row_q3_K */
static void dequant_q3_k(const uint8_t* src, float* y, size_t k)
{
	const uint32_t kmask1 = 0x03030303u, kmask2 = 0x0f0f0f0fu;
	const size_t nb = k / 256;
	for (size_t i = 0; i < nb; ++i)
	{
		const uint8_t* b = src + i * 110;
		const uint8_t* hm = b;
		const uint8_t* q = b + 32;
		const float d_all = oracle_f16_to_f32(load_u16(b + 108));
		uint32_t aux[4];
		aux[0] = load_u32(b + 96);
		aux[1] = load_u32(b + 100);
		aux[2] = load_u32(b + 104);
		const uint32_t tmp = aux[2];
		aux[2] = ((aux[0] >> 4) & kmask2) | (((tmp >> 4) & kmask1) << 4);
		aux[3] = ((aux[1] >> 4) & kmask2) | (((tmp >> 6) & kmask1) << 4);
		aux[0] = (aux[0] & kmask2) | (((tmp >> 0) & kmask1) << 4);
		aux[1] = (aux[1] & kmask2) | (((tmp >> 2) & kmask1) << 4);
		int8_t scales[16];
		for (int s = 0; s < 16; ++s)
		{
			scales[s] = (int8_t)((aux[s / 4] >> (8 * (s % 4))) & 0xff);
		}
		int is = 0;
		uint8_t m = 1;
		for (int n = 0; n < 256; n += 128)
		{
			int shift = 0;
			for (int j = 0; j < 4; ++j)
			{
				float dl = d_all * (float)(scales[is++] - 32);
				for (int l = 0; l < 16; ++l)
				{
					*y++ = dl * (float)((int8_t)((q[l + 0] >> shift) & 3) - ((hm[l + 0] & m) ? 0 : 4));
				}
				dl = d_all * (float)(scales[is++] - 32);
				for (int l = 0; l < 16; ++l)
				{
					*y++ = dl * (float)((int8_t)((q[l + 16] >> shift) & 3) - ((hm[l + 16] & m) ? 0 : 4));
				}
				shift += 2;
				m = (uint8_t)(m << 1);
			}
			q += 32;
		}
	}
}

/* ggml block_q5_K { fp16 d; fp16 dmin; u8 scales[12]; u8 qh[32]; u8 qs[128]; }: dequantize_row_q5_K */
static void dequant_q5_k(const uint8_t* src, float* y, size_t k)
{
	const size_t nb = k / 256;
	for (size_t i = 0; i < nb; ++i)
	{
		const uint8_t* b = src + i * 176;
		const float d = oracle_f16_to_f32(load_u16(b));
		const float dmin = oracle_f16_to_f32(load_u16(b + 2));
		const uint8_t* scales = b + 4;
		const uint8_t* qh = b + 16;
		const uint8_t* ql = b + 48;
		int is = 0;
		uint8_t u1 = 1, u2 = 2;
		for (int j = 0; j < 256; j += 64)
		{
			uint8_t sc, mn;
			scale_min_k4(is + 0, scales, &sc, &mn);
			const float d1 = d * (float)sc;
			const float m1 = dmin * (float)mn;
			scale_min_k4(is + 1, scales, &sc, &mn);
			const float d2 = d * (float)sc;
			const float m2 = dmin * (float)mn;
			for (int l = 0; l < 32; ++l)
			{
				*y++ = d1 * (float)((ql[l] & 0xF) + ((qh[l] & u1) ? 16 : 0)) - m1;
			}
			for (int l = 0; l < 32; ++l)
			{
				*y++ = d2 * (float)((ql[l] >> 4) + ((qh[l] & u2) ? 16 : 0)) - m2;
			}
			ql += 32;
			is += 2;
			u1 = (uint8_t)(u1 << 2);
			u2 = (uint8_t)(u2 << 2);
		}
	}
}

/* ggml block_q4_K { fp16 d; fp16 dmin; u8 scales[12]; u8 qs[128]; }: dequantize_row_q4_K */
static void dequant_q4_k(const uint8_t* src, float* y, size_t k)
{
	const size_t nb = k / 256;
	for (size_t i = 0; i < nb; ++i)
	{
		const uint8_t* b = src + i * 144;
		const float d = oracle_f16_to_f32(load_u16(b));
		const float dmin = oracle_f16_to_f32(load_u16(b + 2));
		const uint8_t* scales = b + 4;
		const uint8_t* q = b + 16;
		int is = 0;
		for (int j = 0; j < 256; j += 64)
		{
			uint8_t sc, mn;
			scale_min_k4(is + 0, scales, &sc, &mn);
			const float d1 = d * (float)sc;
			const float m1 = dmin * (float)mn;
			scale_min_k4(is + 1, scales, &sc, &mn);
			const float d2 = d * (float)sc;
			const float m2 = dmin * (float)mn;
			for (int l = 0; l < 32; ++l)
			{
				*y++ = d1 * (float)(q[l] & 0xF) - m1;
			}
			for (int l = 0; l < 32; ++l)
			{
				*y++ = d2 * (float)(q[l] >> 4) - m2;
			}
			q += 32;
			is += 2;
		}
	}
}

/* ggml block_q6_K { u8 ql[128]; u8 qh[64]; i8 scales[16]; fp16 d; }: dequantize_row_q6_K */
static void dequant_q6_k(const uint8_t* src, float* y, size_t k)
{
	const size_t nb = k / 256;
	for (size_t i = 0; i < nb; ++i)
	{
		const uint8_t* b = src + i * 210;
		const uint8_t* ql = b;
		const uint8_t* qh = b + 128;
		const int8_t* sc = (const int8_t*)(b + 192);
		const float d = oracle_f16_to_f32(load_u16(b + 208));
		for (int n = 0; n < 256; n += 128)
		{
			for (int l = 0; l < 32; ++l)
			{
				const int is = l / 16;
				const int8_t q1 = (int8_t)((ql[l + 0] & 0xF) | (((qh[l] >> 0) & 3) << 4)) - 32;
				const int8_t q2 = (int8_t)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32;
				const int8_t q3 = (int8_t)((ql[l + 0] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
				const int8_t q4 = (int8_t)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
				y[l + 0] = d * (float)sc[is + 0] * (float)q1;
				y[l + 32] = d * (float)sc[is + 2] * (float)q2;
				y[l + 64] = d * (float)sc[is + 4] * (float)q3;
				y[l + 96] = d * (float)sc[is + 6] * (float)q4;
			}
			y += 128;
			ql += 64;
			qh += 32;
			sc += 8;
		}
	}
}

int oracle_dequantize_row(int fmt, const uint8_t* src, float* dst, size_t k)
{
	const int be = oracle_block_elements(fmt);
	if (be == 0)
	{
		return fail("unsupported block format");
	}
	if (k % (size_t)be != 0)
	{
		return fail("row width is not a whole number of blocks");
	}
	switch (fmt)
	{
	case ORACLE_FMT_Q4_0:
		dequant_q4_0(src, dst, k);
		break;
	case ORACLE_FMT_Q4_1:
		dequant_q4_1(src, dst, k);
		break;
	case ORACLE_FMT_Q5_0:
		dequant_q5_0(src, dst, k);
		break;
	case ORACLE_FMT_Q5_1:
		dequant_q5_1(src, dst, k);
		break;
	case ORACLE_FMT_Q8_0:
		dequant_q8_0(src, dst, k);
		break;
	case ORACLE_FMT_Q2_K:
		dequant_q2_k(src, dst, k);
		break;
	case ORACLE_FMT_Q3_K:
		dequant_q3_k(src, dst, k);
		break;
	case ORACLE_FMT_Q4_K:
		dequant_q4_k(src, dst, k);
		break;
	case ORACLE_FMT_Q5_K:
		dequant_q5_k(src, dst, k);
		break;
	case ORACLE_FMT_Q6_K:
		dequant_q6_k(src, dst, k);
		break;
	case ORACLE_FMT_F16:
		for (size_t i = 0; i < k; ++i)
		{
			dst[i] = oracle_f16_to_f32(load_u16(src + 2 * i));
		}
		break;
	case ORACLE_FMT_F32:
		memcpy(dst, src, 4 * k);
		break;
	default:
		return fail("unsupported block format");
	}
	return 0;
}

int oracle_dequantize(int fmt, const uint8_t* src, float* dst, size_t rows, size_t k)
{
	const size_t rb = oracle_row_bytes(fmt, k);
	if (rb == 0)
	{
		return fail("bad format or row width");
	}
	for (size_t r = 0; r < rows; ++r)
	{
		if (oracle_dequantize_row(fmt, src + r * rb, dst + r * k, k) != 0)
		{
			return -1;
		}
	}
	return 0;
}

/* ---------------------------------------------------------------------- */
/* Dense primitives                                                        */
/* ---------------------------------------------------------------------- */

/* Device.h:500-511 */
void oracle_transpose(const float* src, float* dst, size_t rows, size_t cols)
{
	for (size_t r = 0; r < rows; ++r)
	{
		for (size_t c = 0; c < cols; ++c)
		{
			dst[c * rows + r] = src[r * cols + c];
		}
	}
}

/* Device.h:645-658 */
void oracle_matmul_ikj(const float* x, const float* w, float* y, size_t m, size_t k, size_t n)
{
	for (size_t e = 0; e < m * n; ++e)
	{
		y[e] = 0.0f;
	}
	for (size_t i = 0; i < m; ++i)
	{
		float* out_row = y + i * n;
		for (size_t kk = 0; kk < k; ++kk)
		{
			const float lhs = x[i * k + kk];
			const float* rhs_row = w + kk * n;
			for (size_t j = 0; j < n; ++j)
			{
				out_row[j] += lhs * rhs_row[j];
			}
		}
	}
}

int oracle_mul_mat_q(int fmt, const uint8_t* wq, size_t n, size_t k, const float* x, size_t m, float* y)
{
	if (oracle_row_bytes(fmt, k) == 0)
	{
		return fail("bad format or row width");
	}
	float* deq = (float*)malloc(sizeof(float) * n * k);
	float* wt = (float*)malloc(sizeof(float) * n * k);
	if (!deq || !wt)
	{
		free(deq);
		free(wt);
		return fail("out of memory");
	}
	int rc = oracle_dequantize(fmt, wq, deq, n, k); /* LLaMABuilder.cpp:144-150 */
	if (rc == 0)
	{
		oracle_transpose(deq, wt, n, k);        /* LLaMABuilder.cpp:225-230 */
		oracle_matmul_ikj(x, wt, y, m, k, n);   /* Device.h:645-658 */
	}
	free(deq);
	free(wt);
	return rc;
}

#define JB 8

/* acc[jj] += x[kk] * wt[kk][jj] for kk ascending: per output column the same
 * sequence of f32 multiplies and adds as the i-k-j loop. */
__attribute__((target_clones("avx2", "default"))) static void dot_block(const float* x, const float* wt, size_t k,
                                                                         float* acc)
{
	float a[JB];
	for (int jj = 0; jj < JB; ++jj)
	{
		a[jj] = 0.0f;
	}
	for (size_t kk = 0; kk < k; ++kk)
	{
		const float xv = x[kk];
		const float* w = wt + kk * JB;
		for (int jj = 0; jj < JB; ++jj)
		{
			a[jj] += xv * w[jj];
		}
	}
	for (int jj = 0; jj < JB; ++jj)
	{
		acc[jj] = a[jj];
	}
}

int oracle_mul_mat_q_rowwise(int fmt, const uint8_t* wq, size_t n, size_t k, const float* x, size_t m, float* y)
{
	const size_t rb = oracle_row_bytes(fmt, k);
	if (rb == 0)
	{
		return fail("bad format or row width");
	}
	const size_t nblk = (n + JB - 1) / JB;
	int bad = 0;
#pragma omp parallel
	{
		float* row = (float*)malloc(sizeof(float) * k);
		float* wt = (float*)malloc(sizeof(float) * k * JB);
		if (!row || !wt)
		{
#pragma omp atomic write
			bad = 1;
		}
		else
		{
#pragma omp for schedule(static)
			for (size_t b = 0; b < nblk; ++b)
			{
				const size_t j0 = b * JB;
				const size_t jn = (n - j0 < JB) ? (n - j0) : JB;
				for (size_t jj = 0; jj < JB; ++jj)
				{
					if (jj < jn)
					{
						oracle_dequantize_row(fmt, wq + (j0 + jj) * rb, row, k);
						for (size_t kk = 0; kk < k; ++kk)
						{
							wt[kk * JB + jj] = row[kk];
						}
					}
					else
					{
						for (size_t kk = 0; kk < k; ++kk)
						{
							wt[kk * JB + jj] = 0.0f;
						}
					}
				}
				for (size_t i = 0; i < m; ++i)
				{
					float acc[JB];
					dot_block(x + i * k, wt, k, acc);
					for (size_t jj = 0; jj < jn; ++jj)
					{
						y[i * n + j0 + jj] = acc[jj];
					}
				}
			}
		}
		free(row);
		free(wt);
	}
	return bad ? fail("out of memory") : 0;
}

/* ComputePrimitives.h:792-817 (RMSNorm branch, axis = last) */
void oracle_rmsnorm(const float* x, const float* w, double eps, size_t m, size_t d, float* y)
{
	for (size_t o = 0; o < m; ++o)
	{
		double variance = 0.0;
		for (size_t a = 0; a < d; ++a)
		{
			const double raw = (double)x[o * d + a];
			variance += raw * raw;
		}
		variance /= (double)d;
		const double denom = sqrt(variance + eps);
		for (size_t a = 0; a < d; ++a)
		{
			double value = (double)x[o * d + a] / denom;
			if (w)
			{
				value *= (double)w[a]; /* scale [1,d] broadcast over rows */
			}
			y[o * d + a] = (float)value;
		}
	}
}

/* RoPE.h:24-41 (tables in double, stored as f32), :75-116 (f32 rotation) */
void oracle_rope(const float* x, float* y, size_t m, size_t d, size_t rope_dims, double base, double freq_scale,
                 size_t pos_offset)
{
	const size_t half = rope_dims / 2;
	for (size_t pos = 0; pos < m; ++pos)
	{
		const float* in = x + pos * d;
		float* out = y + pos * d;
		for (size_t dim = 0; dim < half; ++dim)
		{
			const double exponent = -2.0 * (double)dim / (double)(half * 2);
			const double inv_freq = pow(base, exponent);
			const double angle = (double)(pos_offset + pos) * inv_freq * freq_scale;
			const float c = (float)cos(angle);
			const float s = (float)sin(angle);
			const float first = in[2 * dim];
			const float second = in[2 * dim + 1];
			const float first_cos = first * c;
			const float second_sin = second * s;
			const float first_sin = first * s;
			const float second_cos = second * c;
			out[2 * dim] = first_cos - second_sin;
			out[2 * dim + 1] = first_sin + second_cos;
		}
		for (size_t t = rope_dims; t < d; ++t)
		{
			out[t] = in[t]; /* LLaMABuilder.cpp:340-347 un-rotated tail */
		}
	}
}

/* FlashAttnExt.h:126-228 with mask/softcap/sinks absent */
void oracle_attention_head(const float* q, size_t mq, const float* k, const float* v, size_t l, size_t d, size_t dv,
                           double scale, int causal, size_t key_pos_offset, size_t query_pos_offset, float* out)
{
	float* s = (float*)malloc(sizeof(float) * (l ? l : 1));
	const float scale_f = (float)scale;        /* MakeScalarTensor(f32, scale) */
	const float masked = (float)-1.0e9;        /* CausalMask.h:16-34 */
	for (size_t row = 0; row < mq; ++row)
	{
		/* scores = q . K^T through the i-k-j MatMul: per (row, col) a k-ascending sum */
		for (size_t col = 0; col < l; ++col)
		{
			s[col] = 0.0f;
		}
		for (size_t kk = 0; kk < d; ++kk)
		{
			const float lhs = q[row * d + kk];
			for (size_t col = 0; col < l; ++col)
			{
				s[col] += lhs * k[col * d + kk];
			}
		}
		if (scale != 1.0)
		{
			for (size_t col = 0; col < l; ++col)
			{
				s[col] = s[col] * scale_f;
			}
		}
		if (causal)
		{
			for (size_t col = 0; col < l; ++col)
			{
				const float mask = (key_pos_offset + col > query_pos_offset + row) ? masked : 0.0f;
				s[col] = s[col] + mask;
			}
		}
		float mx = s[0]; /* Device.h:727-741 ReduceOp::Max */
		for (size_t col = 1; col < l; ++col)
		{
			if (s[col] > mx)
			{
				mx = s[col];
			}
		}
		for (size_t col = 0; col < l; ++col)
		{
			s[col] = expf(s[col] - mx);
		}
		float denom = s[0]; /* ReduceOp::Sum, sequential */
		for (size_t col = 1; col < l; ++col)
		{
			denom += s[col];
		}
		for (size_t col = 0; col < l; ++col)
		{
			s[col] = s[col] / denom;
		}
		for (size_t c = 0; c < dv; ++c)
		{
			out[row * dv + c] = 0.0f;
		}
		for (size_t col = 0; col < l; ++col)
		{
			const float p = s[col];
			for (size_t c = 0; c < dv; ++c)
			{
				out[row * dv + c] += p * v[col * dv + c];
			}
		}
	}
	free(s);
}

/* Detail::ComputeALiBiSlope, FlashAttnExt.h:69-96: 1 when maxBias <= 0 */
double oracle_alibi_slope(size_t head_index, size_t head_count, double max_bias)
{
	if (max_bias <= 0.0)
	{
		return 1.0;
	}
	size_t head_log2 = 1;
	while ((head_log2 << 1) <= head_count)
	{
		head_log2 <<= 1;
	}
	const double m0 = pow(2.0, -max_bias / (double)head_log2);
	const double m1 = pow(2.0, -(max_bias / 2.0) / (double)head_log2);
	if (head_index < head_log2)
	{
		return pow(m0, (double)(head_index + 1));
	}
	return pow(m1, (double)(2 * (head_index - head_log2) + 1));
}

/* One head of AddFlashAttnExt with every option, node by node in f32 (FlashAttnExt.h:126-228):
 * MatMul, scalar multiply by scale (or scale / softcap), AddTanh as (exp(2x) - 1) / (exp(2x) + 1)
 * (Activation.h:34-50) and multiply by softcap, + mask (times the ALiBi slope when maxBias > 0),
 * + causal mask (CausalMask.h:16-34), row max (joined with the sink), exp, sequential sum (+ the
 * sink's term), divide, MatMul.  A scalar multiply by exactly 1 is not emitted (:57-67). */
void oracle_flash_attn_ext(const float* q, size_t mq, const float* k, const float* v, size_t l, size_t d, size_t dv,
                           double scale, double logit_softcap, const float* mask, double mask_slope,
                           const float* sink, int causal, size_t key_pos_offset, size_t query_pos_offset, float* out)
{
	float* s = (float*)malloc(sizeof(float) * (l ? l : 1));
	const double score_scale = logit_softcap != 0.0 ? scale / logit_softcap : scale;
	const float score_scale_f = (float)score_scale; /* MakeScalarTensor(f32, .) */
	const float softcap_f = (float)logit_softcap;
	const float slope_f = (float)mask_slope;
	const float masked = (float)-1.0e9;
	for (size_t row = 0; row < mq; ++row)
	{
		for (size_t col = 0; col < l; ++col)
		{
			s[col] = 0.0f;
		}
		for (size_t kk = 0; kk < d; ++kk)
		{
			const float lhs = q[row * d + kk];
			for (size_t col = 0; col < l; ++col)
			{
				s[col] += lhs * k[col * d + kk];
			}
		}
		if ((scale != 1.0 || logit_softcap != 0.0) && score_scale != 1.0)
		{
			for (size_t col = 0; col < l; ++col)
			{
				s[col] = s[col] * score_scale_f;
			}
		}
		if (logit_softcap != 0.0)
		{
			for (size_t col = 0; col < l; ++col)
			{
				const float scaled = s[col] * 2.0f;
				const float e = expf(scaled);
				const float numerator = e - 1.0f;
				const float denominator = e + 1.0f;
				s[col] = numerator / denominator;
			}
			if (logit_softcap != 1.0)
			{
				for (size_t col = 0; col < l; ++col)
				{
					s[col] = s[col] * softcap_f;
				}
			}
		}
		if (mask)
		{
			for (size_t col = 0; col < l; ++col)
			{
				float mv = mask[row * l + col];
				if (mask_slope != 1.0)
				{
					mv = mv * slope_f;
				}
				s[col] = s[col] + mv;
			}
		}
		if (causal)
		{
			for (size_t col = 0; col < l; ++col)
			{
				const float cm = (key_pos_offset + col > query_pos_offset + row) ? masked : 0.0f;
				s[col] = s[col] + cm;
			}
		}
		float mx = s[0];
		for (size_t col = 1; col < l; ++col)
		{
			if (s[col] > mx)
			{
				mx = s[col];
			}
		}
		if (sink && *sink > mx) /* BinaryOp::Max(maxScores, sink) */
		{
			mx = *sink;
		}
		for (size_t col = 0; col < l; ++col)
		{
			s[col] = expf(s[col] - mx);
		}
		float denom = s[0];
		for (size_t col = 1; col < l; ++col)
		{
			denom += s[col];
		}
		if (sink)
		{
			denom = denom + expf(*sink - mx);
		}
		for (size_t col = 0; col < l; ++col)
		{
			s[col] = s[col] / denom;
		}
		for (size_t c = 0; c < dv; ++c)
		{
			out[row * dv + c] = 0.0f;
		}
		for (size_t col = 0; col < l; ++col)
		{
			const float p = s[col];
			for (size_t c = 0; c < dv; ++c)
			{
				out[row * dv + c] += p * v[col * dv + c];
			}
		}
	}
	free(s);
}

/* Activation.h:22-35,56-63 */
void oracle_silu(const float* x, float* y, size_t n)
{
	for (size_t i = 0; i < n; ++i)
	{
		const float neg = -x[i];
		const float e = expf(neg);
		const float denom = 1.0f + e;
		const float sig = 1.0f / denom;
		y[i] = x[i] * sig;
	}
}

void oracle_silu_mul(const float* gate, const float* up, float* y, size_t n)
{
	for (size_t i = 0; i < n; ++i)
	{
		const float neg = -gate[i];
		const float e = expf(neg);
		const float denom = 1.0f + e;
		const float sig = 1.0f / denom;
		const float act = gate[i] * sig;
		y[i] = act * up[i];
	}
}

int oracle_get_rows(const float* table, size_t rows, size_t cols, const int32_t* idx, size_t n, float* out)
{
	for (size_t i = 0; i < n; ++i)
	{
		if (idx[i] < 0 || (size_t)idx[i] >= rows)
		{
			return fail("GetRows index out of range");
		}
		memcpy(out + i * cols, table + (size_t)idx[i] * cols, sizeof(float) * cols);
	}
	return 0;
}

int32_t oracle_argmax(const float* x, size_t n)
{
	size_t best = 0;
	for (size_t i = 1; i < n; ++i)
	{
		if (x[i] > x[best])
		{
			best = i;
		}
	}
	return (int32_t)best;
}

/* ---------------------------------------------------------------------- */
/* LLaMA decoder, tools/gguf/LLaMABuilder.cpp:568-668,738-800              */
/* ---------------------------------------------------------------------- */

typedef struct
{
	int fmt;
	const uint8_t* data; /* GGUF layout [n, k] */
	size_t n, k;
	float* dense_kn; /* materialised f32 [k, n] when requested */
} qtensor;

typedef struct
{
	qtensor wq, wk, wv, wo, gate, up, down;
	const float* attn_norm;
	const float* ffn_norm;
	float* kcache; /* [ctx, n_kv_head*head_dim] */
	float* vcache;
} layer_t;

struct oracle_llama
{
	int n_layer, d_model, n_head, n_kv_head, head_dim, d_ff, vocab, ctx, rope_dims;
	double eps, rope_base, rope_scale;
	int kv_f16, materialize;
	int past;
	qtensor tok_embd, output;
	const float* output_norm;
	layer_t* layers;
};

oracle_llama* oracle_llama_new(int n_layer, int d_model, int n_head, int n_kv_head, int d_ff, int vocab, int ctx,
                               int rope_dims, double rms_eps, double rope_base, double rope_freq_scale, int kv_f16,
                               int materialize)
{
	if (n_layer <= 0 || d_model <= 0 || n_head <= 0 || n_kv_head <= 0 || d_model % n_head != 0 ||
	    n_head % n_kv_head != 0 || d_ff <= 0 || vocab <= 0 || ctx <= 0)
	{
		fail("bad hyper-parameters");
		return NULL;
	}
	oracle_llama* m = (oracle_llama*)calloc(1, sizeof *m);
	m->n_layer = n_layer;
	m->d_model = d_model;
	m->n_head = n_head;
	m->n_kv_head = n_kv_head;
	m->head_dim = d_model / n_head;
	m->d_ff = d_ff;
	m->vocab = vocab;
	m->ctx = ctx;
	m->rope_dims = rope_dims > 0 ? rope_dims : m->head_dim;
	m->eps = rms_eps;
	m->rope_base = rope_base;
	m->rope_scale = rope_freq_scale;
	m->kv_f16 = kv_f16;
	m->materialize = materialize;
	m->layers = (layer_t*)calloc((size_t)n_layer, sizeof(layer_t));
	const size_t kvw = (size_t)n_kv_head * (size_t)m->head_dim;
	for (int l = 0; l < n_layer; ++l)
	{
		m->layers[l].kcache = (float*)calloc((size_t)ctx * kvw, sizeof(float));
		m->layers[l].vcache = (float*)calloc((size_t)ctx * kvw, sizeof(float));
	}
	return m;
}

static void qtensor_release(qtensor* t)
{
	free(t->dense_kn);
	t->dense_kn = NULL;
}

void oracle_llama_free(oracle_llama* m)
{
	if (!m)
	{
		return;
	}
	qtensor_release(&m->tok_embd);
	qtensor_release(&m->output);
	for (int l = 0; l < m->n_layer; ++l)
	{
		layer_t* L = &m->layers[l];
		qtensor_release(&L->wq);
		qtensor_release(&L->wk);
		qtensor_release(&L->wv);
		qtensor_release(&L->wo);
		qtensor_release(&L->gate);
		qtensor_release(&L->up);
		qtensor_release(&L->down);
		free(L->kcache);
		free(L->vcache);
	}
	free(m->layers);
	free(m);
}

static int qtensor_set(oracle_llama* m, qtensor* t, int fmt, const void* data, size_t n, size_t k, int is_linear)
{
	if (oracle_row_bytes(fmt, k) == 0)
	{
		return fail("tensor row width incompatible with block format");
	}
	qtensor_release(t);
	t->fmt = fmt;
	t->data = (const uint8_t*)data;
	t->n = n;
	t->k = k;
	if (m->materialize && is_linear)
	{
		/* DequantizeGGMLVariable + Transpose, LLaMABuilder.cpp:144-150,225-230 */
		float* deq = (float*)malloc(sizeof(float) * n * k);
		t->dense_kn = (float*)malloc(sizeof(float) * n * k);
		if (!deq || !t->dense_kn)
		{
			free(deq);
			return fail("out of memory");
		}
		oracle_dequantize(fmt, t->data, deq, n, k);
		oracle_transpose(deq, t->dense_kn, n, k);
		free(deq);
	}
	return 0;
}

int oracle_llama_set_tensor(oracle_llama* m, int which, int layer, int fmt, const void* data, size_t n, size_t k)
{
	const size_t d = (size_t)m->d_model, hd = (size_t)m->head_dim;
	const size_t qw = (size_t)m->n_head * hd, kvw = (size_t)m->n_kv_head * hd, ff = (size_t)m->d_ff;
	if (which >= ORACLE_T_ATTN_Q && which != ORACLE_T_OUTPUT_NORM && (layer < 0 || layer >= m->n_layer))
	{
		return fail("layer index out of range");
	}
	layer_t* L = (layer >= 0 && layer < m->n_layer) ? &m->layers[layer] : NULL;
#define CHECK_SHAPE(N, K)                                                                                              \
	if (n != (N) || k != (K))                                                                                          \
	{                                                                                                                  \
		return fail("tensor shape does not match hyper-parameters");                                                   \
	}
	switch (which)
	{
	case ORACLE_T_TOKEN_EMBD:
		CHECK_SHAPE((size_t)m->vocab, d);
		return qtensor_set(m, &m->tok_embd, fmt, data, n, k, 0);
	case ORACLE_T_OUTPUT:
		CHECK_SHAPE((size_t)m->vocab, d);
		return qtensor_set(m, &m->output, fmt, data, n, k, 1);
	case ORACLE_T_ATTN_Q:
		CHECK_SHAPE(qw, d);
		return qtensor_set(m, &L->wq, fmt, data, n, k, 1);
	case ORACLE_T_ATTN_K:
		CHECK_SHAPE(kvw, d);
		return qtensor_set(m, &L->wk, fmt, data, n, k, 1);
	case ORACLE_T_ATTN_V:
		CHECK_SHAPE(kvw, d);
		return qtensor_set(m, &L->wv, fmt, data, n, k, 1);
	case ORACLE_T_ATTN_OUTPUT:
		CHECK_SHAPE(d, qw);
		return qtensor_set(m, &L->wo, fmt, data, n, k, 1);
	case ORACLE_T_FFN_GATE:
		CHECK_SHAPE(ff, d);
		return qtensor_set(m, &L->gate, fmt, data, n, k, 1);
	case ORACLE_T_FFN_UP:
		CHECK_SHAPE(ff, d);
		return qtensor_set(m, &L->up, fmt, data, n, k, 1);
	case ORACLE_T_FFN_DOWN:
		CHECK_SHAPE(d, ff);
		return qtensor_set(m, &L->down, fmt, data, n, k, 1);
	case ORACLE_T_OUTPUT_NORM:
	case ORACLE_T_ATTN_NORM:
	case ORACLE_T_FFN_NORM:
		if (fmt != ORACLE_FMT_F32 || n * k != d)
		{
			return fail("norm weight must be f32 [d_model]");
		}
		if (which == ORACLE_T_OUTPUT_NORM)
		{
			m->output_norm = (const float*)data;
		}
		else if (which == ORACLE_T_ATTN_NORM)
		{
			L->attn_norm = (const float*)data;
		}
		else
		{
			L->ffn_norm = (const float*)data;
		}
		return 0;
	default:
		return fail("unknown tensor id");
	}
#undef CHECK_SHAPE
}

int oracle_llama_past(const oracle_llama* m)
{
	return m->past;
}

void oracle_llama_reset(oracle_llama* m)
{
	m->past = 0;
}

/* AddLinear, Linear.h:67-95: y[M,n] = x[M,k] . W[k,n] */
static int linear(const oracle_llama* m, const qtensor* t, const float* x, size_t rows, float* y)
{
	if (!t->data)
	{
		return fail("missing weight tensor");
	}
	if (m->materialize && t->dense_kn)
	{
		oracle_matmul_ikj(x, t->dense_kn, y, rows, t->k, t->n);
		return 0;
	}
	return oracle_mul_mat_q_rowwise(t->fmt, t->data, t->n, t->k, x, rows, y);
}

int oracle_llama_eval(oracle_llama* m, const int32_t* tokens, int m_tokens, float* logits, float* last_logits)
{
	const size_t M = (size_t)m_tokens;
	const size_t d = (size_t)m->d_model, hd = (size_t)m->head_dim;
	const size_t H = (size_t)m->n_head, KH = (size_t)m->n_kv_head;
	const size_t qw = H * hd, kvw = KH * hd, ff = (size_t)m->d_ff;
	const size_t P = (size_t)m->past;
	const size_t groups = H / KH;
	if (m_tokens <= 0)
	{
		return fail("sequence length must be positive");
	}
	if (P + M > (size_t)m->ctx)
	{
		return fail("context length exceeded");
	}
	if (!m->tok_embd.data || !m->output_norm)
	{
		return fail("missing token_embd / output_norm");
	}
	const size_t L = P + M;
	float* x = (float*)malloc(sizeof(float) * M * d);
	float* xn = (float*)malloc(sizeof(float) * M * d);
	float* q = (float*)malloc(sizeof(float) * M * qw);
	float* kx = (float*)malloc(sizeof(float) * M * kvw);
	float* vx = (float*)malloc(sizeof(float) * M * kvw);
	float* merged = (float*)malloc(sizeof(float) * M * qw);
	float* attn_out = (float*)malloc(sizeof(float) * M * d);
	float* h1 = (float*)malloc(sizeof(float) * M * d);
	float* g = (float*)malloc(sizeof(float) * M * ff);
	float* u = (float*)malloc(sizeof(float) * M * ff);
	float* dn = (float*)malloc(sizeof(float) * M * d);
	int rc = 0;

	/* AddLLaMATokenEmbedding, LLaMABuilder.cpp:738-759: rows of the dequantised table */
	{
		const size_t rb = oracle_row_bytes(m->tok_embd.fmt, d);
		for (size_t i = 0; i < M && rc == 0; ++i)
		{
			if (tokens[i] < 0 || tokens[i] >= m->vocab)
			{
				rc = fail("GetRows index out of range");
				break;
			}
			oracle_dequantize_row(m->tok_embd.fmt, m->tok_embd.data + (size_t)tokens[i] * rb, x + i * d, d);
		}
	}

	for (int li = 0; li < m->n_layer && rc == 0; ++li)
	{
		layer_t* Ly = &m->layers[li];
		if (!Ly->attn_norm || !Ly->ffn_norm)
		{
			rc = fail("missing norm weight");
			break;
		}
		oracle_rmsnorm(x, Ly->attn_norm, m->eps, M, d, xn);
		if ((rc = linear(m, &Ly->wq, xn, M, q)) != 0 || (rc = linear(m, &Ly->wk, xn, M, kx)) != 0 ||
		    (rc = linear(m, &Ly->wv, xn, M, vx)) != 0)
		{
			break;
		}
		/* rotate every KV head at positions P..P+M-1 and append (LLaMABuilder.cpp:596-622) */
		{
			float* kh = (float*)malloc(sizeof(float) * M * hd);
			float* kr = (float*)malloc(sizeof(float) * M * hd);
			for (size_t h = 0; h < KH; ++h)
			{
				for (size_t i = 0; i < M; ++i)
				{
					memcpy(kh + i * hd, kx + i * kvw + h * hd, sizeof(float) * hd);
				}
				oracle_rope(kh, kr, M, hd, (size_t)m->rope_dims, m->rope_base, m->rope_scale, P);
				for (size_t i = 0; i < M; ++i)
				{
					memcpy(Ly->kcache + (P + i) * kvw + h * hd, kr + i * hd, sizeof(float) * hd);
				}
			}
			free(kh);
			free(kr);
			memcpy(Ly->vcache + P * kvw, vx, sizeof(float) * M * kvw);
			if (m->kv_f16)
			{
				for (size_t e = P * kvw; e < L * kvw; ++e)
				{
					Ly->kcache[e] = oracle_f16_to_f32(oracle_f32_to_f16(Ly->kcache[e]));
					Ly->vcache[e] = oracle_f16_to_f32(oracle_f32_to_f16(Ly->vcache[e]));
				}
			}
		}
		/* per query head attention over the updated cache (LLaMABuilder.cpp:624-645) */
#pragma omp parallel for schedule(static)
		for (size_t h = 0; h < H; ++h)
		{
			const size_t kvh = h / groups;
			float* qh = (float*)malloc(sizeof(float) * M * hd);
			float* qr = (float*)malloc(sizeof(float) * M * hd);
			float* keys = (float*)malloc(sizeof(float) * L * hd);
			float* vals = (float*)malloc(sizeof(float) * L * hd);
			float* ctx = (float*)malloc(sizeof(float) * M * hd);
			for (size_t i = 0; i < M; ++i)
			{
				memcpy(qh + i * hd, q + i * qw + h * hd, sizeof(float) * hd);
			}
			oracle_rope(qh, qr, M, hd, (size_t)m->rope_dims, m->rope_base, m->rope_scale, P);
			for (size_t t = 0; t < L; ++t)
			{
				memcpy(keys + t * hd, Ly->kcache + t * kvw + kvh * hd, sizeof(float) * hd);
				memcpy(vals + t * hd, Ly->vcache + t * kvw + kvh * hd, sizeof(float) * hd);
			}
			oracle_attention_head(qr, M, keys, vals, L, hd, hd, 1.0 / sqrt((double)hd), 1, 0, P, ctx);
			for (size_t i = 0; i < M; ++i)
			{
				memcpy(merged + i * qw + h * hd, ctx + i * hd, sizeof(float) * hd);
			}
			free(qh);
			free(qr);
			free(keys);
			free(vals);
			free(ctx);
		}
		if ((rc = linear(m, &Ly->wo, merged, M, attn_out)) != 0)
		{
			break;
		}
		for (size_t e = 0; e < M * d; ++e)
		{
			h1[e] = x[e] + attn_out[e];
		}
		oracle_rmsnorm(h1, Ly->ffn_norm, m->eps, M, d, xn);
		if ((rc = linear(m, &Ly->gate, xn, M, g)) != 0 || (rc = linear(m, &Ly->up, xn, M, u)) != 0)
		{
			break;
		}
		oracle_silu_mul(g, u, g, M * ff);
		if ((rc = linear(m, &Ly->down, g, M, dn)) != 0)
		{
			break;
		}
		for (size_t e = 0; e < M * d; ++e)
		{
			x[e] = h1[e] + dn[e];
		}
	}

	if (rc == 0)
	{
		const qtensor* head = m->output.data ? &m->output : &m->tok_embd; /* LLaMABuilder.cpp:719-733 */
		oracle_rmsnorm(x, m->output_norm, m->eps, M, d, xn);
		if (logits)
		{
			rc = oracle_mul_mat_q_rowwise(head->fmt, head->data, head->n, head->k, xn, M, logits);
			if (rc == 0 && last_logits)
			{
				memcpy(last_logits, logits + (M - 1) * (size_t)m->vocab, sizeof(float) * (size_t)m->vocab);
			}
		}
		else if (last_logits)
		{
			rc = oracle_mul_mat_q_rowwise(head->fmt, head->data, head->n, head->k, xn + (M - 1) * d, 1, last_logits);
		}
	}
	if (rc == 0)
	{
		m->past = (int)L;
	}
	free(x);
	free(xn);
	free(q);
	free(kx);
	free(vx);
	free(merged);
	free(attn_out);
	free(h1);
	free(g);
	free(u);
	free(dn);
	return rc;
}

int oracle_llama_generate(oracle_llama* m, const int32_t* prompt, int n_prompt, int n_new, int32_t* out_tokens,
                          float* margins)
{
	float* lg = (float*)malloc(sizeof(float) * (size_t)m->vocab);
	int rc = oracle_llama_eval(m, prompt, n_prompt, NULL, lg);
	for (int i = 0; i < n_new && rc == 0; ++i)
	{
		const int32_t t = oracle_argmax(lg, (size_t)m->vocab);
		out_tokens[i] = t;
		if (margins)
		{
			float second = -INFINITY;
			for (int j = 0; j < m->vocab; ++j)
			{
				if (j != t && lg[j] > second)
				{
					second = lg[j];
				}
			}
			margins[i] = lg[t] - second;
		}
		if (i + 1 < n_new)
		{
			rc = oracle_llama_eval(m, &t, 1, NULL, lg);
		}
	}
	free(lg);
	return rc;
}

int oracle_llama_get_kv(const oracle_llama* m, int layer, float* k, float* v)
{
	if (layer < 0 || layer >= m->n_layer)
	{
		return fail("layer index out of range");
	}
	const size_t kvw = (size_t)m->n_kv_head * (size_t)m->head_dim;
	memcpy(k, m->layers[layer].kcache, sizeof(float) * (size_t)m->past * kvw);
	memcpy(v, m->layers[layer].vcache, sizeof(float) * (size_t)m->past * kvw);
	return 0;
}

/* Test-harness convenience (no counterpart in the reference): puts back cache rows that
 * oracle_llama_get_kv returned earlier and sets the position, so that a long checker run can be
 * resumed from a saved state.  Rows are copied bit for bit. */
int oracle_llama_set_kv(oracle_llama* m, int layer, int rows, const float* k, const float* v)
{
	if (layer < 0 || layer >= m->n_layer)
	{
		return fail("layer index out of range");
	}
	if (rows < 0 || rows > m->ctx)
	{
		return fail("row count exceeds the context length");
	}
	const size_t kvw = (size_t)m->n_kv_head * (size_t)m->head_dim;
	memcpy(m->layers[layer].kcache, k, sizeof(float) * (size_t)rows * kvw);
	memcpy(m->layers[layer].vcache, v, sizeof(float) * (size_t)rows * kvw);
	return 0;
}

int oracle_llama_set_past(oracle_llama* m, int past)
{
	if (past < 0 || past > m->ctx)
	{
		return fail("position exceeds the context length");
	}
	m->past = past;
	return 0;
}
