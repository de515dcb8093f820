// Scalar fp32 arithmetic of the element-wise layers, written once and used by the gfx950 kernels
// (compiled by hipcc) and by host-side unit tests of the same formulas (compiled by g++).
//
// Rounding policy: every fp32 operation below rounds once, in the order the reference's plain
// testers write it; translation units that include this header are compiled with
// -ffp-contract=off so that no multiply-add pair is fused. The only fused operations are the
// explicit __builtin_fma calls, all of which are part of a documented evaluation scheme.
#pragma once

#include <stdint.h>

#if defined(__HIPCC__)
#define NNF_HD __host__ __device__ __forceinline__
#else
#define NNF_HD inline
#endif

namespace nnf
{
	// 2^(i/32) as IEEE-754 double bit patterns with i << 47 subtracted, i = 0..31: adding k << 47
	// (k = 32*e + i) to entry i yields 2^(k/32) directly.
	#define NNF_EXP2_TABLE_VALUES \
		0x3ff0000000000000ull, 0x3fefd9b0d3158574ull, 0x3fefb5586cf9890full, 0x3fef9301d0125b51ull, \
		0x3fef72b83c7d517bull, 0x3fef54873168b9aaull, 0x3fef387a6e756238ull, 0x3fef1e9df51fdee1ull, \
		0x3fef06fe0a31b715ull, 0x3feef1a7373aa9cbull, 0x3feedea64c123422ull, 0x3feece086061892dull, \
		0x3feebfdad5362a27ull, 0x3feeb42b569d4f82ull, 0x3feeab07dd485429ull, 0x3feea47eb03a5585ull, \
		0x3feea09e667f3bcdull, 0x3fee9f75e8ec5f74ull, 0x3feea11473eb0187ull, 0x3feea589994cce13ull, \
		0x3feeace5422aa0dbull, 0x3feeb737b0cdc5e5ull, 0x3feec49182a3f090ull, 0x3feed503b23e255dull, \
		0x3feee89f995ad3adull, 0x3feeff76f2fb5e47ull, 0x3fef199bdd85529cull, 0x3fef3720dcef9069ull, \
		0x3fef5818dcfba487ull, 0x3fef7c97337b9b5full, 0x3fefa4afa2a490daull, 0x3fefd0765b6e4540ull

	constexpr int exp2_table_size = 32;

	// Two constants of nnf_expf that the kernels keep in registers (read once per lane from LDS, so
	// that the compiler holds them in VGPRs instead of re-materialising them before every use).
	#define NNF_EXP_SHIFT_BITS 0x4338000000000000ull /* 0x1.8p+52 */
	#define NNF_EXP_C1_BITS 0x3f2ebfce50fac4f3ull    /* 0x1.ebfce50fac4f3p-13 = (ln2/32)^2 / 2, minimax-adjusted */

	NNF_HD double bits_to_double(uint64_t u) { return __builtin_bit_cast(double, u); }
	NNF_HD uint64_t double_to_bits(double d) { return __builtin_bit_cast(uint64_t, d); }

	// the two 32-bit halves of a little-endian IEEE-754 double
	struct double_words
	{
		uint32_t lo;
		uint32_t hi;
	};

	// What nnf_expf needs besides its argument.
	struct exp_context
	{
		const uint64_t* table; // the 32 values of NNF_EXP2_TABLE_VALUES (LDS copy on the device)
		double shift;          // NNF_EXP_SHIFT_BITS: adding it rounds to an integer kept in the low mantissa bits
		double c1;             // NNF_EXP_C1_BITS
	};

	NNF_HD exp_context make_exp_context(const uint64_t* table)
	{
		exp_context ctx;
		ctx.table = table;
		ctx.shift = bits_to_double(NNF_EXP_SHIFT_BITS);
		ctx.c1 = bits_to_double(NNF_EXP_C1_BITS);
		return ctx;
	}

	// expf with the result of a double-precision evaluation rounded once to fp32.
	//
	// The reference's plain testers call the C library's expf (e.g.
	// nnforge/plain/exponential_linear_layer_tester_plain.cpp:51). glibc >= 2.27 evaluates expf as
	// 2^(k/32) * p(r) in double precision (x*32/ln2 = k + r, |r| <= 1/2, 32-entry table, cubic p) and
	// rounds the double to float, which makes it correctly rounded for all but a handful of inputs.
	// This is the same published scheme with the argument reduction fused and the cubic in Horner
	// form (7 double-precision operations); it returns the same bits as that expf for every one of
	// the 2^32 fp32 inputs (checked exhaustively on the host by the unit tests; NaN payloads aside).
	//
	// The rounded integer k sits in the low word of the shifted sum; only the high word of the table
	// entry takes part in applying the exponent (k << 47 = (k << 15) in the high word).
	//
	// nnf_expf_core is the arithmetic alone: valid for log(2^-150) < x < log(2^128), NaN in, NaN out;
	// outside that range k does not fit and the value is meaningless (nnf_expf_out_of_range repairs it).
	NNF_HD float nnf_expf_core(float x, const exp_context& ctx)
	{
		const double inv_ln2_times_32 = 0x1.71547652b82fep+5;
		const double c0 = 0x1.c6af84b912394p-20; // (ln2/32)^3 / 6, minimax-adjusted
		const double c2 = 0x1.62e42ff0c52d6p-6;  // ln2/32

		const double xd = static_cast<double>(x);
		double kd = __builtin_fma(inv_ln2_times_32, xd, ctx.shift);
		const uint32_t k = static_cast<uint32_t>(double_to_bits(kd));
		kd -= ctx.shift;
		const double r = __builtin_fma(inv_ln2_times_32, xd, -kd);
		double_words entry = reinterpret_cast<const double_words*>(ctx.table)[k & (exp2_table_size - 1)];
		uint32_t scale_hi = entry.hi + (k << 15);
	#if defined(__HIP_DEVICE_COMPILE__)
		// keeps the addition a 32-bit one (the compiler otherwise widens it to a 64-bit add with
		// extra register moves)
		asm("" : "+v"(scale_hi));
	#endif
		entry.hi = scale_hi;
		const double s = __builtin_bit_cast(double, entry);
		double y = __builtin_fma(c0, r, ctx.c1);
		y = __builtin_fma(y, r, c2);
		y = __builtin_fma(y, r, 1.0);
		y = y * s;
		return static_cast<float>(y);
	}

	// Results outside the range of nnf_expf_core: +inf above log(2^128), 0 below log(2^-150).
	// NaN fails both comparisons and keeps the NaN the arithmetic produced.
	NNF_HD float nnf_expf_out_of_range(float x, float res)
	{
		res = x > 0x1.62e42ep6f ? __builtin_inff() : res;
		res = x < -0x1.9fe368p6f ? 0.0f : res;
		return res;
	}

	NNF_HD float nnf_expf(float x, const exp_context& ctx)
	{
		return nnf_expf_out_of_range(x, nnf_expf_core(x, ctx));
	}

	// res[i] = expf(x[i]) for the small batch of values a lane holds. On the device the range repair
	// is one comparison per value and one wavefront-uniform branch per batch: only a wavefront that
	// holds an |x| above 87 (or a NaN) anywhere in the batch runs the two selects per value; every
	// other wavefront runs the arithmetic alone (|x| <= 87 is inside the range of nnf_expf_core and
	// its results are normal numbers). Returns whether this wavefront took the repair branch; when
	// it did not, every res[i] lies in [exp(-87), exp(87)] (about 1.6e-38 .. 6.1e37).
	template<int N>
	NNF_HD bool nnf_expf_batch(const float (&x)[N], float (&res)[N], const exp_context& ctx)
	{
	#if defined(__HIP_DEVICE_COMPILE__)
		bool repair = false;
		#pragma unroll
		for(int i = 0; i < N; ++i)
		{
			res[i] = nnf_expf_core(x[i], ctx);
			repair |= !(__builtin_fabsf(x[i]) <= 87.0f);
		}
		const bool any_repair = __any(repair);
		if (__builtin_expect(any_repair, 0))
		{
			#pragma unroll
			for(int i = 0; i < N; ++i)
				res[i] = nnf_expf_out_of_range(x[i], res[i]);
		}
		return any_repair;
	#else
		for(int i = 0; i < N; ++i)
			res[i] = nnf_expf(x[i], ctx);
		return true;
	#endif
	}

	// The only divisions the layers below make have the denominator d = e + 1 with e = expf(...) >= 0,
	// i.e. d >= 1, +inf or NaN. On the device they start from the hardware reciprocal estimate r0
	// (within 1 ulp of 1/d):
	//   1 / d             = fma(fma(-d, r0, 1), r0, r0)            (one Newton step)
	//   (e - 1) / (e + 1) = fma(fma(-d, q0, n), r0, q0), q0 = n*r0  (quotient, exact remainder, correction)
	// Both were compared with IEEE division for every non-negative float e with e + 1 <= 2^126 (all
	// 2^31 of them, and the device library's self-check repeats that sweep): identical bits. The
	// second sequence is only claimed for the pair n = e - 1, d = e + 1, not for arbitrary numerators.
	// Above 2^126 (and for inf / NaN) the reciprocal leaves the normal range: a wavefront whose expf
	// batch took the repair branch (general_division: some |x| > 87 or NaN, the only way to an
	// e above exp(87) < 2^126) uses the general IEEE division for the whole batch instead.
	NNF_HD float nnf_fast_reciprocal_of_ge1(float d)
	{
	#if defined(__HIP_DEVICE_COMPILE__)
		const float r = __builtin_amdgcn_rcpf(d);
		const float e = __builtin_fmaf(-d, r, 1.0f);
		return __builtin_fmaf(e, r, r);
	#else
		return 1.0f / d;
	#endif
	}

	NNF_HD float nnf_fast_tanh_quotient(float n, float d)
	{
	#if defined(__HIP_DEVICE_COMPILE__)
		const float r = __builtin_amdgcn_rcpf(d);
		const float q = n * r;
		const float rem = __builtin_fmaf(-d, q, n);
		return __builtin_fmaf(rem, r, q);
	#else
		return n / d;
	#endif
	}

	// 1 / (e[i] + 1), e[i] = expf(...); general_division is uniform across the wavefront
	template<int N>
	NNF_HD void nnf_reciprocal_of_exp_plus_one(const float (&e)[N], float (&quotient)[N], bool general_division)
	{
		if (__builtin_expect(general_division, 0))
		{
			#pragma unroll
			for(int i = 0; i < N; ++i)
				quotient[i] = 1.0f / (e[i] + 1.0f);
		}
		else
		{
			#pragma unroll
			for(int i = 0; i < N; ++i)
				quotient[i] = nnf_fast_reciprocal_of_ge1(e[i] + 1.0f);
		}
	}

	// (e[i] - 1) / (e[i] + 1), e[i] = expf(...); general_division is uniform across the wavefront
	template<int N>
	NNF_HD void nnf_exp_minus_one_over_exp_plus_one(const float (&e)[N], float (&quotient)[N], bool general_division)
	{
		if (__builtin_expect(general_division, 0))
		{
			#pragma unroll
			for(int i = 0; i < N; ++i)
				quotient[i] = (e[i] - 1.0f) / (e[i] + 1.0f);
		}
		else
		{
			#pragma unroll
			for(int i = 0; i < N; ++i)
				quotient[i] = nnf_fast_tanh_quotient(e[i] - 1.0f, e[i] + 1.0f);
		}
	}

	// nnforge/plain/batch_norm_layer_tester_plain.cpp:60-61
	NNF_HD void nnf_batch_norm_coefficients(float gamma, float beta, float mean, float inverse_sigma, float& mult, float& add)
	{
		mult = gamma * inverse_sigma;
		const float mult_mean = mult * mean;
		add = beta - mult_mean;
	}

	// nnforge/plain/batch_norm_layer_tester_plain.cpp:70-71
	NNF_HD float nnf_batch_norm(float x, float mult, float add)
	{
		const float scaled = x * mult;
		return scaled + add;
	}

	// nnforge/plain/rectified_linear_layer_tester_plain.cpp:53-54
	NNF_HD float nnf_rectified_linear(float x, float negative_slope)
	{
		return x >= 0.0f ? x : x * negative_slope;
	}

	// nnforge/plain/absolute_layer_tester_plain.cpp:49 (fabs: clears the sign bit, of NaN as well)
	NNF_HD float nnf_absolute(float x)
	{
		return __builtin_fabsf(x);
	}

	// nnforge/plain/parametric_rectified_linear_layer_tester_plain.cpp:66-67
	NNF_HD float nnf_parametric_rectified_linear(float x, float a)
	{
		return x * (x >= 0.0f ? 1.0f : a);
	}

	// The layers that call expf work on small batches of values (the registers a lane holds), in place.

	// nnforge/plain/exponential_linear_layer_tester_plain.cpp:50-51
	template<int N>
	NNF_HD void nnf_exponential_linear(float (&v)[N], const exp_context& ctx)
	{
		float e[N];
		nnf_expf_batch<N>(v, e, ctx);
		#pragma unroll
		for(int i = 0; i < N; ++i)
			v[i] = v[i] >= 0.0f ? v[i] : (e[i] - 1.0f);
	}

	// nnforge/plain/sigmoid_layer_tester_plain.cpp:50-51
	template<int N>
	NNF_HD void nnf_sigmoid(float (&v)[N], const exp_context& ctx)
	{
		float e[N];
		#pragma unroll
		for(int i = 0; i < N; ++i)
			v[i] = -v[i];
		const bool general_division = nnf_expf_batch<N>(v, e, ctx);
		nnf_reciprocal_of_exp_plus_one<N>(e, v, general_division);
	}

	// nnforge/plain/hyperbolic_tangent_layer_tester_plain.cpp:54-56; steepness2 = steepness * 2.0f
	template<int N>
	NNF_HD void nnf_hyperbolic_tangent(float (&v)[N], float steepness2, float scale, const exp_context& ctx)
	{
		float e[N];
		#pragma unroll
		for(int i = 0; i < N; ++i)
			v[i] = v[i] * steepness2;
		const bool general_division = nnf_expf_batch<N>(v, e, ctx);
		nnf_exp_minus_one_over_exp_plus_one<N>(e, v, general_division);
		#pragma unroll
		for(int i = 0; i < N; ++i)
			v[i] = v[i] * scale;
	}
}
