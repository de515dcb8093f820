// Host build of nnforge_amd/csrc/nnf_math.h for the CPU tests: the same scalar formulas the gfx950
// kernels evaluate, compiled by g++ (-ffp-contract=off), so that the formulas can be checked
// against libm and against the oracle without a GPU.
#include <cmath>
#include <cstdint>
#include <cstring>

#include "../../nnforge_amd/csrc/nnf_math.h"

namespace
{
	const uint64_t exp2_table[nnf::exp2_table_size] = { NNF_EXP2_TABLE_VALUES };

	const nnf::exp_context exp_ctx = nnf::make_exp_context(exp2_table);

	inline uint32_t bits_of(float f) { uint32_t u; std::memcpy(&u, &f, 4); return u; }
	inline float float_of(uint32_t u) { float f; std::memcpy(&f, &u, 4); return f; }
}

extern "C"
{
	// Compares nnf_expf with libm's expf on the bit patterns first, first + stride, ... (count of them);
	// returns the number of inputs whose results differ in bits (two NaNs count as equal) and stores
	// the first differing input bit pattern.
	__attribute__((visibility("default")))
	unsigned long long nnf_host_expf_mismatches(unsigned long long first, unsigned long long stride, unsigned long long count, uint32_t* first_bad)
	{
		unsigned long long bad = 0;
		uint32_t first_bad_local = 0;
		#pragma omp parallel for schedule(static) reduction(+:bad)
		for(long long i = 0; i < static_cast<long long>(count); ++i)
		{
			const uint32_t u = static_cast<uint32_t>(first + static_cast<unsigned long long>(i) * stride);
			const float x = float_of(u);
			const float a = nnf::nnf_expf(x, exp_ctx);
			const float b = expf(x);
			if ((bits_of(a) != bits_of(b)) && !((a != a) && (b != b)))
			{
				if (bad == 0)
				{
					#pragma omp critical
					first_bad_local = u;
				}
				++bad;
			}
		}
		if (first_bad != nullptr)
			*first_bad = first_bad_local;
		return bad;
	}

	__attribute__((visibility("default")))
	void nnf_host_expf(float* out, const float* in, long long count)
	{
		for(long long i = 0; i < count; ++i)
			out[i] = nnf::nnf_expf(in[i], exp_ctx);
	}

	// kind: nnf_hip_op_kind values (1 batch norm .. 6 tanh); p0..p3: per-kind scalars
	// (batch norm: gamma, beta, mean, inverse sigma; relu: slope; prelu: a; tanh: scale, steepness)
	__attribute__((visibility("default")))
	void nnf_host_apply(int kind, float* out, const float* in, long long count, float p0, float p1, float p2, float p3)
	{
		float mult = 0.0f, add = 0.0f;
		if (kind == 1)
			nnf::nnf_batch_norm_coefficients(p0, p1, p2, p3, mult, add);
		const float steepness2 = p1 * 2.0f;
		for(long long i = 0; i < count; ++i)
		{
			const float x = in[i];
			float y = x;
			switch (kind)
			{
			case 1: y = nnf::nnf_batch_norm(x, mult, add); break;
			case 2: y = nnf::nnf_rectified_linear(x, p0); break;
			case 3: y = nnf::nnf_parametric_rectified_linear(x, p0); break;
			case 4: { float one[1] = { x }; nnf::nnf_exponential_linear<1>(one, exp_ctx); y = one[0]; } break;
			case 5: { float one[1] = { x }; nnf::nnf_sigmoid<1>(one, exp_ctx); y = one[0]; } break;
			case 6: { float one[1] = { x }; nnf::nnf_hyperbolic_tangent<1>(one, steepness2, p0, exp_ctx); y = one[0]; } break;
			default: break;
			}
			out[i] = y;
		}
	}
}
