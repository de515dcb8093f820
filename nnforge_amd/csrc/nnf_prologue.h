// Element-wise layers that a subsampling kernel applies to its input values on their way into LDS
// ("prologue"): the layers of a single-input group that feeds the subsampling layer and nothing
// else, so that the group's result is never written to memory. The whole-plane average also takes a
// group of two inputs joined by an Add (the last block of a residual network in front of its global
// average). Same formulas, same order, one
// rounding per operation as the chain kernel: the staged values carry the bits the unfused layers
// would have stored. Shared by the 2-D window kernels (nnf_max.hip) and the whole-plane average
// kernel (nnf_pool.hip).
#pragma once

#include "nnf_common.h"

namespace nnf
{
	namespace
	{
		constexpr int prologue_block_size = 256; // lanes per workgroup of the kernels that apply a prologue

		// n / divisor with magic = ceil(2^32 / divisor), exact while n * divisor < 2^32
		__device__ __forceinline__ uint32_t fast_divide(uint32_t n, uint32_t divisor, uint32_t magic)
		{
			return (divisor == 1) ? n : __umulhi(n, magic);
		}

		constexpr uint32_t prologue_weighted_max = 2;  // layers with weights (batch norm, PReLU) a prologue may hold
		constexpr uint32_t prologue_coef_floats = 768; // LDS a workgroup sets aside for its planes' coefficients
		constexpr uint32_t prologue_planes_max = 256;  // one lane per plane fetches the weights

		struct window_prologue
		{
			uint32_t op_count;
			uint32_t arm_ops[2];             // layers applied to input 0 / input 1 before the join (one input: all of them, 0)
			uint32_t join;                   // 1: two inputs, summed by an Add after their own layers, the rest applied to the sum
			float alpha;                     // the Add's multiplier
			uint32_t fm_count;
			uint32_t need_exp;
			uint32_t in_plane_magic;         // ceil(2^32 / input plane size)
			uint32_t weighted_count;         // layers with weights; every plane has 2 coefficients per such layer
			uint32_t slot[NNF_HIP_MAX_OPS];  // where a layer's coefficients start among a plane's
			int32_t kind[NNF_HIP_MAX_OPS];
			float f0[NNF_HIP_MAX_OPS];
			float f1[NNF_HIP_MAX_OPS];       // TanH: steepness * 2
			int32_t weighted_kind[prologue_weighted_max];
			const float* weights[prologue_weighted_max][4]; // batch norm: gamma, beta, mean, inverse sigma; PReLU: slopes
		};

		// Batch norm's multiplier and addend and PReLU's slope of the planes a workgroup stages are worked
		// out once per plane, by lane plane_in_workgroup, and kept in LDS:
		// coef[plane_in_workgroup * 2 * pro.weighted_count + pro.slot[layer]]. In two steps, so that a kernel
		// can issue these loads in front of its tensor loads and wait for them behind.
		struct prologue_weights
		{
			float w[prologue_weighted_max][4];
		};

		__device__ __forceinline__ prologue_weights load_prologue_weights(uint32_t first_fm, uint32_t planes_here, const window_prologue& pro)
		{
			prologue_weights r;
			uint32_t fm = first_fm + threadIdx.x;
			if (fm >= pro.fm_count)
				fm %= pro.fm_count;
			#pragma unroll
			for(uint32_t j = 0; j < prologue_weighted_max; ++j)
			{
				#pragma unroll
				for(int c = 0; c < 4; ++c)
					r.w[j][c] = 0.0f;
				if ((j < pro.weighted_count) && (threadIdx.x < planes_here))
				{
					r.w[j][0] = pro.weights[j][0][fm];
					if (pro.weighted_kind[j] == NNF_HIP_OP_BATCH_NORM)
					{
						#pragma unroll
						for(int c = 1; c < 4; ++c)
							r.w[j][c] = pro.weights[j][c][fm];
					}
				}
			}
			return r;
		}

		// One plane per workgroup: the plane's weights through the scalar data cache (the index is the same
		// in every lane), its coefficients in registers - no LDS table, no barrier, and a wavefront looks
		// at the weights only after its tensor loads are out.
		struct uniform_weights
		{
			float w[prologue_weighted_max][4];
		};

		__device__ __forceinline__ uniform_weights load_uniform_weights(uint32_t fm, const window_prologue& pro)
		{
			uniform_weights r;
			const uint32_t fm_s = __builtin_amdgcn_readfirstlane(fm);
			#pragma unroll
			for(uint32_t j = 0; j < prologue_weighted_max; ++j)
			{
				#pragma unroll
				for(int c = 0; c < 4; ++c)
					r.w[j][c] = 0.0f;
				if (j < pro.weighted_count)
				{
					r.w[j][0] = pro.weights[j][0][fm_s];
					if (pro.weighted_kind[j] == NNF_HIP_OP_BATCH_NORM)
					{
						#pragma unroll
						for(int c = 1; c < 4; ++c)
							r.w[j][c] = pro.weights[j][c][fm_s];
					}
				}
			}
			return r;
		}

		__device__ __forceinline__ void uniform_coefficients(float (&own)[prologue_weighted_max][2], uniform_weights r, const window_prologue& pro)
		{
			// the weights are not looked at (nor waited for) before this point
			#pragma unroll
			for(uint32_t j = 0; j < prologue_weighted_max; ++j)
			{
				#pragma unroll
				for(int c = 0; c < 4; ++c)
					asm volatile("" : "+s"(r.w[j][c]));
			}
			#pragma unroll
			for(uint32_t j = 0; j < prologue_weighted_max; ++j)
			{
				own[j][0] = r.w[j][0];
				own[j][1] = 0.0f;
				if ((j < pro.weighted_count) && (pro.weighted_kind[j] == NNF_HIP_OP_BATCH_NORM))
					nnf_batch_norm_coefficients(r.w[j][0], r.w[j][1], r.w[j][2], r.w[j][3], own[j][0], own[j][1]);
			}
		}

		__device__ __forceinline__ void stage_prologue_coefficients(float* coef, prologue_weights r, uint32_t planes_here, const window_prologue& pro)
		{
			// The weights are not looked at before this point: without it the compiler works the
			// coefficients out, and waits for the weights, in front of the tensor loads.
			#pragma unroll
			for(uint32_t j = 0; j < prologue_weighted_max; ++j)
			{
				#pragma unroll
				for(int c = 0; c < 4; ++c)
					asm volatile("" : "+v"(r.w[j][c]));
			}
			#pragma unroll
			for(uint32_t j = 0; j < prologue_weighted_max; ++j)
			{
				if ((j < pro.weighted_count) && (threadIdx.x < planes_here))
				{
					float* dst = coef + (threadIdx.x * pro.weighted_count + j) * 2;
					if (pro.weighted_kind[j] == NNF_HIP_OP_BATCH_NORM)
						nnf_batch_norm_coefficients(r.w[j][0], r.w[j][1], r.w[j][2], r.w[j][3], dst[0], dst[1]);
					else
						dst[0] = r.w[j][0];
				}
			}
		}

		// One layer after another over all the float4s a lane has loaded in a round, so that a layer's
		// kind is looked up once and the coefficient reads of the round are in flight together.
		// off[k]: where the coefficients of vector k's plane start in coef.
		// EXP false: compiled without the layers that call expf (the host picks it when the group has none),
		// which leaves the kernel with far fewer registers per lane.
		constexpr int coef_batch = 4; // vectors whose batch norm coefficients are read from LDS together

		// Where the coefficients of a vector's values lie when the four values may belong to two planes: values
		// [0, split) take the coefficients at off (the argument beside this one), the others those at off2.
		template<int VECTORS>
		struct two_plane_offsets
		{
			uint32_t off2[VECTORS];
			uint32_t split[VECTORS];
		};

		// UNIFORM: every value belongs to the same plane, whose coefficients are in own (registers)
		// instead of coef (LDS). SPLIT: a vector's values may belong to two planes (two says which).
		// One layer (kind, the slot of its coefficients, its two constants) over the values of a round.
		template<int VECTORS, bool EXP, bool UNIFORM, bool SPLIT = false>
		__device__ __forceinline__ void apply_prologue_layer(float (&v)[VECTORS][4], const uint32_t (&off)[VECTORS],
			const float* coef, const float (&own)[prologue_weighted_max][2], const exp_context& exp_ctx, const two_plane_offsets<VECTORS>* two,
			const int32_t kind, const uint32_t slot, const float f0, const float f1)
		{
			switch (kind)
			{
			case NNF_HIP_OP_BATCH_NORM:
				if (UNIFORM)
				{
					static_assert(prologue_weighted_max == 2, "the coefficients of a layer are picked from two sets");
					const float mult = (slot == 0) ? own[0][0] : own[1][0];
					const float add = (slot == 0) ? own[0][1] : own[1][1];
					#pragma unroll
					for(int k = 0; k < VECTORS; ++k)
					{
						#pragma unroll
						for(int e = 0; e < 4; ++e)
							v[k][e] = nnf_batch_norm(v[k][e], mult, add);
					}
					break;
				}
				if (SPLIT)
				{
					float mult[VECTORS][2], add[VECTORS][2];
					#pragma unroll
					for(int k = 0; k < VECTORS; ++k)
					{
						mult[k][0] = coef[off[k] + slot];
						add[k][0] = coef[off[k] + slot + 1];
						mult[k][1] = coef[two->off2[k] + slot];
						add[k][1] = coef[two->off2[k] + slot + 1];
					}
					#pragma unroll
					for(int k = 0; k < VECTORS; ++k)
					{
						#pragma unroll
						for(int e = 0; e < 4; ++e)
						{
							const bool first_plane = static_cast<uint32_t>(e) < two->split[k];
							v[k][e] = nnf_batch_norm(v[k][e], first_plane ? mult[k][0] : mult[k][1], first_plane ? add[k][0] : add[k][1]);
						}
					}
					break;
				}
				#pragma unroll
				for(int k0 = 0; k0 < VECTORS; k0 += coef_batch)
				{
					float mult[coef_batch], add[coef_batch];
					#pragma unroll
					for(int k = 0; (k < coef_batch) && (k0 + k < VECTORS); ++k)
					{
						mult[k] = coef[off[k0 + k] + slot];
						add[k] = coef[off[k0 + k] + slot + 1];
					}
					#pragma unroll
					for(int k = 0; (k < coef_batch) && (k0 + k < VECTORS); ++k)
					{
						#pragma unroll
						for(int e = 0; e < 4; ++e)
							v[k0 + k][e] = nnf_batch_norm(v[k0 + k][e], mult[k], add[k]);
					}
				}
				break;
			case NNF_HIP_OP_PRELU:
				if (UNIFORM)
				{
					const float slope = (slot == 0) ? own[0][0] : own[1][0];
					#pragma unroll
					for(int k = 0; k < VECTORS; ++k)
					{
						#pragma unroll
						for(int e = 0; e < 4; ++e)
							v[k][e] = nnf_parametric_rectified_linear(v[k][e], slope);
					}
				}
				else if (SPLIT)
				{
					float slope[VECTORS][2];
					#pragma unroll
					for(int k = 0; k < VECTORS; ++k)
					{
						slope[k][0] = coef[off[k] + slot];
						slope[k][1] = coef[two->off2[k] + slot];
					}
					#pragma unroll
					for(int k = 0; k < VECTORS; ++k)
					{
						#pragma unroll
						for(int e = 0; e < 4; ++e)
							v[k][e] = nnf_parametric_rectified_linear(v[k][e], (static_cast<uint32_t>(e) < two->split[k]) ? slope[k][0] : slope[k][1]);
					}
				}
				else
				{
					float slope[VECTORS];
					#pragma unroll
					for(int k = 0; k < VECTORS; ++k)
						slope[k] = coef[off[k] + slot];
					#pragma unroll
					for(int k = 0; k < VECTORS; ++k)
					{
						#pragma unroll
						for(int e = 0; e < 4; ++e)
							v[k][e] = nnf_parametric_rectified_linear(v[k][e], slope[k]);
					}
				}
				break;
			case NNF_HIP_OP_RELU:
				#pragma unroll
				for(int k = 0; k < VECTORS; ++k)
				{
					#pragma unroll
					for(int e = 0; e < 4; ++e)
						v[k][e] = nnf_rectified_linear(v[k][e], f0);
				}
				break;
			case NNF_HIP_OP_ABSOLUTE:
				#pragma unroll
				for(int k = 0; k < VECTORS; ++k)
				{
					#pragma unroll
					for(int e = 0; e < 4; ++e)
						v[k][e] = nnf_absolute(v[k][e]);
				}
				break;
			case NNF_HIP_OP_ELU:
			case NNF_HIP_OP_SIGMOID:
			case NNF_HIP_OP_TANH:
				if (EXP)
				{
					#pragma unroll
					for(int k = 0; k < VECTORS; ++k)
					{
						if (kind == NNF_HIP_OP_ELU)
							nnf_exponential_linear<4>(v[k], exp_ctx);
						else if (kind == NNF_HIP_OP_SIGMOID)
							nnf_sigmoid<4>(v[k], exp_ctx);
						else
							nnf_hyperbolic_tangent<4>(v[k], f1, f0, exp_ctx);
					}
				}
				break;
			default: // NNF_HIP_OP_DROPOUT: the value passes through
				break;
			}
		}

		// The two groups a residual network puts in front of its subsampling layers, as straight code for kernels compiled for
		// just them: BatchNorm -> ReLU (between the first convolution and its pooling) and BatchNorm + shortcut -> Add -> ReLU
		// (the last block in front of the global average). The loop of apply_prologue keeps the values of a round in fixed
		// registers and copies every one of them once per layer (64 x 64 planes of 112 x 112 through BatchNorm, ReLU and 3 x 3
		// pooling: 20.3 M vector instructions per launch with the loop, of which the two layers need a third). As a second
		// path beside the loop in one kernel the straight code costs that kernel 40 spilled registers, hence kernels of its own:
		// the pooling kernels have one for the first group (44.2 -> 42.1 us on those planes), the whole-plane averages for
		// both (64 x 2048 planes of 7 x 7 with the second group folded in: 13.2 -> 10.8 us, the registers set free going to
		// a second round of loads in flight; planes of 8 x 8 with the first: 11.7 -> 8.2 us).
		constexpr int known_group_none = 0;
		constexpr int known_group_batch_norm_relu = 1;
		constexpr int known_group_batch_norm_shortcut_add_relu = 2; // BatchNorm on input 0, input 1 as it is
		constexpr int known_group_shortcut_batch_norm_add_relu = 3; // input 0 as it is, BatchNorm on input 1

		inline int known_group_of(const window_prologue& pro)
		{
			if ((pro.op_count != 2) || (pro.kind[0] != NNF_HIP_OP_BATCH_NORM) || (pro.kind[1] != NNF_HIP_OP_RELU))
				return known_group_none;
			if (pro.join == 0)
				return known_group_batch_norm_relu;
			if ((pro.arm_ops[0] == 1) && (pro.arm_ops[1] == 0))
				return known_group_batch_norm_shortcut_add_relu;
			return ((pro.arm_ops[0] == 0) && (pro.arm_ops[1] == 1)) ? known_group_shortcut_batch_norm_add_relu : known_group_none;
		}

		template<int VECTORS, int GROUP, bool UNIFORM, bool SPLIT = false>
		__device__ __forceinline__ void apply_known_group(float (&v)[VECTORS][4], float (&u)[VECTORS][4], const uint32_t (&off)[VECTORS],
			const float* coef, const float (&own)[prologue_weighted_max][2], const window_prologue& pro, const exp_context& exp_ctx,
			const two_plane_offsets<VECTORS>* two = nullptr)
		{
			static_assert((GROUP >= known_group_batch_norm_relu) && (GROUP <= known_group_shortcut_batch_norm_add_relu), "one of the known groups");
			apply_prologue_layer<VECTORS, false, UNIFORM, SPLIT>((GROUP == known_group_shortcut_batch_norm_add_relu) ? u : v, off, coef, own, exp_ctx, two, NNF_HIP_OP_BATCH_NORM, 0u, 0.0f, 0.0f);
			if (GROUP != known_group_batch_norm_relu)
			{
				// nnforge/plain/add_layer_tester_plain.cpp:56-59: the sum starts at 0.0F, inputs in order, times alpha
				#pragma unroll
				for(int k = 0; k < VECTORS; ++k)
				{
					#pragma unroll
					for(int e = 0; e < 4; ++e)
					{
						float sum = 0.0f + v[k][e];
						sum = sum + u[k][e];
						v[k][e] = sum * pro.alpha;
					}
				}
			}
			apply_prologue_layer<VECTORS, false, UNIFORM, SPLIT>(v, off, coef, own, exp_ctx, two, NNF_HIP_OP_RELU, 0u, pro.f0[1], 0.0f);
		}

		// Applies the layers first_op .. end_op - 1.
		template<int VECTORS, bool EXP, bool UNIFORM, bool SPLIT = false>
		__device__ __forceinline__ void apply_prologue(float (&v)[VECTORS][4], const uint32_t (&off)[VECTORS],
			const float* coef, const float (&own)[prologue_weighted_max][2], const window_prologue& pro, const exp_context& exp_ctx,
			uint32_t first_op, uint32_t end_op, const two_plane_offsets<VECTORS>* two = nullptr)
		{
			for(uint32_t i = first_op; i < end_op; ++i)
				apply_prologue_layer<VECTORS, EXP, UNIFORM, SPLIT>(v, off, coef, own, exp_ctx, two, pro.kind[i], pro.slot[i], pro.f0[i], pro.f1[i]);
		}


		// The whole group over the values of input 0 (v) and, with JOIN, input 1 (u): each input's own layers, the
		// Add (nnforge/plain/add_layer_tester_plain.cpp:56-59: the sum starts at 0.0F, inputs in order, times
		// alpha), the layers behind it. The result is left in v.
		template<int VECTORS, bool EXP, bool JOIN, bool UNIFORM = false, bool SPLIT = false>
		__device__ __forceinline__ void apply_prologue_group(float (&v)[VECTORS][4], float (&u)[VECTORS][4], const uint32_t (&off)[VECTORS],
			const float* coef, const float (&own)[prologue_weighted_max][2], const window_prologue& pro, const exp_context& exp_ctx,
			const two_plane_offsets<VECTORS>* two = nullptr)
		{
			if (!JOIN)
			{
				apply_prologue<VECTORS, EXP, UNIFORM, SPLIT>(v, off, coef, own, pro, exp_ctx, 0, pro.op_count, two);
				return;
			}
			const uint32_t arm0_end = pro.arm_ops[0];
			const uint32_t arm1_end = arm0_end + pro.arm_ops[1];
			apply_prologue<VECTORS, EXP, UNIFORM, SPLIT>(v, off, coef, own, pro, exp_ctx, 0, arm0_end, two);
			apply_prologue<VECTORS, EXP, UNIFORM, SPLIT>(u, off, coef, own, pro, exp_ctx, arm0_end, arm1_end, two);
			#pragma unroll
			for(int k = 0; k < VECTORS; ++k)
			{
				#pragma unroll
				for(int e = 0; e < 4; ++e)
				{
					float sum = 0.0f + v[k][e];
					sum = sum + u[k][e];
					v[k][e] = sum * pro.alpha;
				}
			}
			apply_prologue<VECTORS, EXP, UNIFORM, SPLIT>(v, off, coef, own, pro, exp_ctx, arm1_end, pro.op_count, two);
		}

		uint32_t magic_of(uint32_t divisor)
		{
			return (divisor >= 2) ? static_cast<uint32_t>(((1ull << 32) + divisor - 1) / divisor) : 0u; // fast_divide does not use it for 1
		}

		// The layers of a single-input group without Add - or, with allow_join, of two inputs joined by an Add -
		// in order, as the kernel wants them. False when the description is not such a group or a weight
		// pointer is missing.
		bool fill_prologue(window_prologue& pro, const nnf_hip_chain_desc& desc, const float* const* chunk_ptrs, uint32_t feature_map_count, uint32_t in_plane,
			bool allow_join = false)
		{
			const bool join = allow_join && (desc.input_count == 2) && (desc.has_add != 0);
			if ((!join && ((desc.input_count != 1) || desc.has_add)) || (feature_map_count == 0))
				return false;
			const uint32_t op_count = desc.arm_op_count[0] + (join ? desc.arm_op_count[1] : 0u) + desc.tail_op_count;
			if (((op_count == 0) && !join) || (op_count > NNF_HIP_MAX_OPS))
				return false;
			pro.op_count = op_count;
			pro.join = join ? 1u : 0u;
			pro.alpha = desc.add_alpha;
			pro.arm_ops[0] = join ? desc.arm_op_count[0] : op_count;
			pro.arm_ops[1] = join ? desc.arm_op_count[1] : 0u;
			pro.fm_count = feature_map_count;
			pro.weighted_count = 0;
			pro.need_exp = 0;
			pro.in_plane_magic = magic_of(in_plane);
			for(uint32_t i = 0; i < op_count; ++i)
			{
				const nnf_hip_op& src = desc.ops[i];
				pro.kind[i] = src.kind;
				pro.f0[i] = src.f0;
				pro.f1[i] = src.f1;
				pro.slot[i] = 2 * pro.weighted_count;
				switch (src.kind)
				{
				case NNF_HIP_OP_BATCH_NORM:
				case NNF_HIP_OP_PRELU:
					{
						const uint32_t j = pro.weighted_count++;
						if (j < prologue_weighted_max)
							pro.weighted_kind[j] = src.kind;
						if ((chunk_ptrs == nullptr) || (src.chunk < 0))
							return false;
						const int chunk_count = (src.kind == NNF_HIP_OP_BATCH_NORM) ? 4 : 1;
						for(int c = 0; c < chunk_count; ++c)
						{
							if (chunk_ptrs[src.chunk + c] == nullptr)
								return false;
							if (j < prologue_weighted_max)
								pro.weights[j][c] = chunk_ptrs[src.chunk + c];
						}
					}
					break;
				case NNF_HIP_OP_TANH:
					pro.f1[i] = src.f1 * 2.0f; // nnforge/plain/hyperbolic_tangent_layer_tester_plain.cpp:49
					pro.need_exp = 1;
					break;
				case NNF_HIP_OP_ELU:
				case NNF_HIP_OP_SIGMOID:
					pro.need_exp = 1;
					break;
				case NNF_HIP_OP_RELU:
				case NNF_HIP_OP_ABSOLUTE:
				case NNF_HIP_OP_DROPOUT:
					break;
				default:
					return false;
				}
			}
			return true;
		}

	}
}
