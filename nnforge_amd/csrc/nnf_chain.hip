// Fused element-wise group kernel: [per-input layers] -> optional Add -> [layers after the join],
// one read of every input tensor and one write of the output, fp32, layout [entry][feature_map][y][x].
//
// Work split: the tensor is a flat array of floats cut into tiles of block_size * U float4s; one
// workgroup per tile. Lane t of the workgroup owns float4s t, t + block_size, ... of the tile, so every
// load and store instruction of a wavefront covers 1 KiB of consecutive memory. A tile spans only a
// few feature-map planes; the per-feature-map coefficients of those planes (batch-norm mult/add,
// PReLU slope) are computed once per workgroup into LDS and looked up by plane index.
#include "nnf_common.h"

namespace nnf
{
	namespace
	{
		constexpr int chain_block_size = 256;
		constexpr int max_slots = NNF_HIP_MAX_OPS;
		constexpr uint32_t exp_table_bytes = exp2_table_size * sizeof(uint64_t);

		struct chain_op
		{
			int32_t kind;
			int32_t slot; // index of the LDS coefficient array of this op, or -1
			float f0;
			float f1;
		};

		struct chain_slot
		{
			const float* p[4]; // batch norm: gamma, beta, mean, inverse sigma; PReLU: slopes
			int32_t kind;
			int32_t reserved;
		};

		struct chain_args
		{
			const float* in[NNF_HIP_MAX_INPUTS];
			float* out;
			uint32_t total;       // elements in the tensor
			uint32_t fm_count;    // C
			uint32_t plane;       // neuron_count_per_feature_map
			uint32_t plane_magic; // ceil(2^32 / plane), used when 2 <= plane < tile
			uint32_t span;        // planes a tile can touch = LDS entries per slot
			uint32_t has_add;
			float alpha;
			uint32_t arm_ops[NNF_HIP_MAX_INPUTS];
			uint32_t tail_ops;
			uint32_t slot_count;
			uint32_t need_exp;
			chain_op ops[NNF_HIP_MAX_OPS];
			chain_slot slots[max_slots];
		};

		// Plane index (relative to the first plane of the tile) of tile-local element offset e,
		// where e already includes the offset of the tile start inside its first plane.
		template<int TILE>
		__device__ __forceinline__ uint32_t plane_of(uint32_t e, uint32_t plane, uint32_t plane_magic)
		{
			if (plane >= static_cast<uint32_t>(TILE))
				return e >= plane ? 1u : 0u; // e < plane + TILE <= 2 * plane
			if (plane == 1)
				return e;
			// e < 2 * TILE <= 2^16 and plane < 2^16: the 32-bit reciprocal is exact for these
			return __umulhi(e, plane_magic);
		}

		// Applies one layer to the U float4s a lane holds. The switch is uniform across the workgroup.
		template<int U, int PL>
		__device__ __forceinline__ void apply_op(
			const chain_op& op,
			float (&v)[U][4],
			const uint32_t (&pl)[U][PL],
			const float2* lds_coeff,
			uint32_t span,
			const uint64_t* lds_exp)
		{
			switch (op.kind)
			{
			case NNF_HIP_OP_BATCH_NORM:
				{
					const float2* coeff = lds_coeff + op.slot * span;
					#pragma unroll
					for(int k = 0; k < U; ++k)
					{
						#pragma unroll
						for(int e = 0; e < 4; ++e)
						{
							const float2 ma = coeff[pl[k][PL == 1 ? 0 : e]];
							v[k][e] = nnf_batch_norm(v[k][e], ma.x, ma.y);
						}
					}
				}
				break;
			case NNF_HIP_OP_RELU:
				#pragma unroll
				for(int k = 0; k < U; ++k)
				{
					#pragma unroll
					for(int e = 0; e < 4; ++e)
						v[k][e] = nnf_rectified_linear(v[k][e], op.f0);
				}
				break;
			case NNF_HIP_OP_PRELU:
				{
					const float2* coeff = lds_coeff + op.slot * span;
					#pragma unroll
					for(int k = 0; k < U; ++k)
					{
						#pragma unroll
						for(int e = 0; e < 4; ++e)
							v[k][e] = nnf_parametric_rectified_linear(v[k][e], coeff[pl[k][PL == 1 ? 0 : e]].x);
					}
				}
				break;
			case NNF_HIP_OP_ELU:
				#pragma unroll
				for(int k = 0; k < U; ++k)
				{
					#pragma unroll
					for(int e = 0; e < 4; ++e)
						v[k][e] = nnf_exponential_linear(v[k][e], lds_exp);
				}
				break;
			case NNF_HIP_OP_SIGMOID:
				#pragma unroll
				for(int k = 0; k < U; ++k)
				{
					#pragma unroll
					for(int e = 0; e < 4; ++e)
						v[k][e] = nnf_sigmoid(v[k][e], lds_exp);
				}
				break;
			case NNF_HIP_OP_TANH:
				#pragma unroll
				for(int k = 0; k < U; ++k)
				{
					#pragma unroll
					for(int e = 0; e < 4; ++e)
						v[k][e] = nnf_hyperbolic_tangent(v[k][e], op.f1, op.f0, lds_exp); // f1 holds steepness * 2
				}
				break;
			default:
				break;
			}
		}

		// NIN: number of input tensors. U: float4s per lane. ALIGNED4: plane % 4 == 0, i.e. a float4 never straddles planes.
		template<int NIN, int U, bool ALIGNED4>
		__global__ void __launch_bounds__(chain_block_size) chain_kernel(const chain_args a)
		{
			constexpr int TILE = chain_block_size * U * 4;
			constexpr int PL = ALIGNED4 ? 1 : 4;
			extern __shared__ __align__(16) unsigned char lds_raw[];
			uint64_t* lds_exp = reinterpret_cast<uint64_t*>(lds_raw);
			float2* lds_coeff = reinterpret_cast<float2*>(lds_raw + exp_table_bytes);

			const uint32_t tile_start = blockIdx.x * static_cast<uint32_t>(TILE);
			const uint32_t first_plane = tile_start / a.plane;
			const uint32_t start_in_plane = tile_start - first_plane * a.plane;
			const uint32_t first_fm = first_plane % a.fm_count;

			// issue all loads first: they are what the kernel waits for
			float x[NIN][U][4];
			#pragma unroll
			for(int j = 0; j < NIN; ++j)
			{
				#pragma unroll
				for(int k = 0; k < U; ++k)
				{
					const uint32_t idx = tile_start + (threadIdx.x + k * chain_block_size) * 4;
					if (idx + 3 < a.total)
					{
						const floatx4 t = load_stream(reinterpret_cast<const floatx4*>(a.in[j] + idx));
						x[j][k][0] = t.x; x[j][k][1] = t.y; x[j][k][2] = t.z; x[j][k][3] = t.w;
					}
					else
					{
						#pragma unroll
						for(int e = 0; e < 4; ++e)
							x[j][k][e] = (idx + e < a.total) ? a.in[j][idx + e] : 0.0f;
					}
				}
			}

			// per-feature-map coefficients of the planes this tile touches
			if (a.need_exp)
				stage_exp2_table(lds_exp);
			for(uint32_t s = 0; s < a.slot_count; ++s)
			{
				const chain_slot& slot = a.slots[s];
				for(uint32_t i = threadIdx.x; i < a.span; i += chain_block_size)
				{
					const uint32_t fm = (first_fm + i) % a.fm_count;
					float2 c;
					if (slot.kind == NNF_HIP_OP_BATCH_NORM)
						nnf_batch_norm_coefficients(slot.p[0][fm], slot.p[1][fm], slot.p[2][fm], slot.p[3][fm], c.x, c.y);
					else
					{
						c.x = slot.p[0][fm];
						c.y = 0.0f;
					}
					lds_coeff[s * a.span + i] = c;
				}
			}
			__syncthreads();

			uint32_t pl[U][PL];
			#pragma unroll
			for(int k = 0; k < U; ++k)
			{
				const uint32_t e0 = start_in_plane + (threadIdx.x + k * chain_block_size) * 4;
				#pragma unroll
				for(int e = 0; e < PL; ++e)
					pl[k][e] = plane_of<TILE>(e0 + e, a.plane, a.plane_magic);
			}

			uint32_t op_index = 0;
			#pragma unroll
			for(int j = 0; j < NIN; ++j)
			{
				const uint32_t arm_end = op_index + a.arm_ops[j];
				for(; op_index < arm_end; ++op_index)
					apply_op<U, PL>(a.ops[op_index], x[j], pl, lds_coeff, a.span, lds_exp);
			}

			if (a.has_add)
			{
				// nnforge/plain/add_layer_tester_plain.cpp:56-59: sum starts at 0.0F
				#pragma unroll
				for(int k = 0; k < U; ++k)
				{
					#pragma unroll
					for(int e = 0; e < 4; ++e)
					{
						float sum = 0.0f + x[0][k][e];
						#pragma unroll
						for(int j = 1; j < NIN; ++j)
							sum = sum + x[j][k][e];
						x[0][k][e] = sum * a.alpha;
					}
				}
			}

			const uint32_t tail_end = op_index + a.tail_ops;
			for(; op_index < tail_end; ++op_index)
				apply_op<U, PL>(a.ops[op_index], x[0], pl, lds_coeff, a.span, lds_exp);

			#pragma unroll
			for(int k = 0; k < U; ++k)
			{
				const uint32_t idx = tile_start + (threadIdx.x + k * chain_block_size) * 4;
				if (idx + 3 < a.total)
				{
					floatx4 t;
					t.x = x[0][k][0]; t.y = x[0][k][1]; t.z = x[0][k][2]; t.w = x[0][k][3];
					store_stream(reinterpret_cast<floatx4*>(a.out + idx), t);
				}
				else
				{
					#pragma unroll
					for(int e = 0; e < 4; ++e)
						if (idx + e < a.total)
							a.out[idx + e] = x[0][k][e];
				}
			}
		}

		typedef void (*chain_kernel_fn)(const chain_args);

		template<int NIN, int U>
		chain_kernel_fn pick_aligned(bool aligned4)
		{
			return aligned4 ? chain_kernel<NIN, U, true> : chain_kernel<NIN, U, false>;
		}

		template<int NIN>
		chain_kernel_fn pick_unroll(int unroll, bool aligned4)
		{
			switch (unroll)
			{
			case 4: return pick_aligned<NIN, 4>(aligned4);
			case 2: return pick_aligned<NIN, 2>(aligned4);
			default: return pick_aligned<NIN, 1>(aligned4);
			}
		}

		chain_kernel_fn pick_kernel(uint32_t input_count, int unroll, bool aligned4)
		{
			switch (input_count)
			{
			case 1: return pick_unroll<1>(unroll, aligned4);
			case 2: return pick_unroll<2>(unroll, aligned4);
			case 3: return pick_unroll<3>(unroll, aligned4);
			default: return pick_unroll<4>(unroll, aligned4);
			}
		}

		bool ranges_overlap(const void* a, const void* b, size_t bytes)
		{
			const uintptr_t pa = reinterpret_cast<uintptr_t>(a);
			const uintptr_t pb = reinterpret_cast<uintptr_t>(b);
			return (pa < pb + bytes) && (pb < pa + bytes);
		}

		constexpr size_t max_dynamic_lds = 64 * 1024;
		// Below this many tiles a smaller tile is used so that more compute units get work.
		constexpr uint32_t min_tiles_wanted = 1024;
	}

	int chain_forward(hipStream_t stream, const nnf_hip_chain_desc* desc, float* output,
		const float* const* inputs, const float* const* chunk_ptrs)
	{
		if ((desc == nullptr) || (output == nullptr) || (inputs == nullptr))
			return NNF_HIP_EINVAL;
		if ((desc->feature_map_count == 0) || (desc->neuron_count_per_feature_map == 0))
			return NNF_HIP_EINVAL;
		if ((desc->input_count < 1) || (desc->input_count > NNF_HIP_MAX_INPUTS))
			return NNF_HIP_EINVAL;
		if ((desc->input_count > 1) && !desc->has_add)
			return NNF_HIP_EINVAL;

		uint32_t op_count = desc->tail_op_count;
		for(uint32_t j = 0; j < NNF_HIP_MAX_INPUTS; ++j)
		{
			if ((j >= desc->input_count) && (desc->arm_op_count[j] != 0))
				return NNF_HIP_EINVAL;
			op_count += desc->arm_op_count[j];
		}
		if (op_count > NNF_HIP_MAX_OPS)
			return NNF_HIP_EINVAL;

		const uint64_t total64 = static_cast<uint64_t>(desc->entry_count) * desc->feature_map_count * desc->neuron_count_per_feature_map;
		if (total64 == 0)
			return NNF_HIP_OK; // nothing to do, as the reference's loops over zero elements
		if (total64 > 0xFFFF0000ull)
			return NNF_HIP_ETOOBIG;
		const size_t bytes = static_cast<size_t>(total64) * sizeof(float);

		chain_args a = {};
		if (!is_aligned16(output))
			return NNF_HIP_EALIGN;
		for(uint32_t j = 0; j < desc->input_count; ++j)
		{
			if (inputs[j] == nullptr)
				return NNF_HIP_EINVAL;
			if (!is_aligned16(inputs[j]))
				return NNF_HIP_EALIGN;
			const bool exact_alias_of_first = (j == 0) && (inputs[j] == output);
			if (!exact_alias_of_first && ranges_overlap(inputs[j], output, bytes))
				return NNF_HIP_EOVERLAP;
			a.in[j] = inputs[j];
		}
		a.out = output;
		a.total = static_cast<uint32_t>(total64);
		a.fm_count = desc->feature_map_count;
		a.plane = desc->neuron_count_per_feature_map;
		a.has_add = desc->has_add ? 1u : 0u;
		a.alpha = desc->add_alpha;
		for(uint32_t j = 0; j < NNF_HIP_MAX_INPUTS; ++j)
			a.arm_ops[j] = desc->arm_op_count[j];
		a.tail_ops = desc->tail_op_count;

		for(uint32_t i = 0; i < op_count; ++i)
		{
			const nnf_hip_op& src = desc->ops[i];
			chain_op& dst = a.ops[i];
			dst.kind = src.kind;
			dst.slot = -1;
			dst.f0 = src.f0;
			dst.f1 = src.f1;
			switch (src.kind)
			{
			case NNF_HIP_OP_BATCH_NORM:
			case NNF_HIP_OP_PRELU:
				{
					if ((chunk_ptrs == nullptr) || (src.chunk < 0))
						return NNF_HIP_EINVAL;
					const int chunk_count = (src.kind == NNF_HIP_OP_BATCH_NORM) ? 4 : 1;
					chain_slot& slot = a.slots[a.slot_count];
					for(int c = 0; c < chunk_count; ++c)
					{
						if (chunk_ptrs[src.chunk + c] == nullptr)
							return NNF_HIP_EINVAL;
						slot.p[c] = chunk_ptrs[src.chunk + c];
					}
					slot.kind = src.kind;
					dst.slot = static_cast<int32_t>(a.slot_count);
					++a.slot_count;
				}
				break;
			case NNF_HIP_OP_RELU:
				break;
			case NNF_HIP_OP_TANH:
				// nnforge/plain/hyperbolic_tangent_layer_tester_plain.cpp:49: steepness * 2.0F, rounded once on the host
				dst.f1 = src.f1 * 2.0f;
				a.need_exp = 1;
				break;
			case NNF_HIP_OP_ELU:
			case NNF_HIP_OP_SIGMOID:
				a.need_exp = 1;
				break;
			default:
				return NNF_HIP_EINVAL;
			}
		}

		// tile size: as large as keeps the coefficient arrays inside LDS and the grid wide enough
		int unroll = 4;
		size_t lds_bytes = 0;
		for(;; unroll /= 2)
		{
			const uint32_t tile = chain_block_size * unroll * 4;
			a.span = (tile + a.plane - 2) / a.plane + 1;
			lds_bytes = exp_table_bytes + static_cast<size_t>(a.slot_count) * a.span * sizeof(float2);
			const uint32_t tiles = (a.total + tile - 1) / tile;
			const bool fits = lds_bytes <= max_dynamic_lds;
			if (unroll == 1)
			{
				if (!fits)
					return NNF_HIP_EUNSUPPORTED;
				break;
			}
			if (fits && (tiles >= min_tiles_wanted))
				break;
		}
		const uint32_t tile = chain_block_size * unroll * 4;
		a.plane_magic = (a.plane >= 2) ? static_cast<uint32_t>(((1ull << 32) + a.plane - 1) / a.plane) : 0u;
		const uint32_t tiles = (a.total + tile - 1) / tile;
		const bool aligned4 = (a.plane % 4) == 0;

		chain_kernel_fn kernel = pick_kernel(desc->input_count, unroll, aligned4);
		hipLaunchKernelGGL(kernel, dim3(tiles), dim3(chain_block_size), lds_bytes, stream, a);
		return launch_status();
	}
}
