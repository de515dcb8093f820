// extern "C" surface of the library (declared in include/nnforge_hip.h): argument checks,
// single-layer wrappers around the fused-group kernel, and the runtime plumbing (memory, streams,
// events) that lets host C++ above this ABI stay free of HIP headers.
#include "nnf_common.h"

#include <algorithm>
#include <cstring>

namespace nnf
{
	namespace
	{
		constexpr int copy_block_size = 256;
		constexpr int copy_unroll = 4;

		// same tiling as the chain kernel: lane t moves float4s t, t + 256, ... of a 16 KiB tile
		__global__ void __launch_bounds__(copy_block_size) copy_kernel_impl(floatx4* dst, const floatx4* src, uint32_t vectors)
		{
			const uint32_t tile_start = blockIdx.x * (copy_block_size * copy_unroll);
			floatx4 v[copy_unroll];
			#pragma unroll
			for(int k = 0; k < copy_unroll; ++k)
			{
				const uint32_t i = tile_start + threadIdx.x + k * copy_block_size;
				if (i < vectors)
					v[k] = load_stream(src + i);
			}
			#pragma unroll
			for(int k = 0; k < copy_unroll; ++k)
			{
				const uint32_t i = tile_start + threadIdx.x + k * copy_block_size;
				if (i < vectors)
					store_stream(dst + i, v[k]);
			}
		}

		// Sweep behind nnf_hip_check_division_sequences: lane-strided over the bit patterns of every
		// non-negative float e with e + 1 <= 2^126.
		__global__ void __launch_bounds__(256) division_check_kernel(unsigned long long* mismatches)
		{
			constexpr uint32_t last_bits = 0x7E800000u; // 2^126
			unsigned long long bad_reciprocal = 0, bad_quotient = 0;
			const uint64_t stride = static_cast<uint64_t>(gridDim.x) * blockDim.x;
			for(uint64_t u = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x; u <= last_bits; u += stride)
			{
				const float e = __uint_as_float(static_cast<uint32_t>(u));
				const float d = e + 1.0f;
				if (!(d <= 0x1p126f))
					continue;
				const float n = e - 1.0f;
				bad_reciprocal += __float_as_uint(nnf_fast_reciprocal_of_ge1(d)) != __float_as_uint(1.0f / d);
				bad_quotient += __float_as_uint(nnf_fast_tanh_quotient(n, d)) != __float_as_uint(n / d);
			}
			if (bad_reciprocal != 0)
				atomicAdd(&mismatches[0], bad_reciprocal);
			if (bad_quotient != 0)
				atomicAdd(&mismatches[1], bad_quotient);
		}

		nnf_hip_chain_desc single_op_desc(uint32_t entry_count, uint32_t fm_count, uint32_t plane, int32_t kind, int32_t chunk, float f0, float f1)
		{
			nnf_hip_chain_desc d;
			std::memset(&d, 0, sizeof(d));
			d.entry_count = entry_count;
			d.feature_map_count = fm_count;
			d.neuron_count_per_feature_map = plane;
			d.input_count = 1;
			d.add_alpha = 1.0f;
			d.arm_op_count[0] = 1;
			d.ops[0].kind = kind;
			d.ops[0].chunk = chunk;
			d.ops[0].f0 = f0;
			d.ops[0].f1 = f1;
			return d;
		}

		// Layers without per-feature-map weights see the tensor as a flat array
		// (e.g. nnforge/plain/rectified_linear_layer_tester_plain.cpp:47): split elem_count into a shape
		// the fused-group kernel accepts.
		bool flat_shape(uint64_t elem_count, uint32_t& entry_count, uint32_t& plane)
		{
			if (elem_count > NNF_HIP_MAX_ELEMENT_COUNT)
				return false;
			entry_count = 1;
			plane = static_cast<uint32_t>(elem_count);
			return true;
		}

		int flat_op(hipStream_t stream, float* output, const float* input, uint64_t elem_count, int32_t kind, float f0, float f1)
		{
			if (elem_count == 0)
				return ((output == nullptr) || (input == nullptr)) ? NNF_HIP_EINVAL : NNF_HIP_OK;
			uint32_t entry_count, plane;
			if (!flat_shape(elem_count, entry_count, plane))
				return NNF_HIP_ETOOBIG;
			const nnf_hip_chain_desc d = single_op_desc(entry_count, 1, plane, kind, 0, f0, f1);
			const float* inputs[1] = { input };
			return chain_forward(stream, &d, output, inputs, nullptr);
		}
	}

	int copy_kernel(hipStream_t stream, void* dst, const void* src, size_t bytes)
	{
		if ((dst == nullptr) || (src == nullptr) || ((bytes % 16) != 0))
			return NNF_HIP_EINVAL;
		if (!is_aligned16(dst) || !is_aligned16(src))
			return NNF_HIP_EALIGN;
		if (bytes == 0)
			return NNF_HIP_OK;
		if (bytes / 16 > NNF_HIP_MAX_ELEMENT_COUNT)
			return NNF_HIP_ETOOBIG;
		const uint32_t vectors = static_cast<uint32_t>(bytes / 16);
		const uint32_t per_block = copy_block_size * copy_unroll;
		NNF_LAUNCH(copy_kernel_impl, dim3((vectors + per_block - 1) / per_block), dim3(copy_block_size), 0, stream,
			static_cast<floatx4*>(dst), static_cast<const floatx4*>(src), vectors);
		return launch_status();
	}
}

using namespace nnf;

extern "C"
{
	int nnf_hip_chain_forward(void* stream, const nnf_hip_chain_desc* desc, float* output,
		const float* const* inputs, const float* const* chunk_ptrs)
	{
		return chain_forward(static_cast<hipStream_t>(stream), desc, output, inputs, chunk_ptrs);
	}

	int nnf_hip_chain_forward_batch(void* stream, uint32_t group_count, const nnf_hip_chain_desc* descs, float* const* outputs,
		const float* const* const* inputs, const float* const* const* chunk_ptrs)
	{
		return chain_forward_batch(static_cast<hipStream_t>(stream), group_count, descs, outputs, inputs, chunk_ptrs);
	}

	int nnf_hip_chain_forward_strided(void* stream, const nnf_hip_chain_desc* desc, float* output, uint32_t output_entry_stride,
		const float* const* inputs, const float* const* chunk_ptrs)
	{
		return chain_forward_strided(static_cast<hipStream_t>(stream), desc, output, output_entry_stride, inputs, chunk_ptrs);
	}

	int nnf_hip_chain_forward_strided_batch(void* stream, uint32_t group_count, const nnf_hip_chain_desc* descs,
		float* const* outputs, const uint32_t* output_entry_strides, const float* const* const* inputs, const float* const* const* chunk_ptrs)
	{
		return chain_forward_strided_batch(static_cast<hipStream_t>(stream), group_count, descs, outputs, output_entry_strides, inputs, chunk_ptrs);
	}

	int nnf_hip_chain_forward_strided_status(const nnf_hip_chain_desc* desc, uint32_t output_entry_stride)
	{
		return chain_forward_strided_status(desc, output_entry_stride);
	}

	int nnf_hip_batch_norm_forward(void* stream, float* output, const float* input,
		const float* gamma, const float* beta, const float* mean, const float* inverse_sigma,
		uint32_t entry_count, uint32_t feature_map_count, uint32_t neuron_count_per_feature_map)
	{
		const nnf_hip_chain_desc d = single_op_desc(entry_count, feature_map_count, neuron_count_per_feature_map, NNF_HIP_OP_BATCH_NORM, 0, 0.0f, 0.0f);
		const float* inputs[1] = { input };
		const float* chunks[4] = { gamma, beta, mean, inverse_sigma };
		return chain_forward(static_cast<hipStream_t>(stream), &d, output, inputs, chunks);
	}

	int nnf_hip_rectified_linear_forward(void* stream, float* output, const float* input, float negative_slope, uint64_t elem_count)
	{
		return flat_op(static_cast<hipStream_t>(stream), output, input, elem_count, NNF_HIP_OP_RELU, negative_slope, 0.0f);
	}

	int nnf_hip_parametric_rectified_linear_forward(void* stream, float* output, const float* input,
		const float* slopes, uint32_t entry_count, uint32_t feature_map_count, uint32_t neuron_count_per_feature_map)
	{
		const nnf_hip_chain_desc d = single_op_desc(entry_count, feature_map_count, neuron_count_per_feature_map, NNF_HIP_OP_PRELU, 0, 0.0f, 0.0f);
		const float* inputs[1] = { input };
		const float* chunks[1] = { slopes };
		return chain_forward(static_cast<hipStream_t>(stream), &d, output, inputs, chunks);
	}

	int nnf_hip_exponential_linear_forward(void* stream, float* output, const float* input, uint64_t elem_count)
	{
		return flat_op(static_cast<hipStream_t>(stream), output, input, elem_count, NNF_HIP_OP_ELU, 0.0f, 0.0f);
	}

	int nnf_hip_sigmoid_forward(void* stream, float* output, const float* input, uint64_t elem_count)
	{
		return flat_op(static_cast<hipStream_t>(stream), output, input, elem_count, NNF_HIP_OP_SIGMOID, 0.0f, 0.0f);
	}

	int nnf_hip_hyperbolic_tangent_forward(void* stream, float* output, const float* input, float scale, float steepness, uint64_t elem_count)
	{
		return flat_op(static_cast<hipStream_t>(stream), output, input, elem_count, NNF_HIP_OP_TANH, scale, steepness);
	}

	int nnf_hip_absolute_forward(void* stream, float* output, const float* input, uint64_t elem_count)
	{
		return flat_op(static_cast<hipStream_t>(stream), output, input, elem_count, NNF_HIP_OP_ABSOLUTE, 0.0f, 0.0f);
	}

	int nnf_hip_dropout_forward(void* stream, float* output, const float* input, uint64_t elem_count)
	{
		if ((output != nullptr) && (output == input))
			return NNF_HIP_OK; // in place: nothing to move
		return flat_op(static_cast<hipStream_t>(stream), output, input, elem_count, NNF_HIP_OP_DROPOUT, 0.0f, 0.0f);
	}

	int nnf_hip_concat_forward(void* stream, float* output, const float* const* inputs,
		const uint32_t* input_neuron_counts, uint32_t input_count, uint32_t entry_count)
	{
		return concat_forward(static_cast<hipStream_t>(stream), output, inputs, input_neuron_counts, nullptr, input_count, entry_count);
	}

	int nnf_hip_concat_forward_partial(void* stream, float* output, const float* const* inputs,
		const uint32_t* input_neuron_counts, const uint8_t* inputs_in_place, uint32_t input_count, uint32_t entry_count)
	{
		return concat_forward(static_cast<hipStream_t>(stream), output, inputs, input_neuron_counts, inputs_in_place, input_count, entry_count);
	}

	int nnf_hip_maxout_forward(void* stream, float* output, const float* input,
		uint32_t entry_count, uint32_t output_feature_map_count, uint32_t neuron_count_per_feature_map,
		uint32_t feature_map_subsampling_size)
	{
		return maxout_forward(static_cast<hipStream_t>(stream), output, input, entry_count, output_feature_map_count,
			neuron_count_per_feature_map, feature_map_subsampling_size);
	}

	int nnf_hip_max_subsampling_forward(void* stream, float* output, const float* input,
		uint32_t output_entry_count, uint32_t input_feature_map_count, uint32_t dimension_count,
		const uint32_t* input_sizes, const uint32_t* subsampling_sizes, const uint32_t* strides, const uint32_t* round_ups,
		uint32_t feature_map_subsampling_size, uint32_t entry_subsampling_size, int32_t is_min)
	{
		return max_subsampling_forward(static_cast<hipStream_t>(stream), output, input, output_entry_count, input_feature_map_count,
			dimension_count, input_sizes, subsampling_sizes, strides, round_ups, feature_map_subsampling_size, entry_subsampling_size, is_min);
	}

	int nnf_hip_feature_map_stat_init(void* stream, nnf_hip_running_stat* device_stats, uint32_t feature_map_count)
	{
		return feature_map_stat_init(static_cast<hipStream_t>(stream), device_stats, feature_map_count);
	}

	int nnf_hip_feature_map_stat_workspace_bytes(uint32_t entry_count, uint32_t feature_map_count, uint32_t neuron_count_per_feature_map, size_t* bytes)
	{
		return feature_map_stat_workspace_bytes(entry_count, feature_map_count, neuron_count_per_feature_map, bytes);
	}

	int nnf_hip_feature_map_stat_partial_count(uint32_t entry_count, uint32_t feature_map_count, uint32_t neuron_count_per_feature_map,
		size_t workspace_bytes, uint32_t* partial_states)
	{
		return feature_map_stat_partial_count(entry_count, feature_map_count, neuron_count_per_feature_map, workspace_bytes, partial_states);
	}

	int nnf_hip_feature_map_stat_accumulate(void* stream, nnf_hip_running_stat* device_stats, void* device_workspace, size_t workspace_bytes,
		const float* input, uint32_t entry_count, uint32_t feature_map_count, uint32_t neuron_count_per_feature_map)
	{
		return feature_map_stat_accumulate(static_cast<hipStream_t>(stream), device_stats, device_workspace, workspace_bytes, input,
			entry_count, feature_map_count, neuron_count_per_feature_map);
	}

	int nnf_hip_feature_map_stat_accumulate_static(void* stream, nnf_hip_running_stat* device_stats,
		const float* input, uint32_t entry_count, uint32_t feature_map_count, uint32_t neuron_count_per_feature_map)
	{
		return feature_map_stat_accumulate_static(static_cast<hipStream_t>(stream), device_stats, input,
			entry_count, feature_map_count, neuron_count_per_feature_map);
	}

	int nnf_hip_add_forward(void* stream, float* output, const float* const* inputs, uint32_t input_count, float alpha, uint64_t elem_count)
	{
		if ((inputs == nullptr) || (input_count == 0) || (output == nullptr))
			return NNF_HIP_EINVAL;
		if (elem_count == 0)
			return NNF_HIP_OK;
		uint32_t entry_count, plane;
		if (!flat_shape(elem_count, entry_count, plane))
			return NNF_HIP_ETOOBIG;
		// The output may alias inputs[0] only; a later input that overlaps the output would be
		// clobbered by the first partial launch, so it is rejected here for every input_count.
		for(uint32_t j = 1; j < input_count; ++j)
		{
			if (inputs[j] == nullptr)
				return NNF_HIP_EINVAL;
			const uintptr_t a = reinterpret_cast<uintptr_t>(output), b = reinterpret_cast<uintptr_t>(inputs[j]);
			const size_t bytes = static_cast<size_t>(elem_count) * sizeof(float);
			if ((a < b + bytes) && (b < a + bytes))
				return NNF_HIP_EOVERLAP;
		}

		// Left-to-right sum in groups of NNF_HIP_MAX_INPUTS: the partial sum (alpha = 1) becomes the
		// first input of the next group. 0.0F + partial == partial bit for bit (a sum that started
		// from +0.0F is never -0.0F), so the grouping does not change the result.
		nnf_hip_chain_desc d;
		std::memset(&d, 0, sizeof(d));
		d.entry_count = entry_count;
		d.feature_map_count = 1;
		d.neuron_count_per_feature_map = plane;
		d.has_add = 1;
		uint32_t done = 0;
		const float* group[NNF_HIP_MAX_INPUTS];
		while (done < input_count)
		{
			uint32_t n = 0;
			if (done > 0)
				group[n++] = output;
			while ((n < NNF_HIP_MAX_INPUTS) && (done < input_count))
				group[n++] = inputs[done++];
			d.input_count = n;
			d.add_alpha = (done == input_count) ? alpha : 1.0f;
			const int rc = chain_forward(static_cast<hipStream_t>(stream), &d, output, group, nullptr);
			if (rc != NNF_HIP_OK)
				return rc;
		}
		return NNF_HIP_OK;
	}

	int nnf_hip_softmax_forward(void* stream, float* output, const float* input,
		uint32_t entry_count, uint32_t feature_map_count, uint32_t neuron_count_per_feature_map)
	{
		return softmax_forward(static_cast<hipStream_t>(stream), output, input, entry_count, feature_map_count, neuron_count_per_feature_map);
	}

	int nnf_hip_average_subsampling_forward(void* stream, float* output, const float* input,
		uint32_t entry_count, uint32_t feature_map_count, uint32_t input_width, uint32_t input_height,
		uint32_t window_width, uint32_t window_height, float mult)
	{
		return average_subsampling_forward(static_cast<hipStream_t>(stream), output, input, entry_count, feature_map_count,
			input_width, input_height, window_width, window_height, mult);
	}

	int nnf_hip_check_division_sequences(void* stream, uint64_t* device_mismatch_counts)
	{
		if (device_mismatch_counts == nullptr)
			return NNF_HIP_EINVAL;
		static_assert(sizeof(unsigned long long) == sizeof(uint64_t), "counter width");
		NNF_LAUNCH(division_check_kernel, dim3(4096), dim3(256), 0, static_cast<hipStream_t>(stream),
			reinterpret_cast<unsigned long long*>(device_mismatch_counts));
		return launch_status();
	}

	int nnf_hip_average_subsampling_nd_forward(void* stream, float* output, const float* input,
		uint32_t output_entry_count, uint32_t input_feature_map_count, uint32_t dimension_count,
		const uint32_t* input_sizes, const uint32_t* subsampling_sizes,
		uint32_t feature_map_subsampling_size, uint32_t entry_subsampling_size, float mult)
	{
		return average_subsampling_nd_forward(static_cast<hipStream_t>(stream), output, input, output_entry_count, input_feature_map_count,
			dimension_count, input_sizes, subsampling_sizes, feature_map_subsampling_size, entry_subsampling_size, mult);
	}

	int nnf_hip_max_subsampling_tiling_forward(void* stream, float* output, const float* input,
		uint32_t input_entry_count, uint32_t feature_map_count, uint32_t dimension_count,
		const uint32_t* input_sizes, const uint32_t* subsampling_sizes, int32_t is_min)
	{
		return max_subsampling_tiling_forward(static_cast<hipStream_t>(stream), output, input, input_entry_count, feature_map_count,
			dimension_count, input_sizes, subsampling_sizes, is_min);
	}

	int nnf_hip_max_subsampling_fused_forward(void* stream, float* output, const float* input,
		const nnf_hip_chain_desc* prologue, const float* const* chunk_ptrs,
		uint32_t output_entry_count, uint32_t input_feature_map_count, uint32_t dimension_count,
		const uint32_t* input_sizes, const uint32_t* subsampling_sizes, const uint32_t* strides, const uint32_t* round_ups,
		uint32_t feature_map_subsampling_size, uint32_t entry_subsampling_size, int32_t is_min)
	{
		if ((prologue == nullptr) || (prologue->feature_map_count != input_feature_map_count))
			return NNF_HIP_EINVAL;
		if ((input_sizes != nullptr) && (dimension_count >= 1) && (dimension_count <= 4))
		{
			uint64_t plane = 1;
			for(uint32_t i = 0; i < dimension_count; ++i)
				plane *= input_sizes[i];
			if (plane != prologue->neuron_count_per_feature_map)
				return NNF_HIP_EINVAL;
		}
		if (const int rc = prologue_status(*prologue, chunk_ptrs))
			return rc;
		return max_subsampling_forward_with_prologue(static_cast<hipStream_t>(stream), output, input, output_entry_count, input_feature_map_count,
			dimension_count, input_sizes, subsampling_sizes, strides, round_ups, feature_map_subsampling_size, entry_subsampling_size, is_min,
			prologue, chunk_ptrs, false);
	}

	int nnf_hip_average_subsampling_fused_forward(void* stream, float* output, const float* input,
		const nnf_hip_chain_desc* prologue, const float* const* chunk_ptrs,
		uint32_t entry_count, uint32_t feature_map_count, uint32_t input_width, uint32_t input_height,
		uint32_t window_width, uint32_t window_height, float mult)
	{
		if ((prologue == nullptr) || (prologue->feature_map_count != feature_map_count)
			|| (static_cast<uint64_t>(input_width) * input_height != prologue->neuron_count_per_feature_map))
			return NNF_HIP_EINVAL;
		if (const int rc = prologue_status(*prologue, chunk_ptrs))
			return rc;
		return average_subsampling_forward_with_prologue(static_cast<hipStream_t>(stream), output, input, nullptr, entry_count, feature_map_count,
			input_width, input_height, window_width, window_height, mult, prologue, chunk_ptrs, false);
	}

	int nnf_hip_average_subsampling_joined_forward(void* stream, float* output, const float* const* inputs,
		const nnf_hip_chain_desc* prologue, const float* const* chunk_ptrs,
		uint32_t entry_count, uint32_t feature_map_count, uint32_t input_width, uint32_t input_height,
		uint32_t window_width, uint32_t window_height, float mult)
	{
		if ((prologue == nullptr) || (inputs == nullptr) || (prologue->input_count != 2) || (prologue->has_add == 0)
			|| (prologue->feature_map_count != feature_map_count)
			|| (static_cast<uint64_t>(input_width) * input_height != prologue->neuron_count_per_feature_map))
			return NNF_HIP_EINVAL;
		if (const int rc = prologue_status(*prologue, chunk_ptrs, true))
			return rc;
		return average_subsampling_forward_with_prologue(static_cast<hipStream_t>(stream), output, inputs[0], inputs[1], entry_count, feature_map_count,
			input_width, input_height, window_width, window_height, mult, prologue, chunk_ptrs, false);
	}

	namespace
	{
		// any single-layer group: the shape checks do not depend on which layers the prologue holds
		nnf_hip_chain_desc planning_prologue(uint32_t feature_map_count)
		{
			nnf_hip_chain_desc d;
			std::memset(&d, 0, sizeof(d));
			d.feature_map_count = feature_map_count;
			d.input_count = 1;
			d.arm_op_count[0] = 1;
			d.ops[0].kind = NNF_HIP_OP_ABSOLUTE;
			return d;
		}
	}

	int nnf_hip_max_subsampling_fusable(uint32_t output_entry_count, uint32_t input_feature_map_count, uint32_t dimension_count,
		const uint32_t* input_sizes, const uint32_t* subsampling_sizes, const uint32_t* strides, const uint32_t* round_ups,
		uint32_t feature_map_subsampling_size, uint32_t entry_subsampling_size)
	{
		const nnf_hip_chain_desc d = planning_prologue(input_feature_map_count);
		return max_subsampling_forward_with_prologue(nullptr, nullptr, nullptr, std::max(1u, output_entry_count), input_feature_map_count, dimension_count,
			input_sizes, subsampling_sizes, strides, round_ups, feature_map_subsampling_size, entry_subsampling_size, 0, &d, nullptr, true);
	}

	int nnf_hip_average_subsampling_fusable(uint32_t entry_count, uint32_t feature_map_count, uint32_t input_width, uint32_t input_height,
		uint32_t window_width, uint32_t window_height)
	{
		const nnf_hip_chain_desc d = planning_prologue(feature_map_count);
		return average_subsampling_forward_with_prologue(nullptr, nullptr, nullptr, nullptr, std::max(1u, entry_count), feature_map_count, input_width, input_height,
			window_width, window_height, 1.0f, &d, nullptr, true);
	}

	int nnf_hip_average_subsampling_joinable(uint32_t entry_count, uint32_t feature_map_count, uint32_t input_width, uint32_t input_height,
		uint32_t window_width, uint32_t window_height)
	{
		nnf_hip_chain_desc d = planning_prologue(feature_map_count);
		d.input_count = 2;
		d.has_add = 1;
		d.add_alpha = 1.0f;
		return average_subsampling_forward_with_prologue(nullptr, nullptr, nullptr, nullptr, std::max(1u, entry_count), feature_map_count, input_width, input_height,
			window_width, window_height, 1.0f, &d, nullptr, true);
	}

	int nnf_hip_copy_kernel(void* stream, void* device_dst, const void* device_src, size_t bytes)
	{
		return copy_kernel(static_cast<hipStream_t>(stream), device_dst, device_src, bytes);
	}

	// ---- runtime plumbing ------------------------------------------------------------------

	int nnf_hip_device_count(int* count)
	{
		if (count == nullptr)
			return NNF_HIP_EINVAL;
		return hip_status(hipGetDeviceCount(count));
	}

	int nnf_hip_set_device(int device_id)
	{
		return hip_status(hipSetDevice(device_id));
	}

	int nnf_hip_device_info(int device_id, char* name, size_t name_capacity, uint64_t* global_memory_bytes,
		uint32_t* compute_unit_count, uint32_t* wavefront_size, uint32_t* clock_khz)
	{
		hipDeviceProp_t prop;
		const hipError_t e = hipGetDeviceProperties(&prop, device_id);
		if (e != hipSuccess)
			return hip_status(e);
		if ((name != nullptr) && (name_capacity > 0))
		{
			std::strncpy(name, prop.name, name_capacity - 1);
			name[name_capacity - 1] = '\0';
		}
		if (global_memory_bytes != nullptr)
			*global_memory_bytes = prop.totalGlobalMem;
		if (compute_unit_count != nullptr)
			*compute_unit_count = static_cast<uint32_t>(prop.multiProcessorCount);
		if (wavefront_size != nullptr)
			*wavefront_size = static_cast<uint32_t>(prop.warpSize);
		if (clock_khz != nullptr)
			*clock_khz = static_cast<uint32_t>(prop.clockRate);
		return NNF_HIP_OK;
	}

	int nnf_hip_malloc(void** device_ptr, size_t bytes)
	{
		if (device_ptr == nullptr)
			return NNF_HIP_EINVAL;
		const size_t padded = (bytes + 15) & ~static_cast<size_t>(15);
		return hip_status(hipMalloc(device_ptr, padded == 0 ? 16 : padded));
	}

	int nnf_hip_free(void* device_ptr)
	{
		return hip_status(hipFree(device_ptr));
	}

	int nnf_hip_memcpy_h2d(void* device_dst, const void* host_src, size_t bytes, void* stream)
	{
		if (stream == nullptr)
			return hip_status(hipMemcpy(device_dst, host_src, bytes, hipMemcpyHostToDevice));
		return hip_status(hipMemcpyAsync(device_dst, host_src, bytes, hipMemcpyHostToDevice, static_cast<hipStream_t>(stream)));
	}

	int nnf_hip_memcpy_d2h(void* host_dst, const void* device_src, size_t bytes, void* stream)
	{
		if (stream == nullptr)
			return hip_status(hipMemcpy(host_dst, device_src, bytes, hipMemcpyDeviceToHost));
		return hip_status(hipMemcpyAsync(host_dst, device_src, bytes, hipMemcpyDeviceToHost, static_cast<hipStream_t>(stream)));
	}

	int nnf_hip_memcpy_d2d(void* device_dst, const void* device_src, size_t bytes, void* stream)
	{
		if (stream == nullptr)
			return hip_status(hipMemcpy(device_dst, device_src, bytes, hipMemcpyDeviceToDevice));
		return hip_status(hipMemcpyAsync(device_dst, device_src, bytes, hipMemcpyDeviceToDevice, static_cast<hipStream_t>(stream)));
	}

	int nnf_hip_host_malloc(void** host_ptr, size_t bytes)
	{
		if (host_ptr == nullptr)
			return NNF_HIP_EINVAL;
		return hip_status(hipHostMalloc(host_ptr, bytes == 0 ? 16 : bytes, hipHostMallocDefault));
	}

	int nnf_hip_host_free(void* host_ptr)
	{
		return hip_status(hipHostFree(host_ptr));
	}

	int nnf_hip_stream_create(void** stream)
	{
		if (stream == nullptr)
			return NNF_HIP_EINVAL;
		hipStream_t s = nullptr;
		const hipError_t e = hipStreamCreateWithFlags(&s, hipStreamNonBlocking); // default priority
		*stream = s;
		return hip_status(e);
	}

	int nnf_hip_stream_destroy(void* stream)
	{
		return hip_status(hipStreamDestroy(static_cast<hipStream_t>(stream)));
	}

	int nnf_hip_stream_synchronize(void* stream)
	{
		return hip_status(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
	}

	int nnf_hip_device_synchronize(void)
	{
		return hip_status(hipDeviceSynchronize());
	}

	int nnf_hip_event_create(void** event)
	{
		if (event == nullptr)
			return NNF_HIP_EINVAL;
		hipEvent_t ev = nullptr;
		const hipError_t e = hipEventCreate(&ev);
		*event = ev;
		return hip_status(e);
	}

	int nnf_hip_event_destroy(void* event)
	{
		return hip_status(hipEventDestroy(static_cast<hipEvent_t>(event)));
	}

	int nnf_hip_event_record(void* event, void* stream)
	{
		return hip_status(hipEventRecord(static_cast<hipEvent_t>(event), static_cast<hipStream_t>(stream)));
	}

	int nnf_hip_event_synchronize(void* event)
	{
		return hip_status(hipEventSynchronize(static_cast<hipEvent_t>(event)));
	}

	int nnf_hip_event_elapsed_ms(float* milliseconds, void* start_event, void* stop_event)
	{
		if (milliseconds == nullptr)
			return NNF_HIP_EINVAL;
		return hip_status(hipEventElapsedTime(milliseconds, static_cast<hipEvent_t>(start_event), static_cast<hipEvent_t>(stop_event)));
	}

	int nnf_hip_stream_wait_event(void* stream, void* event)
	{
		return hip_status(hipStreamWaitEvent(static_cast<hipStream_t>(stream), static_cast<hipEvent_t>(event), 0));
	}

	int nnf_hip_stream_begin_capture(void* stream)
	{
		return hip_status(hipStreamBeginCapture(static_cast<hipStream_t>(stream), hipStreamCaptureModeThreadLocal));
	}

	int nnf_hip_stream_end_capture(void* stream, void** graph_exec)
	{
		if (graph_exec == nullptr)
			return NNF_HIP_EINVAL;
		*graph_exec = nullptr;
		hipGraph_t graph = nullptr;
		hipError_t e = hipStreamEndCapture(static_cast<hipStream_t>(stream), &graph);
		if (e != hipSuccess)
			return hip_status(e);
		hipGraphExec_t exec = nullptr;
		e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
		(void)hipGraphDestroy(graph);
		if (e != hipSuccess)
			return hip_status(e);
		*graph_exec = exec;
		return NNF_HIP_OK;
	}

	int nnf_hip_graph_launch(void* graph_exec, void* stream)
	{
		if (graph_exec == nullptr)
			return NNF_HIP_EINVAL;
		return hip_status(hipGraphLaunch(static_cast<hipGraphExec_t>(graph_exec), static_cast<hipStream_t>(stream)));
	}

	int nnf_hip_graph_destroy(void* graph_exec)
	{
		if (graph_exec == nullptr)
			return NNF_HIP_OK;
		return hip_status(hipGraphExecDestroy(static_cast<hipGraphExec_t>(graph_exec)));
	}

	const char* nnf_hip_error_string(int code)
	{
		switch (code)
		{
		case NNF_HIP_OK: return "success";
		case NNF_HIP_EINVAL: return "nnforge_hip: invalid argument (null pointer, zero-sized dimension or malformed descriptor)";
		case NNF_HIP_EUNSUPPORTED: return "nnforge_hip: shape or option not supported by the kernels";
		case NNF_HIP_EALIGN: return "nnforge_hip: tensor base pointer is not 16-byte aligned";
		case NNF_HIP_EOVERLAP: return "nnforge_hip: output overlaps an input (only output == inputs[0] is allowed)";
		case NNF_HIP_ETOOBIG: return "nnforge_hip: element count exceeds the 32-bit index range of the kernels";
		case NNF_HIP_ESCRATCH: return "nnforge_hip: shape needs more partial states than the library's static scratch array holds (NNF_HIP_STAT_STATIC_SCRATCH_BYTES); use the entry point that takes a workspace";
		default:
			if (code > 0)
				return hipGetErrorString(static_cast<hipError_t>(code));
			return "nnforge_hip: unknown error code";
		}
	}

	int nnf_hip_launch_count(uint64_t* count)
	{
		if (count == nullptr)
			return NNF_HIP_EINVAL;
		*count = launches_of_this_thread();
		return NNF_HIP_OK;
	}

	const char* nnf_hip_version(void)
	{
		return "nnforge_hip 0.2 (gfx950)";
	}
}
