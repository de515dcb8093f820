// Concatenation along feature maps (nnforge/plain/concat_layer_tester_plain.cpp:45-58): per entry
// the neurons of input 0, then of input 1, ... A pure copy, so the only concern is moving every
// byte once with wide, coalesced accesses.
#include "nnf_common.h"

#include <algorithm>

namespace nnf
{
	namespace
	{
		constexpr int concat_block_size = 256;
		constexpr int concat_unroll = 4;            // accesses per lane
		constexpr uint32_t concat_max_inputs = 8;   // per launch

		struct concat_args
		{
			float* out;
			const float* in[concat_max_inputs];
			uint32_t length[concat_max_inputs];      // neurons per entry of each input
			uint32_t offset[concat_max_inputs];      // where the input starts inside an output entry
			uint32_t first_block[concat_max_inputs + 1]; // blockIdx.x range of each input
			uint32_t input_count;
			uint32_t output_length;                  // neurons per output entry
			uint32_t entry_count;
			uint32_t hold_ticks;                     // stores wait until this many 10 ns ticks after the workgroup's start (0: no wait)
		};

		// VEC: floats per access; 4 when every length is a multiple of 4 (then every offset is as well)
		template<int VEC>
		__global__ void __launch_bounds__(concat_block_size) concat_kernel(const concat_args a)
		{
			typedef float vec_t __attribute__((ext_vector_type(VEC)));
			uint32_t i = 0;
			while ((i + 1 < a.input_count) && (blockIdx.x >= a.first_block[i + 1]))
				++i;
			const uint32_t tile = (blockIdx.x - a.first_block[i]) * (concat_block_size * concat_unroll * VEC);
			const uint32_t length = a.length[i];
			const uint64_t started = (a.hold_ticks != 0) ? wall_clock64() : 0;
			for(uint32_t entry = blockIdx.y; entry < a.entry_count; entry += gridDim.y)
			{
				const float* src = a.in[i] + static_cast<size_t>(entry) * length;
				float* dst = a.out + static_cast<size_t>(entry) * a.output_length + a.offset[i];
				// (Loads without the branch around them - lanes past the end loading the last vector once more - are
				// issued back to back instead of one after the other's arrival, and measured slower here: 32 entries of
				// 64 + 128 + 32 + 32 maps of 28 x 28, 10.0 -> 11.4 us.)
				vec_t v[concat_unroll];
				#pragma unroll
				for(int k = 0; k < concat_unroll; ++k)
				{
					const uint32_t r = tile + (k * concat_block_size + threadIdx.x) * VEC;
					if (r < length)
						v[k] = __builtin_nontemporal_load(reinterpret_cast<const vec_t*>(src + r));
				}
				if (a.hold_ticks != 0)
				{
					// the values wait in their registers until the launch's reads have had their time (read_phase_ticks)
					#pragma unroll
					for(int k = 0; k < concat_unroll; ++k)
						asm volatile("" : "+v"(v[k]));
					hold_until(started, a.hold_ticks);
				}
				#pragma unroll
				for(int k = 0; k < concat_unroll; ++k)
				{
					const uint32_t r = tile + (k * concat_block_size + threadIdx.x) * VEC;
					if (r < length)
						__builtin_nontemporal_store(v[k], reinterpret_cast<vec_t*>(dst + r));
				}
			}
		}

		template<>
		__global__ void __launch_bounds__(concat_block_size) concat_kernel<1>(const concat_args a)
		{
			uint32_t i = 0;
			while ((i + 1 < a.input_count) && (blockIdx.x >= a.first_block[i + 1]))
				++i;
			const uint32_t tile = (blockIdx.x - a.first_block[i]) * (concat_block_size * concat_unroll);
			const uint32_t length = a.length[i];
			for(uint32_t entry = blockIdx.y; entry < a.entry_count; entry += gridDim.y)
			{
				const float* src = a.in[i] + static_cast<size_t>(entry) * length;
				float* dst = a.out + static_cast<size_t>(entry) * a.output_length + a.offset[i];
				#pragma unroll
				for(int k = 0; k < concat_unroll; ++k)
				{
					const uint32_t r = tile + k * concat_block_size + threadIdx.x;
					if (r < length)
						dst[r] = src[r];
				}
			}
		}
	}

	// inputs_in_place (may be null): inputs that lie in their part of the output already; they take their room and no copy
	int concat_forward(hipStream_t stream, float* output, const float* const* inputs, const uint32_t* input_neuron_counts,
		const uint8_t* inputs_in_place, uint32_t input_count, uint32_t entry_count)
	{
		const auto in_place = [inputs_in_place] (uint32_t i) { return (inputs_in_place != nullptr) && (inputs_in_place[i] != 0); };
		if ((output == nullptr) || (inputs == nullptr) || (input_neuron_counts == nullptr) || (input_count == 0))
			return NNF_HIP_EINVAL;
		if (!is_aligned16(output))
			return NNF_HIP_EALIGN;
		uint64_t output_length = 0;
		bool vector = true;
		for(uint32_t i = 0; i < input_count; ++i)
		{
			if ((input_neuron_counts[i] != 0) && !in_place(i)) // an input without neurons is never read
			{
				if (inputs[i] == nullptr)
					return NNF_HIP_EINVAL;
				if (!is_aligned16(inputs[i]))
					return NNF_HIP_EALIGN;
			}
			output_length += input_neuron_counts[i];
			vector = vector && ((input_neuron_counts[i] % 4) == 0);
		}
		const uint64_t output_total = output_length * entry_count;
		if (output_total == 0)
			return NNF_HIP_OK;
		if (output_total > NNF_HIP_MAX_ELEMENT_COUNT)
			return NNF_HIP_ETOOBIG;
		for(uint32_t i = 0; i < input_count; ++i)
		{
			const uintptr_t a = reinterpret_cast<uintptr_t>(output), b = reinterpret_cast<uintptr_t>(inputs[i]);
			const uint64_t b_bytes = in_place(i) ? 0 : static_cast<uint64_t>(input_neuron_counts[i]) * entry_count * sizeof(float);
			if ((b_bytes != 0) && (a < b + b_bytes) && (b < a + output_total * sizeof(float)))
				return NNF_HIP_EOVERLAP;
		}

		const uint32_t per_block = concat_block_size * concat_unroll * (vector ? 4 : 1);
		uint32_t offset = 0;
		for(uint32_t first = 0; first < input_count; first += concat_max_inputs)
		{
			concat_args a = {};
			a.out = output;
			a.input_count = std::min(concat_max_inputs, input_count - first);
			a.output_length = static_cast<uint32_t>(output_length);
			a.entry_count = entry_count;
			uint32_t blocks = 0;
			for(uint32_t i = 0; i < a.input_count; ++i)
			{
				a.in[i] = in_place(first + i) ? nullptr : inputs[first + i];
				a.length[i] = input_neuron_counts[first + i];
				a.offset[i] = offset;
				a.first_block[i] = blocks;
				offset += a.length[i];
				blocks += in_place(first + i) ? 0 : (a.length[i] + per_block - 1) / per_block;
			}
			a.first_block[a.input_count] = blocks;
			if (blocks == 0)
				continue;
			const dim3 grid(blocks, std::min(entry_count, 65535u));
			// one round of resident workgroups: the stores wait for the launch's reads (read_phase_ticks)
			uint64_t copied = 0;
			for(uint32_t i = 0; i < a.input_count; ++i)
				copied += (a.in[i] != nullptr) ? static_cast<uint64_t>(a.length[i]) * entry_count * sizeof(float) : 0;
			a.hold_ticks = vector ? read_phase_ticks(static_cast<uint64_t>(grid.x) * grid.y, 8, copied) : 0;
			if (vector)
				NNF_LAUNCH(concat_kernel<4>, grid, dim3(concat_block_size), 0, stream, a);
			else
				NNF_LAUNCH(concat_kernel<1>, grid, dim3(concat_block_size), 0, stream, a);
			const int status = launch_status();
			if (status != NNF_HIP_OK)
				return status;
		}
		return NNF_HIP_OK;
	}
}
