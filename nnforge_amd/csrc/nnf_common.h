// Shared declarations of the gfx950 kernel translation units.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "../../include/nnforge_hip.h"
#include "nnf_math.h"

namespace nnf
{
	typedef float floatx4 __attribute__((ext_vector_type(4)));

	constexpr int wave_size = 64;

	// 2^(i/32) table of nnf_expf followed by the two constants of exp_context, in device memory
	// (one copy per translation unit); kernels copy all of it to LDS before use.
	constexpr int exp_lds_entries = exp2_table_size + 2;
	static __device__ const uint64_t exp2_table_device[exp_lds_entries] = { NNF_EXP2_TABLE_VALUES, NNF_EXP_SHIFT_BITS, NNF_EXP_C1_BITS };

	__device__ __forceinline__ void stage_exp2_table(uint64_t* lds_table)
	{
		if (threadIdx.x < exp_lds_entries)
			lds_table[threadIdx.x] = exp2_table_device[threadIdx.x];
	}

	// after the barrier that follows stage_exp2_table; the constants come from LDS so that they
	// live in registers
	__device__ __forceinline__ exp_context exp_context_from_lds(const uint64_t* lds_table)
	{
		exp_context ctx;
		ctx.table = lds_table;
		ctx.shift = bits_to_double(lds_table[exp2_table_size]);
		ctx.c1 = bits_to_double(lds_table[exp2_table_size + 1]);
		return ctx;
	}

	// Consecutive workgroups are handed to consecutive XCDs (eight dies, an L2 each). Work items that touch common memory -
	// the bands of a plane: the input rows two of them stage, the output cache line two of them write - are `together`
	// consecutive work items; of every 8 * together workgroups the ones with the same index modulo 8 take them, so that
	// they meet in one die's L2 (what is left over at the end of the grid keeps its order). Measured on the tiling
	// kernel, 64 x 64 planes of 112 x 112 in five bands each: 72.7 -> 67.7 us. The pooling kernels, whose bands share
	// an input row but no output cache line, gain nothing from it (3 x 3 every 2 on the same planes, two bands each:
	// 40.9 -> 40.7 us, with BatchNorm and ReLU folded in 44.1 -> 45.3 us) and keep the plain order. The softmax kernel
	// that shares columns out over lanes takes neighbouring blocks of positions through it.
	__device__ __forceinline__ uint32_t xcd_grouped(uint32_t block, uint32_t together, uint32_t blocks)
	{
		const uint32_t chunk = 8 * together;
		const uint32_t in_chunk = block % chunk;
		if ((together < 2) || (block - in_chunk + chunk > blocks))
			return block;
		return block - in_chunk + (in_chunk % 8) * together + in_chunk / 8;
	}

	// Wavefront-private variant in two steps: every wavefront of the workgroup copies the table into
	// its own exp_lds_entries slots of lds_tables and reads only those, so no workgroup barrier is
	// needed (the LDS operations of one wavefront execute in program order). The global load of the
	// lane's table entry is issued first, unconditionally, so that a kernel can put its tensor and
	// weight loads behind it and wait for all of them once; the LDS copy follows those loads.
	__device__ __forceinline__ uint64_t load_exp2_table_entry()
	{
		const uint32_t lane = threadIdx.x % wave_size;
		return exp2_table_device[lane < exp_lds_entries ? lane : exp_lds_entries - 1];
	}

	__device__ __forceinline__ exp_context stage_exp2_table_per_wavefront(uint64_t* lds_tables, uint64_t entry)
	{
		const uint32_t lane = threadIdx.x % wave_size;
		uint64_t* own = lds_tables + (threadIdx.x / wave_size) * exp_lds_entries;
		if (lane < exp_lds_entries)
			own[lane] = entry;
		__builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
		__builtin_amdgcn_wave_barrier();
		__builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
		return exp_context_from_lds(own);
	}

	// Streaming accesses: each byte of an activation tensor is touched once per launch, so loads
	// and stores carry the non-temporal hint and do not displace what the caches hold. Measured with ordinary
	// stores instead: BatchNorm -> ReLU on 25.7 MB 9.2 -> 10.7 us, the ResNet-50 stack of 64 entries 1022 -> 1077 us
	// (of 8 entries, where a block's result could stay in the last-level cache for the next block: 160 -> 159 us);
	// with ordinary loads instead: 9.2 -> 9.7 us, 1022 -> 1083 us, BatchNorm -> Add -> PReLU on 411 MB tensors 192 -> 207 us.
	__device__ __forceinline__ floatx4 load_stream(const floatx4* p)
	{
		return __builtin_nontemporal_load(p);
	}

	__device__ __forceinline__ void store_stream(floatx4* p, floatx4 v)
	{
		__builtin_nontemporal_store(v, p);
	}

	inline bool is_aligned16(const void* p)
	{
		return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
	}

	inline int hip_status(hipError_t e)
	{
		return static_cast<int>(e);
	}

	// compute units of the current device (asked once per device)
	inline uint32_t compute_unit_count()
	{
		constexpr int max_devices = 64;
		static std::atomic<uint32_t> known[max_devices];
		int device = 0;
		if ((hipGetDevice(&device) != hipSuccess) || (device < 0) || (device >= max_devices))
			return 256;
		uint32_t count = known[device].load(std::memory_order_relaxed);
		if (count == 0)
		{
			int value = 0;
			if ((hipDeviceGetAttribute(&value, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess) || (value <= 0))
				value = 256;
			count = static_cast<uint32_t>(value);
			known[device].store(count, std::memory_order_relaxed);
		}
		return count;
	}

	// One round of resident workgroups whose loads are all requested in the launch's first half microsecond: memory serves
	// a stream of reads followed by a stream of writes faster than the two mixed (a kernel that only reads gets 7.0 TB/s, one
	// that only writes 6.8, a copy 6.1 to 6.3), so a kernel whose values are ready early keeps them in registers until the
	// launch's reads have had their time and stores then. (Kernels that need per-feature-map weights have that wait
	// by themselves: the weights come back behind the tensor. Measured on 25.7 MB in, 25.7 MB out: a copy of four inputs
	// 10.0 -> 9.5 us (12.8 MB: 7.2 -> 6.7 us, 19.3 MB: 8.3 -> 7.6 us); a bare BatchNorm -> ReLU 10.5 -> 8.9 us; held 20 % longer
	// than needed: + 2.5 %. The fused-group kernel does not use it: the few instructions it takes there cost the groups that
	// do not need it 4 to 13 %.)
	// -> 10 ns ticks from a workgroup's start to its first store, 0 when the launch is not of that kind.
	inline uint32_t read_phase_ticks(uint64_t workgroups, uint32_t workgroups_per_compute_unit, uint64_t bytes_read)
	{
		constexpr uint64_t least_bytes = 12u << 20;       // below this a launch is over before a wait could pay (9.6 MB: a loss)
		constexpr uint64_t bytes_per_tick = 68000;        // 6.8 TB/s
		constexpr uint32_t start_ticks = 30;              // the workgroups of a launch start within 0.3 to 0.5 us
		if ((workgroups > static_cast<uint64_t>(workgroups_per_compute_unit) * compute_unit_count()) || (bytes_read < least_bytes))
			return 0;
		return start_ticks + static_cast<uint32_t>(bytes_read / bytes_per_tick);
	}

#ifdef __HIPCC__
	// started: wall_clock64() at the workgroup's start (100 MHz). The wait ends by the clock alone.
	__device__ __forceinline__ void hold_until(uint64_t started, uint32_t ticks)
	{
		while (wall_clock64() - started < ticks)
			__builtin_amdgcn_s_sleep(8);
	}
#endif

	// Kernels the library has launched from the calling thread (nnf_hip_launch_count): every launch goes through NNF_LAUNCH.
	inline uint64_t& launches_of_this_thread()
	{
		static thread_local uint64_t count = 0;
		return count;
	}

#define NNF_LAUNCH(...) do { ++::nnf::launches_of_this_thread(); hipLaunchKernelGGL(__VA_ARGS__); } while (0)

	// Launch errors are reported by hipGetLastError right after the launch; asynchronous faults
	// surface at the caller's next synchronising call, as with any HIP work.
	inline int launch_status()
	{
		return hip_status(hipGetLastError());
	}

	// entry points implemented in the individual translation units
	int chain_forward(hipStream_t stream, const nnf_hip_chain_desc* desc, float* output,
		const float* const* inputs, const float* const* chunk_ptrs);
	int chain_forward_strided_status(const nnf_hip_chain_desc* desc, uint32_t output_entry_stride);
	int chain_forward_strided_batch(hipStream_t stream, uint32_t group_count, const nnf_hip_chain_desc* descs, float* const* outputs,
		const uint32_t* output_entry_strides, const float* const* const* inputs, const float* const* const* chunk_ptrs);
	int chain_forward_strided(hipStream_t stream, const nnf_hip_chain_desc* desc, float* output, uint32_t output_entry_stride,
		const float* const* inputs, const float* const* chunk_ptrs);
	int chain_forward_batch(hipStream_t stream, uint32_t group_count, const nnf_hip_chain_desc* descs, float* const* outputs,
		const float* const* const* inputs, const float* const* const* chunk_ptrs);
	int softmax_forward(hipStream_t stream, float* output, const float* input,
		uint32_t entry_count, uint32_t feature_map_count, uint32_t neuron_count_per_feature_map);
	int average_subsampling_forward(hipStream_t stream, float* output, const float* input,
		uint32_t entry_count, uint32_t feature_map_count, uint32_t input_width, uint32_t input_height,
		uint32_t window_width, uint32_t window_height, float mult);
	int concat_forward(hipStream_t stream, float* output, const float* const* inputs, const uint32_t* input_neuron_counts,
		const uint8_t* inputs_in_place, uint32_t input_count, uint32_t entry_count);
	int maxout_forward(hipStream_t stream, float* output, const float* input,
		uint32_t entry_count, uint32_t output_feature_map_count, uint32_t neuron_count_per_feature_map,
		uint32_t feature_map_subsampling_size);
	int max_subsampling_forward(hipStream_t stream, float* output, const float* input,
		uint32_t output_entry_count, uint32_t input_feature_map_count, uint32_t dimension_count,
		const uint32_t* input_sizes, const uint32_t* subsampling_sizes, const uint32_t* strides, const uint32_t* round_ups,
		uint32_t feature_map_subsampling_size, uint32_t entry_subsampling_size, int32_t is_min);
	int prologue_status(const nnf_hip_chain_desc& desc, const float* const* chunk_ptrs, bool allow_join = false);
	bool window2d_launch_with_prologue(hipStream_t stream, int op, float mult, float* output, const float* input, uint32_t input_total, uint32_t plane_count,
		uint32_t in_w, uint32_t in_h, uint32_t out_w, uint32_t out_h, uint32_t win_w, uint32_t win_h, uint32_t stride_x, uint32_t stride_y,
		const nnf_hip_chain_desc* prologue, const float* const* chunk_ptrs, uint32_t feature_map_count, bool plan_only);
	int max_subsampling_forward_with_prologue(hipStream_t stream, float* output, const float* input,
		uint32_t output_entry_count, uint32_t input_feature_map_count, uint32_t dimension_count,
		const uint32_t* input_sizes, const uint32_t* subsampling_sizes, const uint32_t* strides, const uint32_t* round_ups,
		uint32_t feature_map_subsampling_size, uint32_t entry_subsampling_size, int32_t is_min,
		const nnf_hip_chain_desc* prologue, const float* const* chunk_ptrs, bool plan_only);
	int max_subsampling_tiling_forward(hipStream_t stream, float* output, const float* input,
		uint32_t input_entry_count, uint32_t feature_map_count, uint32_t dimension_count,
		const uint32_t* input_sizes, const uint32_t* subsampling_sizes, int32_t is_min);
	int average_subsampling_nd_forward(hipStream_t stream, float* output, const float* input,
		uint32_t output_entry_count, uint32_t input_feature_map_count, uint32_t dimension_count,
		const uint32_t* input_sizes, const uint32_t* subsampling_sizes,
		uint32_t feature_map_subsampling_size, uint32_t entry_subsampling_size, float mult);
	int average_subsampling_forward_with_prologue(hipStream_t stream, float* output, const float* input, const float* input2,
		uint32_t entry_count, uint32_t feature_map_count, uint32_t input_width, uint32_t input_height,
		uint32_t window_width, uint32_t window_height, float mult,
		const nnf_hip_chain_desc* prologue, const float* const* chunk_ptrs, bool plan_only);
	bool window2d_launch(hipStream_t stream, int op, float mult, float* output, const float* input, uint32_t input_total, uint32_t plane_count,
		uint32_t in_w, uint32_t in_h, uint32_t out_w, uint32_t out_h, uint32_t win_w, uint32_t win_h, uint32_t stride_x, uint32_t stride_y);
	int feature_map_stat_init(hipStream_t stream, nnf_hip_running_stat* device_stats, uint32_t feature_map_count);
	int feature_map_stat_workspace_bytes(uint32_t entry_count, uint32_t feature_map_count, uint32_t neuron_count_per_feature_map, size_t* bytes);
	int feature_map_stat_partial_count(uint32_t entry_count, uint32_t feature_map_count, uint32_t neuron_count_per_feature_map,
		size_t workspace_bytes, uint32_t* partial_states);
	int feature_map_stat_accumulate(hipStream_t stream, nnf_hip_running_stat* device_stats, void* workspace, size_t workspace_bytes,
		const float* input, uint32_t entry_count, uint32_t feature_map_count, uint32_t neuron_count_per_feature_map);
	int feature_map_stat_accumulate_static(hipStream_t stream, nnf_hip_running_stat* device_stats,
		const float* input, uint32_t entry_count, uint32_t feature_map_count, uint32_t neuron_count_per_feature_map);
	int copy_kernel(hipStream_t stream, void* dst, const void* src, size_t bytes);
}
