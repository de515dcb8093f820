// Per-feature-map statistics of a tensor on the device: count, mean, sum of squared deviations
// (double precision), minimum and maximum - the running state of nnForge's stat_data_bunch_writer
// (nnforge/stat_data_bunch_writer.cpp:45-79), which the reference fills on the host, one value at
// a time, from outputs copied back entry by entry.
//
// The reference's update is sequential (Welford). Here every workgroup reduces a run of entries of
// one feature map to (n, mean, m2) and the runs are merged in a fixed order with the pairwise
// update of Chan et al., also in double precision; the result does not depend on scheduling.
// Inside a workgroup the sums are taken of (x - pivot), the pivot being the run's first value, so
// that a mean far from zero does not cancel the deviation. mean and m2 agree with the sequential
// update to a few units of double rounding; after the reference's conversion to fp32 that is
// at most one unit in the last place. Minimum and maximum use the reference's comparisons
// (NaN never enters); which of +0.0 / -0.0 is reported when both occur is not defined here.
#include "nnf_common.h"

#include <algorithm>
#include <cstdlib>
#include <mutex>

namespace nnf
{
	namespace
	{
		constexpr int stat_block_size = 256;
		constexpr int stat_unroll = 4;                    // loads a lane has in flight
		// Workgroups of this kernel an MI355X holds at once: 256 compute units x 8 workgroups of 256
		// lanes (the kernel needs 32 vector registers: 8 wavefronts per SIMD).
		// The grid is cut so that it fills whole rounds of that many.
		constexpr uint32_t stat_resident_blocks = 2048;
		// what starting and finishing a workgroup costs, in floats of streaming (wavefront and LDS
		// reductions, the partial state)
		constexpr uint64_t stat_block_overhead_floats = 8192;

		// Partial states of nnf_hip_feature_map_stat_accumulate_static: a fixed array in the library's device
		// image instead of a caller's workspace. Every device the library runs on holds its own copy at its own
		// address for the life of the process. In host code the name `scratch` is only a handle for
		// hipGetSymbolAddress, never an address a kernel may be given.
		constexpr size_t stat_static_states = NNF_HIP_STAT_STATIC_SCRATCH_BYTES / sizeof(nnf_hip_running_stat);
		static __device__ __align__(256) unsigned char scratch[NNF_HIP_STAT_STATIC_SCRATCH_BYTES];

		constexpr int stat_max_devices = 64;
		std::mutex scratch_mutex;
		void* scratch_address[stat_max_devices] = {}; // per device, looked up once with that device current

		// address of the current device's copy of `scratch`
		int static_scratch_of_current_device(void** address)
		{
			int device = -1;
			hipError_t e = hipGetDevice(&device);
			if (e != hipSuccess)
				return hip_status(e);
			if ((device < 0) || (device >= stat_max_devices))
				return NNF_HIP_EUNSUPPORTED;
			std::lock_guard<std::mutex> lock(scratch_mutex);
			if (scratch_address[device] == nullptr)
			{
				void* found = nullptr;
				e = hipGetSymbolAddress(&found, HIP_SYMBOL(scratch));
				if (e != hipSuccess)
					return hip_status(e);
				if (found == nullptr)
					return NNF_HIP_EINVAL;
				scratch_address[device] = found;
			}
			*address = scratch_address[device];
			return NNF_HIP_OK;
		}

		struct stat_plan
		{
			uint32_t entries_per_run;
			uint32_t runs;
			uint32_t segments;          // pieces a plane is cut into (> 1 only with one entry per run)
			uint32_t units_per_segment; // in loads (float4s when the plane is a multiple of 4, else floats)
		};

		// The grid is (runs of entries) x (feature maps), every workgroup streaming entries_per_run
		// planes. All workgroups take equally long, so the launch lasts
		// ceil(workgroups / resident) rounds of one workgroup's time: the run length that minimises
		// rounds x (run length + overhead) is chosen. Measured on 128 entries of 256 feature maps of
		// 56x56: 6 runs of 22 entries (1536 workgroups, one round) 67.5 us, 13 runs of 10 (3328, two
		// nearly full rounds) 69-71 us, 8 runs of 16 (2048, one round and a seventh of another) 83 us.
		//
		// capacity: partial states the workspace holds; plans that need more are passed over. The longest
		// run the index arithmetic allows gives the fewest partial states, and that number never grows when
		// entries are taken away, so a workspace sized for some entry count holds a plan for every smaller
		// count as well (not necessarily with the same number of runs: 16 entries may be cut into 16 runs
		// where 29 entries were cut into 15). runs == 0 in the result: no plan fits the capacity.
		stat_plan plan_runs(uint32_t entry_count, uint32_t feature_map_count, uint32_t plane, uint64_t capacity)
		{
			// the kernel divides flat indices by the plane size with a multiplication, exact while
			// index * divisor < 2^32; a run of one entry needs no division
			const uint64_t units = ((plane % 4) == 0) ? plane / 4 : plane;
			stat_plan best = { 1, 0, 1, static_cast<uint32_t>(units) };
			uint64_t best_cost = ~0ull;
			for(uint32_t entries_per_run = 1; entries_per_run <= entry_count; ++entries_per_run)
			{
				if ((entries_per_run > 1) && (static_cast<uint64_t>(entries_per_run) * units * units >= (1ull << 32)))
					break;
				const uint32_t runs = (entry_count + entries_per_run - 1) / entries_per_run;
				const uint64_t blocks = static_cast<uint64_t>(runs) * feature_map_count;
				if (blocks > capacity)
					continue;
				const uint64_t rounds = (blocks + stat_resident_blocks - 1) / stat_resident_blocks;
				const uint64_t cost = rounds * (static_cast<uint64_t>(entries_per_run) * plane + stat_block_overhead_floats);
				if (cost < best_cost)
				{
					best_cost = cost;
					best.entries_per_run = entries_per_run;
					best.runs = runs;
				}
			}
			// Few planes, each long (statistics of input images, say): a plane is cut into segments so that
			// the grid still covers the machine; a segment keeps at least two rounds of loads per lane.
			if (best.runs == 0)
				return best;
			const uint64_t blocks = static_cast<uint64_t>(best.runs) * feature_map_count;
			const uint64_t min_segment_units = static_cast<uint64_t>(stat_block_size) * stat_unroll * 2;
			if ((best.entries_per_run == 1) && (blocks * 2 <= stat_resident_blocks) && (units >= 2 * min_segment_units))
			{
				const uint64_t wanted = std::min<uint64_t>(std::min<uint64_t>(stat_resident_blocks, capacity) / blocks, units / min_segment_units);
				best.units_per_segment = static_cast<uint32_t>((units + wanted - 1) / wanted);
				best.segments = static_cast<uint32_t>((units + best.units_per_segment - 1) / best.units_per_segment);
			}
			return best;
		}

		__device__ __forceinline__ void accumulate(float v, double pivot, double& s1, double& s2, float& mn, float& mx)
		{
			const double d = static_cast<double>(v) - pivot;
			s1 += d;
			s2 = fma(d, d, s2);
			// std::min(current, val) / std::max(current, val) never take a NaN val, and current is never NaN:
			// that is fminf / fmaxf (one instruction each)
			mn = __builtin_fminf(mn, v);
			mx = __builtin_fmaxf(mx, v);
		}

		// grid: (runs x segments, feature maps). VEC: floats per load (4 when plane is a multiple of 4).
		template<int VEC>
		__global__ void __launch_bounds__(stat_block_size) stat_runs_kernel(
			nnf_hip_running_stat* partial, const float* in, uint32_t entry_count, uint32_t feature_map_count, uint32_t plane,
			uint32_t entries_per_run, uint32_t unit_magic, uint32_t segments, uint32_t units_per_segment)
		{
			typedef float vec_t __attribute__((ext_vector_type(VEC)));
			__shared__ double lds_s1[stat_block_size / wave_size], lds_s2[stat_block_size / wave_size];
			__shared__ float lds_mn[stat_block_size / wave_size], lds_mx[stat_block_size / wave_size];

			const uint32_t run = blockIdx.x / segments, segment = blockIdx.x - run * segments, fm = blockIdx.y;
			const uint32_t e0 = run * entries_per_run;
			const uint32_t entries_here = min(entries_per_run, entry_count - e0);
			const uint32_t units_per_plane = plane / VEC;
			// segments > 1: one entry per run, this workgroup takes a piece of its plane
			const uint32_t unit_begin = segment * units_per_segment;
			const uint32_t units = (segments > 1) ? min(units_per_segment, units_per_plane - unit_begin) : entries_here * units_per_plane;
			const uint32_t entry_gap = (feature_map_count - 1) * plane;
			const float* base = in + (static_cast<size_t>(e0) * feature_map_count + fm) * plane + static_cast<size_t>(unit_begin) * VEC;
			const double pivot = static_cast<double>(base[0]);

			double s1 = 0.0, s2 = 0.0;
			float mn = 3.402823466e+38f, mx = -3.402823466e+38f;
			for(uint32_t first = 0; first < units; first += stat_block_size * stat_unroll)
			{
				vec_t v[stat_unroll];
				#pragma unroll
				for(int k = 0; k < stat_unroll; ++k)
				{
					// No branch around a load (lanes past the end load the run's last unit once more and leave it out of
					// the sums): with one, every load of a round waited for the one before it.
					const uint32_t t = min(first + k * stat_block_size + threadIdx.x, units - 1);
					// element t of the run lies t * VEC floats into it plus the other feature maps of the
					// entries before it: e * (entry_stride - plane); the tensor has fewer than 2^32 floats
					const uint32_t e = (entries_here == 1) ? 0u : ((units_per_plane == 1) ? t : __umulhi(t, unit_magic));
					v[k] = __builtin_nontemporal_load(reinterpret_cast<const vec_t*>(base + (t * VEC + e * entry_gap)));
				}
				#pragma unroll
				for(int k = 0; k < stat_unroll; ++k)
				{
					const uint32_t t = first + k * stat_block_size + threadIdx.x;
					if (t < units)
					{
						#pragma unroll
						for(int c = 0; c < VEC; ++c)
							accumulate(v[k][c], pivot, s1, s2, mn, mx);
					}
				}
			}

			// wavefront, then workgroup
			#pragma unroll
			for(int offset = wave_size / 2; offset > 0; offset /= 2)
			{
				s1 += __shfl_xor(s1, offset);
				s2 += __shfl_xor(s2, offset);
				const float other_mn = __shfl_xor(mn, offset), other_mx = __shfl_xor(mx, offset);
				mn = (other_mn < mn) ? other_mn : mn;
				mx = (mx < other_mx) ? other_mx : mx;
			}
			const uint32_t wave = threadIdx.x / wave_size;
			if ((threadIdx.x % wave_size) == 0)
			{
				lds_s1[wave] = s1; lds_s2[wave] = s2; lds_mn[wave] = mn; lds_mx[wave] = mx;
			}
			__syncthreads();
			if (threadIdx.x == 0)
			{
				for(uint32_t w = 1; w < stat_block_size / wave_size; ++w)
				{
					s1 += lds_s1[w];
					s2 += lds_s2[w];
					mn = (lds_mn[w] < mn) ? lds_mn[w] : mn;
					mx = (mx < lds_mx[w]) ? lds_mx[w] : mx;
				}
				const double n = static_cast<double>(units) * static_cast<double>(VEC);
				nnf_hip_running_stat r;
				r.n = n;
				r.mean = pivot + s1 / n;
				const double m2 = s2 - s1 * s1 / n;
				r.m2 = (m2 < 0.0) ? 0.0 : m2; // rounding may leave a tiny negative value where the deviation is zero
				r.min_val = mn;
				r.max_val = mx;
				partial[static_cast<size_t>(blockIdx.x) * feature_map_count + fm] = r;
			}
		}

		// One lane per feature map folds the runs into the running state, run 0 first.
		__global__ void __launch_bounds__(stat_block_size) stat_merge_kernel(
			nnf_hip_running_stat* state, const nnf_hip_running_stat* partial, uint32_t feature_map_count, uint32_t runs)
		{
			const uint32_t fm = blockIdx.x * stat_block_size + threadIdx.x;
			if (fm >= feature_map_count)
				return;
			nnf_hip_running_stat s = state[fm];
			constexpr uint32_t batch = 8; // partial states fetched together: the merge itself is a dependent chain
			for(uint32_t first = 0; first < runs; first += batch)
			{
				nnf_hip_running_stat b[batch];
				#pragma unroll
				for(uint32_t k = 0; k < batch; ++k)
					if (first + k < runs)
						b[k] = partial[static_cast<size_t>(first + k) * feature_map_count + fm];
				#pragma unroll
				for(uint32_t k = 0; k < batch; ++k)
				{
					if (first + k >= runs)
						break;
					const double n = s.n + b[k].n;
					const double delta = b[k].mean - s.mean;
					if (s.n == 0.0)
						s.mean = b[k].mean;
					else
						s.mean = s.mean + delta * (b[k].n / n);
					s.m2 = s.m2 + b[k].m2 + delta * delta * (s.n * b[k].n / n);
					s.n = n;
					s.min_val = (b[k].min_val < s.min_val) ? b[k].min_val : s.min_val;
					s.max_val = (s.max_val < b[k].max_val) ? b[k].max_val : s.max_val;
				}
			}
			state[fm] = s;
		}

		__global__ void __launch_bounds__(stat_block_size) stat_init_kernel(nnf_hip_running_stat* state, uint32_t feature_map_count)
		{
			const uint32_t fm = blockIdx.x * stat_block_size + threadIdx.x;
			if (fm >= feature_map_count)
				return;
			// nnforge/stat_data_bunch_writer.h:48-55
			nnf_hip_running_stat s;
			s.n = 0.0;
			s.mean = 0.0;
			s.m2 = 0.0;
			s.min_val = 3.402823466e+38f;
			s.max_val = -3.402823466e+38f;
			state[fm] = s;
		}
	}

	int feature_map_stat_init(hipStream_t stream, nnf_hip_running_stat* device_stats, uint32_t feature_map_count)
	{
		if ((device_stats == nullptr) || (feature_map_count == 0))
			return NNF_HIP_EINVAL;
		if (!is_aligned16(device_stats))
			return NNF_HIP_EALIGN;
		NNF_LAUNCH(stat_init_kernel, dim3((feature_map_count + stat_block_size - 1) / stat_block_size), dim3(stat_block_size), 0, stream,
			device_stats, feature_map_count);
		const int status = launch_status();
		// Set-up of the statistics path on this device: the address of its static scratch array is looked up here,
		// so that nnf_hip_feature_map_stat_accumulate_static finds it ready (a failure is reported there).
		void* unused = nullptr;
		static_scratch_of_current_device(&unused);
		return status;
	}

	int feature_map_stat_workspace_bytes(uint32_t entry_count, uint32_t feature_map_count, uint32_t neuron_count_per_feature_map, size_t* bytes)
	{
		if ((bytes == nullptr) || (feature_map_count == 0) || (neuron_count_per_feature_map == 0))
			return NNF_HIP_EINVAL;
		const stat_plan p = plan_runs(std::max(1u, entry_count), feature_map_count, neuron_count_per_feature_map, ~0ull);
		*bytes = static_cast<size_t>(p.runs) * p.segments * feature_map_count * sizeof(nnf_hip_running_stat);
		return NNF_HIP_OK;
	}

	int feature_map_stat_partial_count(uint32_t entry_count, uint32_t feature_map_count, uint32_t neuron_count_per_feature_map,
		size_t workspace_bytes, uint32_t* partial_states)
	{
		if ((partial_states == nullptr) || (feature_map_count == 0) || (neuron_count_per_feature_map == 0))
			return NNF_HIP_EINVAL;
		*partial_states = 0;
		if (entry_count == 0)
			return NNF_HIP_OK;
		const stat_plan p = plan_runs(entry_count, feature_map_count, neuron_count_per_feature_map, workspace_bytes / sizeof(nnf_hip_running_stat));
		if (p.runs == 0)
			return NNF_HIP_EINVAL;
		*partial_states = p.runs * p.segments * feature_map_count;
		return NNF_HIP_OK;
	}

	namespace
	{
		// argument checks shared by the two accumulate entry points; NNF_HIP_OK with *nothing_to_do set for zero entries
		int check_accumulate_arguments(const nnf_hip_running_stat* device_stats, const float* input,
			uint32_t entry_count, uint32_t feature_map_count, uint32_t neuron_count_per_feature_map, bool* nothing_to_do)
		{
			*nothing_to_do = false;
			if ((device_stats == nullptr) || (feature_map_count == 0) || (neuron_count_per_feature_map == 0))
				return NNF_HIP_EINVAL;
			if (entry_count == 0)
			{
				*nothing_to_do = true; // nothing to fold in
				return NNF_HIP_OK;
			}
			if (input == nullptr)
				return NNF_HIP_EINVAL;
			if (!is_aligned16(device_stats) || !is_aligned16(input))
				return NNF_HIP_EALIGN;
			const uint64_t total = static_cast<uint64_t>(entry_count) * feature_map_count * neuron_count_per_feature_map;
			if ((total > NNF_HIP_MAX_ELEMENT_COUNT) || (feature_map_count > 65535u))
				return NNF_HIP_ETOOBIG;
			return NNF_HIP_OK;
		}

		// the two launches: runs of entries into `partial` (every state of the plan is written, none is read
		// before), then their merge into device_stats in run order
		int launch_accumulate(hipStream_t stream, nnf_hip_running_stat* device_stats, nnf_hip_running_stat* partial, const stat_plan& p,
			const float* input, uint32_t entry_count, uint32_t feature_map_count, uint32_t neuron_count_per_feature_map)
		{
			const dim3 grid(p.runs * p.segments, feature_map_count);
			if ((neuron_count_per_feature_map % 4) == 0)
			{
				const uint32_t units = neuron_count_per_feature_map / 4;
				const uint32_t magic = (units >= 2) ? static_cast<uint32_t>(((1ull << 32) + units - 1) / units) : 0u;
				NNF_LAUNCH(stat_runs_kernel<4>, grid, dim3(stat_block_size), 0, stream, partial, input, entry_count, feature_map_count,
					neuron_count_per_feature_map, p.entries_per_run, magic, p.segments, p.units_per_segment);
			}
			else
			{
				const uint32_t units = neuron_count_per_feature_map;
				const uint32_t magic = (units >= 2) ? static_cast<uint32_t>(((1ull << 32) + units - 1) / units) : 0u;
				NNF_LAUNCH(stat_runs_kernel<1>, grid, dim3(stat_block_size), 0, stream, partial, input, entry_count, feature_map_count,
					neuron_count_per_feature_map, p.entries_per_run, magic, p.segments, p.units_per_segment);
			}
			int status = launch_status();
			if (status != NNF_HIP_OK)
				return status;
			NNF_LAUNCH(stat_merge_kernel, dim3((feature_map_count + stat_block_size - 1) / stat_block_size), dim3(stat_block_size), 0, stream,
				device_stats, partial, feature_map_count, p.runs * p.segments);
			return launch_status();
		}
	}

	int feature_map_stat_accumulate(hipStream_t stream, nnf_hip_running_stat* device_stats, void* workspace, size_t workspace_bytes,
		const float* input, uint32_t entry_count, uint32_t feature_map_count, uint32_t neuron_count_per_feature_map)
	{
		bool nothing_to_do = false;
		const int rc = check_accumulate_arguments(device_stats, input, entry_count, feature_map_count, neuron_count_per_feature_map, &nothing_to_do);
		if ((rc != NNF_HIP_OK) || nothing_to_do)
			return rc;
		if (!is_aligned16(workspace))
			return NNF_HIP_EALIGN;
		if (workspace == nullptr)
			return NNF_HIP_EINVAL;
		// the plan is made inside what the workspace holds: a workspace sized for a packet of entries also
		// serves every shorter packet
		const stat_plan p = plan_runs(entry_count, feature_map_count, neuron_count_per_feature_map, workspace_bytes / sizeof(nnf_hip_running_stat));
		if (p.runs == 0)
			return NNF_HIP_EINVAL;
		return launch_accumulate(stream, device_stats, static_cast<nnf_hip_running_stat*>(workspace), p, input, entry_count, feature_map_count,
			neuron_count_per_feature_map);
	}

	int feature_map_stat_accumulate_static(hipStream_t stream, nnf_hip_running_stat* device_stats,
		const float* input, uint32_t entry_count, uint32_t feature_map_count, uint32_t neuron_count_per_feature_map)
	{
		bool nothing_to_do = false;
		const int rc = check_accumulate_arguments(device_stats, input, entry_count, feature_map_count, neuron_count_per_feature_map, &nothing_to_do);
		if ((rc != NNF_HIP_OK) || nothing_to_do)
			return rc;
		// one partial state per feature map is the least any launch shape needs
		if (feature_map_count > stat_static_states)
			return NNF_HIP_ESCRATCH;
		const stat_plan p = plan_runs(entry_count, feature_map_count, neuron_count_per_feature_map, stat_static_states);
		if (p.runs == 0)
			return NNF_HIP_ESCRATCH; // planes so long that the entries cannot share runs, and too many of them
		void* partial = nullptr;
		const int found = static_scratch_of_current_device(&partial);
		if (found != NNF_HIP_OK)
			return found;
		// nothing in the array has to start at zero: the first launch writes every state the second one reads
		return launch_accumulate(stream, device_stats, static_cast<nnf_hip_running_stat*>(partial), p, input, entry_count, feature_map_count,
			neuron_count_per_feature_map);
	}
}
