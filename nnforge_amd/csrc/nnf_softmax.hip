// Softmax across feature maps at every (entry, spatial position), fp32
// (nnforge/plain/softmax_layer_tester_plain.cpp:61-89): max over feature maps starting from
// -1.0e37F, val = expf(x - max), sum of val, mult = 1/sum, out = val * mult.
//
// Two data shapes:
//  - neuron_count_per_feature_map == 1: the feature maps of an entry are contiguous ("rows").
//    A row lives in the registers of one wavefront, or of several when the row is long or the rows
//    are few; max and sum are 64-lane reductions (combined through LDS across wavefronts); the row is
//    read once and written once. The sum is a fixed tree, so it can differ from the reference's
//    left-to-right sum in the last bits.
//  - neuron_count_per_feature_map > 1: feature maps are strided by the plane size ("columns").
//    Lanes run along the spatial positions (coalesced), each lane walks its column in feature-map
//    order with the reference's own sequential sum.
#include "nnf_common.h"

namespace nnf
{
	namespace
	{
		constexpr float softmax_max_init = -1.0e+37F; // nnforge/plain/softmax_layer_tester_plain.cpp:71

		// std::max(a, b) as the reference evaluates it: (a < b) ? b : a, so a NaN in b is never picked
		__device__ __forceinline__ float ref_max(float a, float b)
		{
			return (a < b) ? b : a;
		}

		template<int CTRL>
		__device__ __forceinline__ float dpp_move(float v)
		{
			return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false));
		}

		__device__ __forceinline__ float read_lane(float v, int lane)
		{
			return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
		}

		// 64-lane all-reduce: four DPP steps combine each row of 16 lanes (quad swaps 0xB1 and 0x4E,
		// row_half_mirror 0x141, row_mirror 0x140), then the four row results are read as scalars.
		struct max_op { __device__ __forceinline__ float operator()(float a, float b) const { return ref_max(a, b); } };
		struct sum_op { __device__ __forceinline__ float operator()(float a, float b) const { return a + b; } };

		// GROUP 16: every row of 16 lanes keeps its own result (four rows of a tensor to a wavefront).
		template<int GROUP = 64, class OP>
		__device__ __forceinline__ float wave_all_reduce(float v, OP op)
		{
			static_assert((GROUP == 64) || (GROUP == 16), "a wavefront, or one of its rows of 16 lanes");
			v = op(v, dpp_move<0xB1>(v));
			v = op(v, dpp_move<0x4E>(v));
			v = op(v, dpp_move<0x141>(v));
			v = op(v, dpp_move<0x140>(v));
			if (GROUP == 16)
				return v;
			const float r0 = read_lane(v, 0);
			const float r1 = read_lane(v, 16);
			const float r2 = read_lane(v, 32);
			const float r3 = read_lane(v, 48);
			return op(op(r0, r1), op(r2, r3));
		}

		// Rows and register-held columns are read once and written once: non-temporal accesses from 2 M floats on (8192
		// rows of 1000 15.0 -> 12.6-13.3 us, 64 x 21 feature maps of 64 x 64 12.8 -> 9.2 us, 256 x 64 of 28 x 28 29.8 -> 25.0 us).
		// Small tensors keep ordinary accesses: a launch that only waits for its own latencies ends later when its stores
		// go all the way to memory (256 rows of 1000: 2.7 us, non-temporal 3.2 us). The kernels that share a column out over
		// lanes keep them at every size: neighbouring workgroups there complete each other's cache lines (64 x 1000 maps
		// of 7 x 7 22.0 us, non-temporal 26.9 us).
		constexpr uint64_t softmax_streaming_floats = 2u << 20;

		template<int W, bool STREAMING> struct vec_io;
		template<bool STREAMING> struct vec_io<4, STREAMING>
		{
			static __device__ __forceinline__ void load(const float* p, float (&d)[4])
			{
				const floatx4 t = STREAMING ? load_stream(reinterpret_cast<const floatx4*>(p)) : *reinterpret_cast<const floatx4*>(p);
				d[0] = t.x; d[1] = t.y; d[2] = t.z; d[3] = t.w;
			}
			static __device__ __forceinline__ void store(float* p, const float (&d)[4])
			{
				floatx4 t;
				t.x = d[0]; t.y = d[1]; t.z = d[2]; t.w = d[3];
				if (STREAMING)
					store_stream(reinterpret_cast<floatx4*>(p), t);
				else
					*reinterpret_cast<floatx4*>(p) = t;
			}
		};
		template<bool STREAMING> struct vec_io<1, STREAMING>
		{
			static __device__ __forceinline__ void load(const float* p, float (&d)[1]) { d[0] = STREAMING ? __builtin_nontemporal_load(p) : *p; }
			static __device__ __forceinline__ void store(float* p, const float (&d)[1])
			{
				if (STREAMING)
					__builtin_nontemporal_store(d[0], p);
				else
					*p = d[0];
			}
		};

		// One row per group of THREADS lanes (THREADS = 64: a wavefront; larger: a whole workgroup; 16: a quarter of a
		// wavefront, for many short rows - 65536 rows of 100 floats keep 25 of a wavefront's 64 lanes busy, of 32 lanes 25).
		// Lane t holds vectors t, t + THREADS, ... of its row: VPT vectors of W floats.
		// Rows per workgroup = blockDim.x / THREADS. Requires fm_count <= THREADS * VPT * W and,
		// for W == 4, fm_count % 4 == 0 (then every row start is 16-byte aligned).
		// STREAMING: non-temporal loads and stores (the host's choice, by the tensor's size)
		template<int THREADS, int VPT, int W, bool STREAMING>
		__global__ void __launch_bounds__(1024) softmax_rows_kernel(float* out, const float* in, uint32_t rows, uint32_t fm_count)
		{
			__shared__ uint64_t lds_exp[exp_lds_entries];
			__shared__ float lds_partial[2][1024 / wave_size];

			const uint32_t rows_per_block = blockDim.x / THREADS;
			const uint32_t lane = threadIdx.x % THREADS;
			const uint32_t row = blockIdx.x * rows_per_block + threadIdx.x / THREADS;
			const bool row_valid = row < rows;
			const float* src = in + static_cast<size_t>(row_valid ? row : 0) * fm_count;
			float* dst = out + static_cast<size_t>(row_valid ? row : 0) * fm_count;

			// the row is requested first; the expf table is copied to LDS while it is on its way
			float v[VPT][W];
			#pragma unroll
			for(int k = 0; k < VPT; ++k)
			{
				const uint32_t c = (lane + k * THREADS) * W;
				if (row_valid && (c < fm_count))
					vec_io<W, STREAMING>::load(src + c, v[k]);
			}
			stage_exp2_table(lds_exp);
			__syncthreads();
			const exp_context exp_ctx = exp_context_from_lds(lds_exp);

			float m = softmax_max_init;
			#pragma unroll
			for(int k = 0; k < VPT; ++k)
			{
				const uint32_t c = (lane + k * THREADS) * W;
				if (row_valid && (c < fm_count))
				{
					#pragma unroll
					for(int e = 0; e < W; ++e)
						m = ref_max(m, v[k][e]);
				}
			}
			m = wave_all_reduce<(THREADS == 16) ? 16 : 64>(m, max_op());
			if (THREADS > wave_size)
			{
				const uint32_t wave = threadIdx.x / wave_size;
				if ((threadIdx.x % wave_size) == 0)
					lds_partial[0][wave] = m;
				__syncthreads();
				m = softmax_max_init;
				for(uint32_t w = 0; w < THREADS / wave_size; ++w)
					m = ref_max(m, lds_partial[0][w]);
			}

			float sum = 0.0f;
			#pragma unroll
			for(int k = 0; k < VPT; ++k)
			{
				const uint32_t c = (lane + k * THREADS) * W;
				if (row_valid && (c < fm_count))
				{
					float x[W];
					#pragma unroll
					for(int e = 0; e < W; ++e)
						x[e] = v[k][e] - m;
					nnf_expf_batch<W>(x, v[k], exp_ctx);
					#pragma unroll
					for(int e = 0; e < W; ++e)
						sum += v[k][e];
				}
			}
			sum = wave_all_reduce<(THREADS == 16) ? 16 : 64>(sum, sum_op());
			if (THREADS > wave_size)
			{
				const uint32_t wave = threadIdx.x / wave_size;
				if ((threadIdx.x % wave_size) == 0)
					lds_partial[1][wave] = sum;
				__syncthreads();
				sum = 0.0f;
				for(uint32_t w = 0; w < THREADS / wave_size; ++w)
					sum += lds_partial[1][w];
			}

			const float mult = 1.0f / sum;
			#pragma unroll
			for(int k = 0; k < VPT; ++k)
			{
				const uint32_t c = (lane + k * THREADS) * W;
				if (row_valid && (c < fm_count))
				{
					#pragma unroll
					for(int e = 0; e < W; ++e)
						v[k][e] = v[k][e] * mult;
					vec_io<W, STREAMING>::store(dst + c, v[k]);
				}
			}
		}

		// Rows longer than a workgroup's registers hold: one workgroup per row, three passes over the
		// row (the second and third mostly served by the L2 cache), expf values parked in the output
		// like the reference does.
		__global__ void __launch_bounds__(1024) softmax_long_rows_kernel(float* out, const float* in, uint32_t fm_count)
		{
			__shared__ uint64_t lds_exp[exp_lds_entries];
			__shared__ float lds_partial[2][1024 / wave_size];
			stage_exp2_table(lds_exp);

			const float* src = in + static_cast<size_t>(blockIdx.x) * fm_count;
			float* dst = out + static_cast<size_t>(blockIdx.x) * fm_count;
			const uint32_t wave = threadIdx.x / wave_size;
			const uint32_t wave_count = blockDim.x / wave_size;

			float m = softmax_max_init;
			for(uint32_t c = threadIdx.x; c < fm_count; c += blockDim.x)
				m = ref_max(m, src[c]);
			m = wave_all_reduce(m, max_op());
			if ((threadIdx.x % wave_size) == 0)
				lds_partial[0][wave] = m;
			__syncthreads();
			const exp_context exp_ctx = exp_context_from_lds(lds_exp);
			m = softmax_max_init;
			for(uint32_t w = 0; w < wave_count; ++w)
				m = ref_max(m, lds_partial[0][w]);

			float sum = 0.0f;
			for(uint32_t c = threadIdx.x; c < fm_count; c += blockDim.x)
			{
				const float val = nnf_expf(src[c] - m, exp_ctx);
				sum += val;
				dst[c] = val;
			}
			sum = wave_all_reduce(sum, sum_op());
			if ((threadIdx.x % wave_size) == 0)
				lds_partial[1][wave] = sum;
			__syncthreads();
			sum = 0.0f;
			for(uint32_t w = 0; w < wave_count; ++w)
				sum += lds_partial[1][w];

			const float mult = 1.0f / sum;
			for(uint32_t c = threadIdx.x; c < fm_count; c += blockDim.x)
				dst[c] = dst[c] * mult; // each lane re-reads only what it wrote itself
		}

		// neuron_count_per_feature_map > 1. One lane per (entry, position); consecutive lanes take
		// consecutive positions, so every load and store of a wavefront covers 256 consecutive bytes.
		// Same operation order as the reference, including the sequential sum over feature maps.
		//
		// CACHED > 0: the column (fm_count <= CACHED) stays in registers: one read, one write. All
		// CACHED loads are issued at once; the ones beyond fm_count re-read the last feature map
		// (folding a value into the maximum twice changes nothing) and take no part in the sum.
		// CACHED == 0: three passes in batches of eight feature maps (eight loads in flight per lane),
		// expf values parked in the output like the reference does; a lane re-reads only what it wrote.
		constexpr int softmax_column_batch = 8;

		template<int CACHED, bool STREAMING = false>
		__global__ void __launch_bounds__(256) softmax_columns_kernel(float* out, const float* in, uint32_t columns, uint32_t fm_count, uint32_t plane)
		{
			__shared__ uint64_t lds_exp[exp_lds_entries];
			// a feature map's row of a workgroup's columns starts anywhere in a cache line when the plane is no multiple of
			// 32 floats: eight neighbouring workgroups to one XCD, whose L2 then holds the lines they share (256 x 64 feature
			// maps of 28 x 28: 24.5 -> 21.3 us; planes that are multiples of 32 floats unchanged)
			const uint32_t column = xcd_grouped(blockIdx.x, 8u, gridDim.x) * blockDim.x + threadIdx.x;
			const bool valid = column < columns;
			const uint32_t col = valid ? column : columns - 1; // lanes past the end shadow the last column and store nothing
			const uint32_t entry = col / plane;
			const uint32_t pos = col - entry * plane;
			const size_t base = static_cast<size_t>(entry) * fm_count * plane + pos;
			const float* src = in + base;
			float* dst = out + base;
			const uint32_t last = fm_count - 1;

			// The table first: in a streaming kernel the wavefronts of a workgroup should not wait at the
			// barrier for the first wavefront's column loads to come back ahead of its table entry.
			stage_exp2_table(lds_exp);
			__syncthreads();
			const exp_context exp_ctx = exp_context_from_lds(lds_exp);
			if (!valid)
				return;

			if (CACHED > 0)
			{
				constexpr int COUNT = CACHED > 0 ? CACHED : softmax_column_batch;
				constexpr int B = COUNT < softmax_column_batch ? COUNT : softmax_column_batch;
				static_assert(COUNT % B == 0, "whole batches");
				float v[COUNT];
				#pragma unroll
				for(int c = 0; c < COUNT; ++c)
				{
					const float* from = src + static_cast<size_t>(min(static_cast<uint32_t>(c), last)) * plane;
					v[c] = STREAMING ? __builtin_nontemporal_load(from) : *from;
				}
				float m = softmax_max_init;
				#pragma unroll
				for(int c = 0; c < COUNT; ++c)
					m = ref_max(m, v[c]);
				float sum = 0.0f;
				#pragma unroll
				for(int c0 = 0; c0 < COUNT; c0 += B)
				{
					if (static_cast<uint32_t>(c0) < fm_count) // uniform
					{
						float x[B], e[B];
						#pragma unroll
						for(int i = 0; i < B; ++i)
							x[i] = v[c0 + i] - m;
						nnf_expf_batch<B>(x, e, exp_ctx);
						#pragma unroll
						for(int i = 0; i < B; ++i)
						{
							v[c0 + i] = e[i];
							if (static_cast<uint32_t>(c0 + i) < fm_count) // uniform
								sum += e[i];
						}
					}
				}
				const float mult = 1.0f / sum;
				#pragma unroll
				for(int c = 0; c < COUNT; ++c)
				{
					if (static_cast<uint32_t>(c) < fm_count) // uniform
					{
						if (STREAMING)
							__builtin_nontemporal_store(v[c] * mult, dst + static_cast<size_t>(c) * plane);
						else
							dst[static_cast<size_t>(c) * plane] = v[c] * mult;
					}
				}
			}
			else
			{
				constexpr int B = softmax_column_batch;
				float m = softmax_max_init;
				for(uint32_t c0 = 0; c0 < fm_count; c0 += B)
				{
					float x[B];
					#pragma unroll
					for(int i = 0; i < B; ++i)
						x[i] = src[static_cast<size_t>(min(c0 + i, last)) * plane];
					#pragma unroll
					for(int i = 0; i < B; ++i)
						m = ref_max(m, x[i]);
				}
				float sum = 0.0f;
				for(uint32_t c0 = 0; c0 < fm_count; c0 += B)
				{
					float x[B], e[B];
					#pragma unroll
					for(int i = 0; i < B; ++i)
						x[i] = src[static_cast<size_t>(min(c0 + i, last)) * plane] - m;
					nnf_expf_batch<B>(x, e, exp_ctx);
					#pragma unroll
					for(int i = 0; i < B; ++i)
					{
						if (c0 + i < fm_count) // uniform
						{
							sum += e[i];
							dst[static_cast<size_t>(c0 + i) * plane] = e[i];
						}
					}
				}
				const float mult = 1.0f / sum;
				for(uint32_t c0 = 0; c0 < fm_count; c0 += B)
				{
					float x[B];
					#pragma unroll
					for(int i = 0; i < B; ++i)
						x[i] = dst[static_cast<size_t>(min(c0 + i, last)) * plane];
					#pragma unroll
					for(int i = 0; i < B; ++i)
					{
						if (c0 + i < fm_count) // uniform
							dst[static_cast<size_t>(c0 + i) * plane] = x[i] * mult;
					}
				}
			}
		}

		// Columns of up to 16 feature maps when the plane is a multiple of four (more would cost occupancy): a lane takes four neighbouring
		// positions, so every access is a float4 (1 KiB per wavefront) and four independent columns
		// keep the expf pipeline busy. Same operation order per column as above: bit-exact.
		template<int CACHED>
		__global__ void __launch_bounds__(256) softmax_columns_vec4_kernel(float* out, const float* in, uint32_t column_quads, uint32_t fm_count, uint32_t plane)
		{
			__shared__ uint64_t lds_exp[exp_lds_entries];
			const uint32_t quad_id = blockIdx.x * blockDim.x + threadIdx.x;
			const bool valid = quad_id < column_quads;
			const uint32_t quad = valid ? quad_id : column_quads - 1; // lanes past the end shadow the last quad and store nothing
			const uint32_t quads_per_plane = plane / 4;
			const uint32_t entry = quad / quads_per_plane;
			const uint32_t pos = (quad - entry * quads_per_plane) * 4;
			const size_t base = static_cast<size_t>(entry) * fm_count * plane + pos;
			const float* src = in + base;
			float* dst = out + base;
			const uint32_t last = fm_count - 1;

			stage_exp2_table(lds_exp);
			__syncthreads();
			const exp_context exp_ctx = exp_context_from_lds(lds_exp);
			if (!valid)
				return;

			float v[CACHED][4];
			#pragma unroll
			for(int c = 0; c < CACHED; ++c)
			{
				const floatx4 t = load_stream(reinterpret_cast<const floatx4*>(src + static_cast<size_t>(min(static_cast<uint32_t>(c), last)) * plane));
				v[c][0] = t.x; v[c][1] = t.y; v[c][2] = t.z; v[c][3] = t.w;
			}
			float m[4] = { softmax_max_init, softmax_max_init, softmax_max_init, softmax_max_init };
			#pragma unroll
			for(int c = 0; c < CACHED; ++c)
			{
				#pragma unroll
				for(int e = 0; e < 4; ++e)
					m[e] = ref_max(m[e], v[c][e]);
			}
			float sum[4] = { 0.0f, 0.0f, 0.0f, 0.0f };
			#pragma unroll
			for(int c = 0; c < CACHED; ++c)
			{
				if (static_cast<uint32_t>(c) < fm_count) // uniform
				{
					float x[4];
					#pragma unroll
					for(int e = 0; e < 4; ++e)
						x[e] = v[c][e] - m[e];
					nnf_expf_batch<4>(x, v[c], exp_ctx);
					#pragma unroll
					for(int e = 0; e < 4; ++e)
						sum[e] += v[c][e];
				}
			}
			float mult[4];
			#pragma unroll
			for(int e = 0; e < 4; ++e)
				mult[e] = 1.0f / sum[e];
			#pragma unroll
			for(int c = 0; c < CACHED; ++c)
			{
				if (static_cast<uint32_t>(c) < fm_count) // uniform
				{
					floatx4 t;
					t.x = v[c][0] * mult[0]; t.y = v[c][1] * mult[1]; t.z = v[c][2] * mult[2]; t.w = v[c][3] * mult[3];
					store_stream(reinterpret_cast<floatx4*>(dst + static_cast<size_t>(c) * plane), t);
				}
			}
		}

		// neuron_count_per_feature_map > 1 and more than 64 feature maps: one lane per column would make
		// every lane walk a long column alone, with three passes over memory. A workgroup of 256 lanes
		// takes P consecutive columns; the feature maps are cut into S = 256 / P contiguous slices, lane
		// (slice, position) walks its slice in batches of eight, and the slices are combined through LDS
		// in slice order. The maximum is the reference's; the sum is S sequential partial sums added in
		// order instead of one sequential sum, so results can differ from the reference in the last bits
		// (bar: 1e-5 relative, as for rows).
		// STAGED: the workgroup's fm_count x P values stay in LDS between the passes (dynamic LDS of
		// that size): one read and one write of memory. Otherwise the second and third pass re-read
		// memory (small tensors: from the caches), expf values parked in the output.
		template<int P, bool STAGED>
		__global__ void __launch_bounds__(256) softmax_columns_sliced_kernel(float* out, const float* in, uint32_t columns, uint32_t fm_count, uint32_t plane)
		{
			constexpr int S = 256 / P;
			constexpr int B = softmax_column_batch;
			extern __shared__ __align__(16) float lds_values[]; // STAGED: [feature map][position]
			__shared__ uint64_t lds_exp[exp_lds_entries];
			__shared__ float lds_partial[2][S][P];
			stage_exp2_table(lds_exp);
			__syncthreads();
			const exp_context exp_ctx = exp_context_from_lds(lds_exp);

			const uint32_t p = threadIdx.x % P;
			const uint32_t slice = threadIdx.x / P;
			// Neighbouring blocks of positions lie in the same cache lines (P positions are P * 4 bytes of every feature
			// map's row): sixteen of them (four of the wide ones) go to workgroups of one XCD, where the lines meet in one
			// L2 (64 x 1000 feature maps of 7 x 7: 22.0 -> 17.2 us; 256 x 128 of 28 x 28: 45.8 -> 43.8 us).
			const uint32_t column = xcd_grouped(blockIdx.x, (P < 32) ? 16u : 4u, gridDim.x) * P + p;
			const bool valid = column < columns;
			const uint32_t col = valid ? column : columns - 1; // lanes past the end shadow the last column and store nothing
			const uint32_t entry = col / plane;
			const uint32_t pos = col - entry * plane;
			const size_t base = static_cast<size_t>(entry) * fm_count * plane + pos;
			const float* src = in + base;
			float* dst = out + base;

			const uint32_t per_slice = (fm_count + S - 1) / S;
			const uint32_t c_begin = min(slice * per_slice, fm_count);
			const uint32_t c_end = min(c_begin + per_slice, fm_count);
			const uint32_t c_last = (c_end > c_begin) ? c_end - 1 : 0; // an empty slice runs no batch

			float m = softmax_max_init;
			for(uint32_t c0 = c_begin; c0 < c_end; c0 += B)
			{
				float x[B];
				#pragma unroll
				for(int i = 0; i < B; ++i)
					x[i] = src[static_cast<size_t>(min(c0 + i, c_last)) * plane];
				#pragma unroll
				for(int i = 0; i < B; ++i)
				{
					m = ref_max(m, x[i]);
					if (STAGED && (c0 + i < c_end))
						lds_values[(c0 + i) * P + p] = x[i];
				}
			}
			lds_partial[0][slice][p] = m;
			__syncthreads();
			m = softmax_max_init;
			#pragma unroll
			for(int s = 0; s < S; ++s)
				m = ref_max(m, lds_partial[0][s][p]);

			float sum = 0.0f;
			for(uint32_t c0 = c_begin; c0 < c_end; c0 += B)
			{
				float x[B], e[B];
				#pragma unroll
				for(int i = 0; i < B; ++i)
				{
					const uint32_t c = min(c0 + i, c_last);
					x[i] = (STAGED ? lds_values[c * P + p] : src[static_cast<size_t>(c) * plane]) - m;
				}
				nnf_expf_batch<B>(x, e, exp_ctx);
				#pragma unroll
				for(int i = 0; i < B; ++i)
				{
					if (c0 + i < c_end)
					{
						sum += e[i];
						if (STAGED)
							lds_values[(c0 + i) * P + p] = e[i]; // a lane rewrites only what it wrote itself
						else if (valid)
							dst[static_cast<size_t>(c0 + i) * plane] = e[i];
					}
				}
			}
			lds_partial[1][slice][p] = sum;
			__syncthreads();
			sum = 0.0f;
			#pragma unroll
			for(int s = 0; s < S; ++s)
				sum += lds_partial[1][s][p];

			const float mult = 1.0f / sum;
			if (!valid)
				return;
			for(uint32_t c0 = c_begin; c0 < c_end; c0 += B)
			{
				float x[B];
				#pragma unroll
				for(int i = 0; i < B; ++i)
				{
					const uint32_t c = min(c0 + i, c_last);
					x[i] = STAGED ? lds_values[c * P + p] : dst[static_cast<size_t>(c) * plane];
				}
				#pragma unroll
				for(int i = 0; i < B; ++i)
				{
					if (c0 + i < c_end)
						dst[static_cast<size_t>(c0 + i) * plane] = x[i] * mult;
				}
			}
		}

		template<int THREADS, int VPT, int W>
		void launch_rows_kernel(hipStream_t stream, dim3 grid, dim3 block, float* out, const float* in, uint32_t rows, uint32_t fm_count)
		{
			if (static_cast<uint64_t>(rows) * fm_count >= softmax_streaming_floats)
				NNF_LAUNCH((softmax_rows_kernel<THREADS, VPT, W, true>), grid, block, 0, stream, out, in, rows, fm_count);
			else
				NNF_LAUNCH((softmax_rows_kernel<THREADS, VPT, W, false>), grid, block, 0, stream, out, in, rows, fm_count);
		}

		template<int CACHED>
		void launch_columns_kernel(hipStream_t stream, dim3 grid, dim3 block, float* out, const float* in, uint32_t columns, uint32_t fm_count, uint32_t plane)
		{
			if (static_cast<uint64_t>(columns) * fm_count >= softmax_streaming_floats)
				NNF_LAUNCH((softmax_columns_kernel<CACHED, true>), grid, block, 0, stream, out, in, columns, fm_count, plane);
			else
				NNF_LAUNCH((softmax_columns_kernel<CACHED, false>), grid, block, 0, stream, out, in, columns, fm_count, plane);
		}

		template<int THREADS, int W>
		void launch_rows(hipStream_t stream, float* out, const float* in, uint32_t rows, uint32_t fm_count, uint32_t vectors_per_lane)
		{
			// one wavefront per workgroup while there are few rows (spreads them over the compute units)
			const uint32_t block = (THREADS > wave_size) ? THREADS : ((rows >= 4096) ? 256 : wave_size);
			const uint32_t rows_per_block = block / THREADS;
			const dim3 grid((rows + rows_per_block - 1) / rows_per_block);
			if (vectors_per_lane <= 1)
				launch_rows_kernel<THREADS, 1, W>(stream, grid, dim3(block), out, in, rows, fm_count);
			else if (vectors_per_lane <= 2)
				launch_rows_kernel<THREADS, 2, W>(stream, grid, dim3(block), out, in, rows, fm_count);
			else if (vectors_per_lane <= 4)
				launch_rows_kernel<THREADS, 4, W>(stream, grid, dim3(block), out, in, rows, fm_count);
			else if (vectors_per_lane <= 8)
				launch_rows_kernel<THREADS, 8, W>(stream, grid, dim3(block), out, in, rows, fm_count);
			else
				launch_rows_kernel<THREADS, (W == 1) ? 16 : 8, W>(stream, grid, dim3(block), out, in, rows, fm_count);
		}

		template<int THREADS, int W>
		void launch_one_vector_per_lane(hipStream_t stream, float* out, const float* in, uint32_t rows, uint32_t fm_count)
		{
			launch_rows_kernel<THREADS, 1, W>(stream, dim3(rows), dim3(THREADS), out, in, rows, fm_count);
		}

		// Few rows cannot fill the machine with one wavefront each, and what a launch then costs is
		// the serial work of a lane (one expf chain per value it holds): below this row count a row is
		// spread over as many lanes as it has vectors. Measured on 256 rows of 1000 floats: 3.1 us
		// with 256 lanes per row against 4.3 us with one wavefront per row.
		constexpr uint32_t few_rows = 2048;

		// Columns (neuron_count_per_feature_map > 1) of more than 64 feature maps are shared out over
		// the lanes of a workgroup: always when the workgroup's values fit this much LDS (they are
		// then read from memory once), otherwise up to this many columns (small tensors, re-read from
		// the caches); beyond both, one lane walks a column in three passes.
		constexpr size_t staged_bytes_limit = 60 * 1024;
		constexpr uint32_t sliced_columns_limit = 65536;

		template<int W>
		bool try_launch_rows(hipStream_t stream, float* out, const float* in, uint32_t rows, uint32_t fm_count)
		{
			const uint32_t vectors = (fm_count + W - 1) / W;
			if ((rows < few_rows) && (vectors > wave_size) && (vectors <= 1024))
			{
				if (vectors <= 128)
					launch_one_vector_per_lane<128, W>(stream, out, in, rows, fm_count);
				else if (vectors <= 256)
					launch_one_vector_per_lane<256, W>(stream, out, in, rows, fm_count);
				else if (vectors <= 512)
					launch_one_vector_per_lane<512, W>(stream, out, in, rows, fm_count);
				else
					launch_one_vector_per_lane<1024, W>(stream, out, in, rows, fm_count);
				return true;
			}
			if ((rows >= 4096) && (vectors <= 32))
			{
				launch_rows<16, W>(stream, out, in, rows, fm_count, (vectors + 15) / 16);
				return true;
			}
			// (single floats - rows that are no multiple of four floats long, 1001 classes - up to sixteen per lane: a
			// wavefront per row and no barrier, 8192 rows of 1001 37.5 us as one workgroup of 1024 lanes per row)
			if (vectors <= wave_size * ((W == 1) ? 16 : 8))
			{
				launch_rows<wave_size, W>(stream, out, in, rows, fm_count, (vectors + wave_size - 1) / wave_size);
				return true;
			}
			if (vectors <= 1024 * 8)
			{
				launch_rows<1024, W>(stream, out, in, rows, fm_count, (vectors + 1023) / 1024);
				return true;
			}
			return false;
		}
	}

	int softmax_forward(hipStream_t stream, float* output, const float* input,
		uint32_t entry_count, uint32_t feature_map_count, uint32_t neuron_count_per_feature_map)
	{
		if ((output == nullptr) || (input == nullptr) || (feature_map_count == 0) || (neuron_count_per_feature_map == 0))
			return NNF_HIP_EINVAL;
		const uint64_t total64 = static_cast<uint64_t>(entry_count) * feature_map_count * neuron_count_per_feature_map;
		if (total64 == 0)
			return NNF_HIP_OK;
		if (total64 > NNF_HIP_MAX_ELEMENT_COUNT)
			return NNF_HIP_ETOOBIG;
		if (!is_aligned16(output) || !is_aligned16(input))
			return NNF_HIP_EALIGN;
		if (output != input)
		{
			const uintptr_t a = reinterpret_cast<uintptr_t>(output), b = reinterpret_cast<uintptr_t>(input);
			const size_t bytes = static_cast<size_t>(total64) * sizeof(float);
			if ((a < b + bytes) && (b < a + bytes))
				return NNF_HIP_EOVERLAP;
		}

		if (neuron_count_per_feature_map == 1)
		{
			bool launched;
			if ((feature_map_count % 4) == 0)
				launched = try_launch_rows<4>(stream, output, input, entry_count, feature_map_count);
			else
				launched = try_launch_rows<1>(stream, output, input, entry_count, feature_map_count);
			if (!launched)
				NNF_LAUNCH(softmax_long_rows_kernel, dim3(entry_count), dim3(1024), 0, stream, output, input, feature_map_count);
		}
		else
		{
			const uint32_t columns = entry_count * neuron_count_per_feature_map;
			if (feature_map_count > 64)
			{
				// a whole wavefront along the positions (256-byte accesses) once that still gives every
				// compute unit a few workgroups; fewer positions when that is what lets the values fit LDS
				uint32_t positions = (columns >= 64u * 512u) ? 64u : 16u;
				// half a wavefront along the positions when that lets a compute unit hold twice the workgroups
				// (256 x 128 feature maps of 28 x 28: 52.7 us with 64 positions and 32 KB, 46.3 us with 32)
				if ((positions == 64u) && (static_cast<size_t>(feature_map_count) * positions * sizeof(float) > 24u * 1024u))
					positions = 32u;
				while ((positions > 16u) && (static_cast<size_t>(feature_map_count) * positions * sizeof(float) > staged_bytes_limit))
					positions /= 2;
				// eight positions for small tensors whose values then fit: 1000 feature maps of 7 x 7 in one read and one
				// write, 22 us for 64 entries against 36 us in three passes with sixteen (large tensors: 32-byte accesses
				// cost more than the passes, 315 against 137 us on 32 x 150 feature maps of 128 x 128)
				if ((positions == 16u) && (columns <= sliced_columns_limit)
					&& (static_cast<size_t>(feature_map_count) * 16u * sizeof(float) > staged_bytes_limit)
					&& (static_cast<size_t>(feature_map_count) * 8u * sizeof(float) <= staged_bytes_limit))
					positions = 8u;
				const size_t staged_bytes = static_cast<size_t>(feature_map_count) * positions * sizeof(float);
				const dim3 sliced_grid((columns + positions - 1) / positions);
				if (staged_bytes <= staged_bytes_limit)
				{
					if (positions == 64)
						NNF_LAUNCH((softmax_columns_sliced_kernel<64, true>), sliced_grid, dim3(256), staged_bytes, stream,
							output, input, columns, feature_map_count, neuron_count_per_feature_map);
					else if (positions == 32)
						NNF_LAUNCH((softmax_columns_sliced_kernel<32, true>), sliced_grid, dim3(256), staged_bytes, stream,
							output, input, columns, feature_map_count, neuron_count_per_feature_map);
					else if (positions == 16)
						NNF_LAUNCH((softmax_columns_sliced_kernel<16, true>), sliced_grid, dim3(256), staged_bytes, stream,
							output, input, columns, feature_map_count, neuron_count_per_feature_map);
					else
						NNF_LAUNCH((softmax_columns_sliced_kernel<8, true>), sliced_grid, dim3(256), staged_bytes, stream,
							output, input, columns, feature_map_count, neuron_count_per_feature_map);
					return launch_status();
				}
				if (columns <= sliced_columns_limit)
				{
					if (columns >= 64u * 512u)
						NNF_LAUNCH((softmax_columns_sliced_kernel<64, false>), dim3((columns + 63) / 64), dim3(256), 0, stream,
							output, input, columns, feature_map_count, neuron_count_per_feature_map);
					else
						NNF_LAUNCH((softmax_columns_sliced_kernel<16, false>), dim3((columns + 15) / 16), dim3(256), 0, stream,
							output, input, columns, feature_map_count, neuron_count_per_feature_map);
					return launch_status();
				}
			}
			// few columns: one wavefront per workgroup spreads them over more compute units
			const uint32_t block_size = (columns >= 256u * 1024u) ? 256u : 64u;
			const dim3 block(block_size);
			const dim3 grid((columns + block_size - 1) / block_size);
			if (((neuron_count_per_feature_map % 4) == 0) && (feature_map_count <= 16) && (columns >= 4u * 64u * 1024u))
			{
				// four positions per lane while that still leaves every compute unit several wavefronts
				const uint32_t quads = columns / 4;
				const dim3 quad_grid((quads + 255) / 256);
				if (feature_map_count <= 2)
					NNF_LAUNCH(softmax_columns_vec4_kernel<2>, quad_grid, dim3(256), 0, stream, output, input, quads, feature_map_count, neuron_count_per_feature_map);
				else if (feature_map_count <= 4)
					NNF_LAUNCH(softmax_columns_vec4_kernel<4>, quad_grid, dim3(256), 0, stream, output, input, quads, feature_map_count, neuron_count_per_feature_map);
				else if (feature_map_count <= 8)
					NNF_LAUNCH(softmax_columns_vec4_kernel<8>, quad_grid, dim3(256), 0, stream, output, input, quads, feature_map_count, neuron_count_per_feature_map);
				else
					NNF_LAUNCH(softmax_columns_vec4_kernel<16>, quad_grid, dim3(256), 0, stream, output, input, quads, feature_map_count, neuron_count_per_feature_map);
				return launch_status();
			}
			if (feature_map_count <= 2)
				launch_columns_kernel<2>(stream, grid, block, output, input, columns, feature_map_count, neuron_count_per_feature_map);
			else if (feature_map_count <= 4)
				launch_columns_kernel<4>(stream, grid, block, output, input, columns, feature_map_count, neuron_count_per_feature_map);
			else if (feature_map_count <= 8)
				launch_columns_kernel<8>(stream, grid, block, output, input, columns, feature_map_count, neuron_count_per_feature_map);
			else if (feature_map_count <= 16)
				launch_columns_kernel<16>(stream, grid, block, output, input, columns, feature_map_count, neuron_count_per_feature_map);
			else if (feature_map_count <= 32)
				launch_columns_kernel<32>(stream, grid, block, output, input, columns, feature_map_count, neuron_count_per_feature_map);
			else if (feature_map_count <= 64)
				launch_columns_kernel<64>(stream, grid, block, output, input, columns, feature_map_count, neuron_count_per_feature_map);
			else
				NNF_LAUNCH(softmax_columns_kernel<0>, grid, block, 0, stream, output, input, columns, feature_map_count, neuron_count_per_feature_map);
		}
		return launch_status();
	}
}
