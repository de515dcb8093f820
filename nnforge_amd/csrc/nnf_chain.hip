// Fused element-wise group kernel: [per-input layers] -> optional Add -> [layers after the join],
// one read of every input tensor and one write of the output, fp32, layout [entry][feature_map][y][x].
//
// Work split: the tensor is a flat array of floats cut into tiles of block_size * U float4s; one
// workgroup per tile. Lane t of the workgroup owns float4s t, t + block_size, ... of the tile, so every
// load and store instruction of a wavefront covers 1 KiB of consecutive memory. A tile spans only a
// few feature-map planes. When planes are float4-aligned, a lane reads the per-feature-map weights of
// its float4 straight from memory (the lanes of a wavefront hit one or two addresses); otherwise the
// coefficients of the planes a tile touches (batch-norm mult/add, PReLU slope) are computed once per
// workgroup into LDS and looked up per element.
#include "nnf_common.h"

#include <algorithm>
#include <atomic>
#include <cstdlib>
#include <vector>

namespace nnf
{
	namespace
	{

		constexpr int max_slots = NNF_HIP_MAX_OPS;
		// one copy of the expf table per wavefront of the largest workgroup (256 lanes)
		constexpr uint32_t exp_table_bytes = exp_lds_entries * sizeof(uint64_t) * (256 / wave_size);

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

		// SLOTS: layers with per-feature-map weights the group may hold (a single launch takes up to max_slots; the
		// groups of a shared launch travel side by side in the kernel arguments and take batch_slots at most)
		template<int SLOTS>
		struct chain_args_t
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
			chain_slot slots[SLOTS];
		};
		typedef chain_args_t<max_slots> chain_args;
		constexpr int batch_slots = 3;
		typedef chain_args_t<batch_slots> chain_batch_group_args;

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

		// DIRECT path: the COUNT weights of the feature map of each float4 a lane holds. When all lanes
		// of the wavefront agree on the feature map of float4 k (a plane is many wavefront rows long, so
		// they do except where a row crosses a plane boundary), the weights are fetched once per
		// wavefront through the scalar cache and stay out of the vector memory pipeline that streams
		// the tensors; otherwise every lane reads its own.
		template<int U, int COUNT>
		__device__ __forceinline__ void load_direct_weights(const chain_slot& slot, const uint32_t (&where)[U][1], float (&w)[U][COUNT])
		{
			#pragma unroll
			for(int k = 0; k < U; ++k)
			{
				const uint32_t fm = where[k][0];
				const uint32_t wave_fm = __builtin_amdgcn_readfirstlane(fm);
				if (__all(fm == wave_fm))
				{
					#pragma unroll
					for(int c = 0; c < COUNT; ++c)
						w[k][c] = slot.p[c][wave_fm];
				}
				else
				{
					#pragma unroll
					for(int c = 0; c < COUNT; ++c)
						w[k][c] = slot.p[c][fm];
				}
			}
		}

		// Applies one layer to the U float4s a lane holds. The switch is uniform across the workgroup.
		// DIRECT: where[k][0] is the feature map of float4 k and per-feature-map weights are read from
		// memory (all lanes of a wavefront read the same one or two addresses: one cache line).
		// Otherwise where[k][e] indexes the coefficient arrays the workgroup staged in LDS.
		template<int U, bool DIRECT, int EXP_BATCH, class A>
		__device__ __forceinline__ void apply_op(
			int kind,
			const chain_op& op,
			const A& a,
			float (&v)[U][4],
			const uint32_t (&where)[U][DIRECT ? 1 : 4],
			const float2* lds_coeff,
			const exp_context& exp_ctx)
		{
			switch (kind)
			{
			case NNF_HIP_OP_BATCH_NORM:
				if (DIRECT)
				{
					float w[U][4];
					load_direct_weights<U, 4>(a.slots[op.slot], reinterpret_cast<const uint32_t (&)[U][1]>(where), w);
					#pragma unroll
					for(int k = 0; k < U; ++k)
					{
						float mult, add;
						nnf_batch_norm_coefficients(w[k][0], w[k][1], w[k][2], w[k][3], mult, add);
						#pragma unroll
						for(int e = 0; e < 4; ++e)
							v[k][e] = nnf_batch_norm(v[k][e], mult, add);
					}
				}
				else
				{
					const float2* coeff = lds_coeff + op.slot * a.span;
					#pragma unroll
					for(int k = 0; k < U; ++k)
					{
						#pragma unroll
						for(int e = 0; e < 4; ++e)
						{
							const float2 ma = coeff[where[k][DIRECT ? 0 : e]];
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
				if (DIRECT)
				{
					float w[U][1];
					load_direct_weights<U, 1>(a.slots[op.slot], reinterpret_cast<const uint32_t (&)[U][1]>(where), w);
					#pragma unroll
					for(int k = 0; k < U; ++k)
					{
						#pragma unroll
						for(int e = 0; e < 4; ++e)
							v[k][e] = nnf_parametric_rectified_linear(v[k][e], w[k][0]);
					}
				}
				else
				{
					const float2* coeff = lds_coeff + op.slot * a.span;
					#pragma unroll
					for(int k = 0; k < U; ++k)
					{
						#pragma unroll
						for(int e = 0; e < 4; ++e)
							v[k][e] = nnf_parametric_rectified_linear(v[k][e], coeff[where[k][DIRECT ? 0 : e]].x);
					}
				}
				break;
			// The layers that call expf work on batches of EXP_BATCH values (a divisor of 4, or U * 4:
			// the registers of a lane are contiguous). Wider batches
			// let independent evaluations interleave but cost registers, and with them occupancy, in every
			// group a kernel instance runs: the general instance, which also runs the bandwidth-bound
			// groups, uses 1.
			case NNF_HIP_OP_ELU:
				#pragma unroll
				for(int i = 0; i < U * 4; i += EXP_BATCH)
					nnf_exponential_linear<EXP_BATCH>(reinterpret_cast<float (&)[EXP_BATCH]>(v[i / 4][i % 4]), exp_ctx);
				break;
			case NNF_HIP_OP_SIGMOID:
				#pragma unroll
				for(int i = 0; i < U * 4; i += EXP_BATCH)
					nnf_sigmoid<EXP_BATCH>(reinterpret_cast<float (&)[EXP_BATCH]>(v[i / 4][i % 4]), exp_ctx);
				break;
			case NNF_HIP_OP_TANH:
				#pragma unroll
				for(int i = 0; i < U * 4; i += EXP_BATCH)
					nnf_hyperbolic_tangent<EXP_BATCH>(reinterpret_cast<float (&)[EXP_BATCH]>(v[i / 4][i % 4]), op.f1, op.f0, exp_ctx); // f1 holds steepness * 2
				break;
			case NNF_HIP_OP_ABSOLUTE:
				#pragma unroll
				for(int k = 0; k < U; ++k)
				{
					#pragma unroll
					for(int e = 0; e < 4; ++e)
						v[k][e] = nnf_absolute(v[k][e]);
				}
				break;
			default: // NNF_HIP_OP_DROPOUT: the value passes through
				break;
			}
		}

		// ---- pieces of a tile's life, shared by the kernel that takes one tile per workgroup and the one that
		// walks over several -------------------------------------------------------------------------------------

		// The U float4s a lane owns in the tile that starts at element tile_start, for every input tensor.
		// Only one float4 of a whole tensor can be partial: the one that starts at tail_start when the
		// element count is not a multiple of four. It is left out here (zeros) and travels through scalar
		// loads and stores of its own, so that every other access is a float4 guarded by one comparison.
		template<int NIN, int BLOCK, int U, class A>
		__device__ __forceinline__ void load_tile(const A& a, uint32_t tile_start, uint32_t tail_start, float (&x)[NIN][U][4])
		{
			#pragma unroll
			for(int j = 0; j < NIN; ++j)
			{
				#pragma unroll
				for(int k = 0; k < U; ++k)
				{
					const uint32_t idx = tile_start + (threadIdx.x + k * BLOCK) * 4;
					floatx4 t = {0.0f, 0.0f, 0.0f, 0.0f};
					if (idx < tail_start)
						t = load_stream(reinterpret_cast<const floatx4*>(a.in[j] + idx));
					x[j][k][0] = t.x; x[j][k][1] = t.y; x[j][k][2] = t.z; x[j][k][3] = t.w;
				}
			}
		}

		// Whether this lane owns the tensor's partial float4 in the tile at tile_start, and as which of its U.
		template<int BLOCK, int U, class A>
		__device__ __forceinline__ bool owns_tail_vector(const A& a, uint32_t tile_start, uint32_t tail_start, uint32_t& k_tail)
		{
			const uint32_t tail_vector = (tail_start - tile_start) / 4; // float4 index inside this tile, if it is here
			k_tail = tail_vector / BLOCK;
			return (tail_start != a.total) && (tail_start >= tile_start) && (tail_vector < static_cast<uint32_t>(BLOCK * U))
				&& ((tail_vector % BLOCK) == threadIdx.x);
		}

		template<int NIN, int U, class A>
		__device__ __forceinline__ void load_tail_vector(const A& a, uint32_t tail_start, uint32_t k_tail, float (&x)[NIN][U][4])
		{
			#pragma unroll
			for(int j = 0; j < NIN; ++j)
			{
				float tail[3];
				#pragma unroll
				for(int e = 0; e < 3; ++e)
					tail[e] = (tail_start + e < a.total) ? a.in[j][tail_start + e] : 0.0f;
				#pragma unroll
				for(int k = 0; k < U; ++k)
				{
					if (static_cast<uint32_t>(k) == k_tail)
					{
						x[j][k][0] = tail[0]; x[j][k][1] = tail[1]; x[j][k][2] = tail[2];
					}
				}
			}
		}

		template<int BLOCK, int U, class A>
		__device__ __forceinline__ void store_tile(const A& a, uint32_t tile_start, uint32_t tail_start, const float (&v)[U][4])
		{
			#pragma unroll
			for(int k = 0; k < U; ++k)
			{
				const uint32_t idx = tile_start + (threadIdx.x + k * BLOCK) * 4;
				if (idx < tail_start)
				{
					floatx4 t;
					t.x = v[k][0]; t.y = v[k][1]; t.z = v[k][2]; t.w = v[k][3];
					store_stream(reinterpret_cast<floatx4*>(a.out + idx), t);
				}
			}
		}

		template<int U, class A>
		__device__ __forceinline__ void store_tail_vector(const A& a, uint32_t tail_start, uint32_t k_tail, const float (&v)[U][4])
		{
			#pragma unroll
			for(int k = 0; k < U; ++k)
			{
				if (static_cast<uint32_t>(k) == k_tail)
				{
					#pragma unroll
					for(int e = 0; e < 3; ++e)
						if (tail_start + e < a.total)
							a.out[tail_start + e] = v[k][e];
				}
			}
		}

		// Where the lane's values lie: DIRECT - the feature map of each float4; otherwise the index of each
		// element's plane among the planes the tile touches (= its slot in the LDS coefficient arrays).
		// first_fm: feature map of the tile's first plane.
		template<int BLOCK, int U, bool DIRECT, class A>
		__device__ __forceinline__ void locate_tile(const A& a, uint32_t tile_start, uint32_t (&where)[U][DIRECT ? 1 : 4], uint32_t& first_fm)
		{
			constexpr int TILE = BLOCK * U * 4;
			const uint32_t first_plane = tile_start / a.plane;
			const uint32_t start_in_plane = tile_start - first_plane * a.plane;
			first_fm = first_plane % a.fm_count;
			#pragma unroll
			for(int k = 0; k < U; ++k)
			{
				const uint32_t e0 = start_in_plane + (threadIdx.x + k * BLOCK) * 4;
				#pragma unroll
				for(int e = 0; e < (DIRECT ? 1 : 4); ++e)
				{
					uint32_t w = plane_of<TILE>(e0 + e, a.plane, a.plane_magic);
					if (DIRECT)
					{
						w += first_fm; // < 2 * fm_count: the host picks this path only when span <= fm_count
						w = (w >= a.fm_count) ? w - a.fm_count : w;
					}
					where[k][e] = w;
				}
			}
		}

		// Coefficients of the planes a tile touches, once per workgroup into LDS (the caller adds the barrier):
		// batch norm's multiplier and addend, PReLU's slope.
		template<int BLOCK, class A>
		__device__ __forceinline__ void stage_coefficients(const A& a, uint32_t first_fm, float2* lds_coeff)
		{
			for(uint32_t s = 0; s < a.slot_count; ++s)
			{
				const chain_slot& slot = a.slots[s];
				for(uint32_t i = threadIdx.x; i < a.span; i += BLOCK)
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
		}

		// The group's layers in the order the arguments list them: every input's own layers, the Add that
		// joins the inputs (if any), the layers behind it. The result is left in x[0].
		template<int NIN, int U, bool DIRECT, class A>
		__device__ __forceinline__ void run_listed_layers(const A& a, float (&x)[NIN][U][4], const uint32_t (&where)[U][DIRECT ? 1 : 4],
			const float2* lds_coeff, const exp_context& exp_ctx)
		{
			uint32_t op_index = 0;
			#pragma unroll
			for(int j = 0; j < NIN; ++j)
			{
				const uint32_t arm_end = op_index + a.arm_ops[j];
				for(; op_index < arm_end; ++op_index)
					apply_op<U, DIRECT, 1>(a.ops[op_index].kind, a.ops[op_index], a, x[j], where, lds_coeff, exp_ctx);
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
				apply_op<U, DIRECT, 1>(a.ops[op_index].kind, a.ops[op_index], a, x[0], where, lds_coeff, exp_ctx);
		}

		// NIN: number of input tensors. BLOCK: lanes per workgroup. U: float4s per lane.
		// DIRECT: plane % 4 == 0 (a float4 never straddles planes) and a tile touches no feature map
		// twice; per-feature-map weights are then read straight from memory and the workgroup needs
		// neither LDS coefficients nor a barrier. Otherwise coefficients of the planes the tile touches
		// are staged in LDS and looked up per element.
		// PROGRAM: 0 = the layer kinds are read from the arguments (any group); > 0 = index into
		// known_programs: a single-input group whose layer kinds are compile-time constants, so that
		// the whole chain becomes straight-line code (used for the groups that are bound by the
		// vector ALU, i.e. the ones that call expf).
		struct known_program
		{
			int op_count;
			int kinds[NNF_HIP_MAX_OPS];
		};
		constexpr known_program known_programs[] = {
			{ 0, {} },
			{ 4, { NNF_HIP_OP_BATCH_NORM, NNF_HIP_OP_ELU, NNF_HIP_OP_SIGMOID, NNF_HIP_OP_TANH } },
			{ 1, { NNF_HIP_OP_ELU } },
			{ 1, { NNF_HIP_OP_SIGMOID } },
			{ 1, { NNF_HIP_OP_TANH } },
			{ 2, { NNF_HIP_OP_BATCH_NORM, NNF_HIP_OP_ELU } },
			{ 2, { NNF_HIP_OP_BATCH_NORM, NNF_HIP_OP_SIGMOID } },
			{ 2, { NNF_HIP_OP_BATCH_NORM, NNF_HIP_OP_TANH } },
		};
		constexpr int known_program_count = sizeof(known_programs) / sizeof(known_programs[0]);

		// One tile of one group, by one workgroup: the body of the two kernels below.
		template<int NIN, int BLOCK, int U, bool DIRECT, int PROGRAM, class A>
		__device__ __forceinline__ void chain_tile(const A& a, const uint32_t tile_index, unsigned char* lds_raw)
		{
			constexpr int TILE = BLOCK * U * 4;
			constexpr int PL = DIRECT ? 1 : 4;
			uint64_t* lds_exp = reinterpret_cast<uint64_t*>(lds_raw);
			float2* lds_coeff = reinterpret_cast<float2*>(lds_raw + exp_table_bytes);

			const uint32_t tile_start = tile_index * static_cast<uint32_t>(TILE);

			// All loads are issued before anything else: the tensors first (nothing but the tile index
			// goes into their addresses), then the lane's expf table entry and (compile-time programs) the
			// weights of a leading batch norm; the index arithmetic runs while they are in flight.
			const uint32_t tail_start = a.total & ~3u;
			float x[NIN][U][4];
			load_tile<NIN, BLOCK, U>(a, tile_start, tail_start, x);
			uint32_t k_tail;
			const bool owns_tail = owns_tail_vector<BLOCK, U>(a, tile_start, tail_start, k_tail);
			if (owns_tail)
				load_tail_vector<NIN, U>(a, tail_start, k_tail, x);

			constexpr bool program_has_exp = PROGRAM > 0; // every compile-time program calls expf
			uint64_t exp_entry = 0;
			if (program_has_exp || a.need_exp)
				exp_entry = load_exp2_table_entry();

			uint32_t where[U][PL];
			uint32_t first_fm;
			locate_tile<BLOCK, U, DIRECT>(a, tile_start, where, first_fm);

			// compile-time program that starts with a batch norm, weights read straight from memory
			constexpr bool leading_batch_norm = DIRECT && (PROGRAM > 0) && (known_programs[PROGRAM].kinds[0] == NNF_HIP_OP_BATCH_NORM);
			float lead_weights[U][4] = {};
			if (leading_batch_norm)
			{
				load_direct_weights<U, 4>(a.slots[a.ops[0].slot], reinterpret_cast<const uint32_t (&)[U][1]>(where), lead_weights);
			}

			// expf table: one private copy per wavefront, so the direct path has no workgroup barrier
			exp_context exp_ctx = make_exp_context(lds_exp);
			if (program_has_exp || a.need_exp)
				exp_ctx = stage_exp2_table_per_wavefront(lds_exp, exp_entry);
			if (!DIRECT)
			{
				stage_coefficients<BLOCK>(a, first_fm, lds_coeff);
				__syncthreads();
			}

			if (PROGRAM > 0)
			{
				if (leading_batch_norm)
				{
					#pragma unroll
					for(int k = 0; k < U; ++k)
					{
						float mult, add;
						nnf_batch_norm_coefficients(lead_weights[k][0], lead_weights[k][1], lead_weights[k][2], lead_weights[k][3], mult, add);
						#pragma unroll
						for(int e = 0; e < 4; ++e)
							x[0][k][e] = nnf_batch_norm(x[0][k][e], mult, add);
					}
				}
				#pragma unroll
				for(int i = leading_batch_norm ? 1 : 0; i < known_programs[PROGRAM].op_count; ++i)
					apply_op<U, DIRECT, U * 4>(known_programs[PROGRAM].kinds[i], a.ops[i], a, x[0], where, lds_coeff, exp_ctx);
			}
			else
				run_listed_layers<NIN, U, DIRECT>(a, x, where, lds_coeff, exp_ctx);

			store_tile<BLOCK, U>(a, tile_start, tail_start, x[0]);
			if (owns_tail)
				store_tail_vector<U>(a, tail_start, k_tail, x[0]);
		}

		template<int NIN, int BLOCK, int U, bool DIRECT, int PROGRAM>
		__global__ void __launch_bounds__(BLOCK) chain_kernel(const chain_args a)
		{
			extern __shared__ __align__(16) unsigned char lds_raw[];
			chain_tile<NIN, BLOCK, U, DIRECT, PROGRAM>(a, blockIdx.x, lds_raw);
		}

		// A group whose result goes to a part of a wider tensor: entry e of the result starts out_entry_stride floats
		// behind entry e - 1 instead of right behind it (the group writes its feature maps into the tensor of the Concat
		// layer that would otherwise copy them there). The grid is (tiles of one entry) x (entries): a workgroup sees
		// the arguments of a group of one entry, with the tensors' addresses moved to its entry, and does what
		// chain_kernel does. The arguments' a.total is the number of elements of one entry.
		template<int SLOTS>
		struct chain_entry_view
		{
			const float* in[NNF_HIP_MAX_INPUTS];
			float* out;
			uint32_t total, fm_count, plane, plane_magic, span, has_add;
			float alpha;
			uint32_t arm_ops[NNF_HIP_MAX_INPUTS];
			uint32_t tail_ops, slot_count, need_exp;
			const chain_op (&ops)[NNF_HIP_MAX_OPS];
			const chain_slot (&slots)[SLOTS];
		};

		// Up to max_strided_batch such groups in one launch (the branches in front of one Concat layer): along x the
		// tiles of one entry of every group, one group after the other, along y the entries. A workgroup finds its group
		// by its x index and takes the body of the group's kind (one input or two, weights straight from memory or
		// through LDS coefficients), 256 lanes x 2 float4s each.
		constexpr uint32_t max_strided_batch = NNF_HIP_MAX_STRIDED_GROUPS_PER_LAUNCH;
		struct chain_strided_batch_args
		{
			uint32_t count;
			uint32_t direct_mask;     // bit g: group g reads its weights straight from memory
			uint32_t two_input_mask;  // bit g: group g has two inputs
			uint32_t entry_count;
			uint32_t tile_end[max_strided_batch];         // running total of the groups' tiles per entry
			uint32_t out_entry_stride[max_strided_batch]; // floats from one entry of the group's result to the next
			chain_args group[max_strided_batch];          // total: the elements of one entry
		};
		static_assert(sizeof(chain_strided_batch_args) <= 4096, "kernel arguments of a strided batch beyond 4 KB");

		// ALL_DIRECT: every group of the launch reads its weights straight from memory; ONE_INPUT: every group has one
		// input. The launch whose groups are all of one kind holds one body instead of four and half the registers
		// (48 against 102 per lane: four Inception branches of 512 entries 135 against 172 us).
		// U: float4s per lane - 2, or 4 for the launch of one kind whose workgroups then make one round of the machine
		// (four branches of 32 entries, 51 MB moved: 11.7 -> 10.7 us; at 128 entries no difference, at 512 entries 3 % slower)
		template<int BLOCK, bool ALL_DIRECT, bool ONE_INPUT, int U = 2>
		__global__ void __launch_bounds__(BLOCK) chain_entries_batch_kernel(const chain_strided_batch_args b)
		{
			extern __shared__ __align__(16) unsigned char lds_raw[];
			uint32_t g = 0;
			while ((g + 1 < b.count) && (blockIdx.x >= b.tile_end[g]))
				++g;
			const uint32_t tile_index = blockIdx.x - ((g == 0) ? 0u : b.tile_end[g - 1]);
			const chain_args& a = b.group[g];
			const bool direct = ALL_DIRECT || (((b.direct_mask >> g) & 1u) != 0);
			const bool two_inputs = !ONE_INPUT && (((b.two_input_mask >> g) & 1u) != 0);
			for(uint32_t entry = blockIdx.y; entry < b.entry_count; entry += gridDim.y)
			{
				chain_entry_view<max_slots> v = {
					{}, a.out + static_cast<size_t>(entry) * b.out_entry_stride[g],
					a.total, a.fm_count, a.plane, a.plane_magic, a.span, a.has_add, a.alpha,
					{}, a.tail_ops, a.slot_count, a.need_exp, a.ops, a.slots };
				#pragma unroll
				for(int j = 0; j < NNF_HIP_MAX_INPUTS; ++j)
				{
					v.in[j] = ((j == 0) || ((j == 1) && two_inputs)) ? a.in[j] + static_cast<size_t>(entry) * a.total : nullptr;
					v.arm_ops[j] = a.arm_ops[j];
				}
				if (two_inputs)
				{
					if (direct)
						chain_tile<2, BLOCK, U, true, 0>(v, tile_index, lds_raw);
					else
						chain_tile<2, BLOCK, U, false, 0>(v, tile_index, lds_raw);
				}
				else
				{
					if (direct)
						chain_tile<1, BLOCK, U, true, 0>(v, tile_index, lds_raw);
					else
						chain_tile<1, BLOCK, U, false, 0>(v, tile_index, lds_raw);
				}
				if (entry + gridDim.y < b.entry_count)
					__syncthreads(); // the next entry's coefficients go where this one's are still being read
			}
		}

		// Several groups that have nothing to do with each other in one launch: the grid is the groups' tiles one
		// after the other, a workgroup finds its group by its index and then does what chain_kernel does. The time a
		// launch loses while the device fills and drains is paid once for all of them (measured with 51 one-read-
		// one-write tensors of the ResNet-50 stack's sizes: 915 us one by one, 831 us six per launch, at 64 entries;
		// 214 against 121 us at 8 entries). All groups of a launch share NIN and the launch shape (groups of two kinds
		// in one launch: chain_batch_mixed_kernel below). DIRECT_MODE: how
		// they read their weights - all through LDS coefficients (0), all straight from memory (1), or each its own way
		// (2: direct_mask says which; the workgroup takes one path or the other as a whole).
		constexpr uint32_t max_batch = NNF_HIP_MAX_GROUPS_PER_LAUNCH; // what 4 KB of kernel arguments hold
		struct chain_batch_args
		{
			uint32_t count;
			uint32_t direct_mask;         // bit g: group g reads its weights straight from memory
			uint32_t two_input_mask;      // bit g: group g has two inputs (chain_batch_mixed_kernel)
			uint32_t tile_end[max_batch]; // running total of the groups' tile counts
			chain_batch_group_args group[max_batch];
		};
		static_assert(sizeof(chain_batch_args) <= 4096, "kernel arguments of a batch beyond 4 KB");

		template<int NIN, int BLOCK, int U, int DIRECT_MODE>
		__global__ void __launch_bounds__(BLOCK) chain_batch_kernel(const chain_batch_args b)
		{
			extern __shared__ __align__(16) unsigned char lds_raw[];
			uint32_t g = 0;
			while ((g + 1 < b.count) && (blockIdx.x >= b.tile_end[g]))
				++g;
			const uint32_t tile_index = blockIdx.x - ((g == 0) ? 0u : b.tile_end[g - 1]);
			if ((DIRECT_MODE == 1) || ((DIRECT_MODE == 2) && (((b.direct_mask >> g) & 1u) != 0)))
				chain_tile<NIN, BLOCK, U, true, 0>(b.group[g], tile_index, lds_raw);
			else
				chain_tile<NIN, BLOCK, U, false, 0>(b.group[g], tile_index, lds_raw);
		}

		// Groups with one input (four float4s per lane; two where the weights go through LDS coefficients, which keeps
		// the kernel at 60 registers per lane, eight wavefronts per SIMD) and groups with two (two float4s per lane) in one
		// launch: the tiles differ in size, the workgroups do not (BLOCK lanes), and a workgroup takes the body of its
		// group's kind.
		// What this buys: the groups of a residual network that wait for each other (the joins of a stage) are few
		// per level of the graph, and each level can take a share of the groups that wait for nothing along, instead of
		// being a small launch of its own.
		template<int BLOCK, int DIRECT_MODE>
		__global__ void __launch_bounds__(BLOCK) chain_batch_mixed_kernel(const chain_batch_args b)
		{
			extern __shared__ __align__(16) unsigned char lds_raw[];
			uint32_t g = 0;
			while ((g + 1 < b.count) && (blockIdx.x >= b.tile_end[g]))
				++g;
			const uint32_t tile_index = blockIdx.x - ((g == 0) ? 0u : b.tile_end[g - 1]);
			const bool direct = (DIRECT_MODE == 1) || ((DIRECT_MODE == 2) && (((b.direct_mask >> g) & 1u) != 0));
			if (((b.two_input_mask >> g) & 1u) != 0)
			{
				if (direct)
					chain_tile<2, BLOCK, 2, true, 0>(b.group[g], tile_index, lds_raw);
				else
					chain_tile<2, BLOCK, 2, false, 0>(b.group[g], tile_index, lds_raw);
			}
			else
			{
				if (direct)
					chain_tile<1, BLOCK, 4, true, 0>(b.group[g], tile_index, lds_raw);
				else
					chain_tile<1, BLOCK, 2, false, 0>(b.group[g], tile_index, lds_raw);
			}
		}

		// The same group on a grid that stays put: as many workgroups as the device holds at once (or fewer), each
		// walking over tiles blockIdx.x, blockIdx.x + gridDim.x, ... with the next tile's loads issued before the
		// current tile is computed and stored, so a lane always has loads in flight. Tiles that run at the same
		// moment are neighbours in memory, as with one tile per workgroup. Planes are float4-aligned and no tile
		// touches a feature map twice (the DIRECT case above): weights come straight from memory, no LDS
		// coefficients, no barrier.
		template<int NIN, int BLOCK, int U>
		__global__ void __launch_bounds__(BLOCK) chain_kernel_persistent(const chain_args a, const uint32_t tile_count)
		{
			constexpr int TILE = BLOCK * U * 4;
			extern __shared__ __align__(16) unsigned char lds_raw[];
			uint64_t* lds_exp = reinterpret_cast<uint64_t*>(lds_raw);

			const uint32_t tail_start = a.total & ~3u;
			uint32_t tile = blockIdx.x;
			if (tile >= tile_count)
				return;
			float x[NIN][U][4];
			load_tile<NIN, BLOCK, U>(a, tile * static_cast<uint32_t>(TILE), tail_start, x);

			exp_context exp_ctx = make_exp_context(lds_exp);
			if (a.need_exp)
				exp_ctx = stage_exp2_table_per_wavefront(lds_exp, load_exp2_table_entry());

			for(;;)
			{
				const uint32_t tile_start = tile * static_cast<uint32_t>(TILE);
				const uint32_t next_tile = tile + gridDim.x;
				const bool more = next_tile < tile_count;
				float next_x[NIN][U][4];
				if (more)
					load_tile<NIN, BLOCK, U>(a, next_tile * static_cast<uint32_t>(TILE), tail_start, next_x);

				uint32_t k_tail;
				const bool owns_tail = owns_tail_vector<BLOCK, U>(a, tile_start, tail_start, k_tail);
				if (owns_tail)
					load_tail_vector<NIN, U>(a, tail_start, k_tail, x);
				uint32_t where[U][1];
				uint32_t first_fm;
				locate_tile<BLOCK, U, true>(a, tile_start, where, first_fm);
				run_listed_layers<NIN, U, true>(a, x, where, nullptr, exp_ctx);
				store_tile<BLOCK, U>(a, tile_start, tail_start, x[0]);
				if (owns_tail)
					store_tail_vector<U>(a, tail_start, k_tail, x[0]);

				if (!more)
					break;
				#pragma unroll
				for(int j = 0; j < NIN; ++j)
				{
					#pragma unroll
					for(int k = 0; k < U; ++k)
					{
						#pragma unroll
						for(int e = 0; e < 4; ++e)
							x[j][k][e] = next_x[j][k][e];
					}
				}
				tile = next_tile;
			}
		}

		typedef void (*chain_kernel_fn)(const chain_args);
		typedef void (*chain_persistent_kernel_fn)(const chain_args, const uint32_t);

		// Launch shapes (lanes per workgroup, float4s per lane), largest tile first; the last one is the
		// grid that stays put (chain_kernel_persistent).
		struct launch_shape
		{
			int block;
			int unroll;
			bool persistent;
		};
		constexpr launch_shape launch_shapes[] = { {256, 4, false}, {256, 2, false}, {256, 1, false}, {64, 1, false}, {256, 4, true} };
		constexpr int launch_shape_count = sizeof(launch_shapes) / sizeof(launch_shapes[0]);
		constexpr int persistent_shape = 4;

		template<int NIN, int BLOCK, int U, int PROGRAM>
		chain_kernel_fn pick_direct(bool direct)
		{
			return direct ? chain_kernel<NIN, BLOCK, U, true, PROGRAM> : chain_kernel<NIN, BLOCK, U, false, PROGRAM>;
		}

		template<int NIN, int PROGRAM>
		chain_kernel_fn pick_shape(int shape, bool direct)
		{
			switch (shape)
			{
			// the compile-time programs are bound by the vector ALU: four float4s per lane would only
			// cost them occupancy
			case 0: return pick_direct<NIN, 256, (PROGRAM > 0) ? 2 : 4, PROGRAM>(direct);
			case 1: return pick_direct<NIN, 256, 2, PROGRAM>(direct);
			case 2: return pick_direct<NIN, 256, 1, PROGRAM>(direct);
			default: return pick_direct<NIN, 64, 1, PROGRAM>(direct);
			}
		}

		chain_kernel_fn pick_kernel(uint32_t input_count, int shape, bool direct, int program)
		{
			switch (program)
			{
			case 1: return pick_shape<1, 1>(shape, direct);
			case 2: return pick_shape<1, 2>(shape, direct);
			case 3: return pick_shape<1, 3>(shape, direct);
			case 4: return pick_shape<1, 4>(shape, direct);
			case 5: return pick_shape<1, 5>(shape, direct);
			case 6: return pick_shape<1, 6>(shape, direct);
			case 7: return pick_shape<1, 7>(shape, direct);
			default: break;
			}
			switch (input_count)
			{
			case 1: return pick_shape<1, 0>(shape, direct);
			case 2: return pick_shape<2, 0>(shape, direct);
			case 3: return pick_shape<3, 0>(shape, direct);
			default: return pick_shape<4, 0>(shape, direct);
			}
		}

		chain_persistent_kernel_fn pick_persistent_kernel(uint32_t input_count)
		{
			return chain_kernel_persistent<1, 256, 4>; // one input only: see persistent_max_inputs
		}

		// index into known_programs of a single-input group without Add, 0 when it is not one of them
		int match_known_program(const nnf_hip_chain_desc& desc, uint32_t op_count)
		{
			if ((desc.input_count != 1) || desc.has_add)
				return 0;
			for(int p = 1; p < known_program_count; ++p)
			{
				if (known_programs[p].op_count != static_cast<int>(op_count))
					continue;
				bool same = true;
				for(uint32_t i = 0; i < op_count; ++i)
					same = same && (known_programs[p].kinds[i] == desc.ops[i].kind);
				if (same)
					return p;
			}
			return 0;
		}

		// NNF_HIP_CHAIN_SHAPE=<index into launch_shapes> (declared in nnforge_hip.h) forces a launch shape where it is
		// possible; read once per process. -1 = automatic.
		int forced_shape()
		{
			static const int value = []
			{
				const char* s = getenv("NNF_HIP_CHAIN_SHAPE");
				if ((s == nullptr) || (*s == '\0'))
					return -1;
				const int v = atoi(s);
				return ((v >= 0) && (v < launch_shape_count)) ? v : -1;
			}();
			return value;
		}

		bool ranges_overlap(const void* a, size_t a_bytes, const void* b, size_t b_bytes)
		{
			const uintptr_t pa = reinterpret_cast<uintptr_t>(a);
			const uintptr_t pb = reinterpret_cast<uintptr_t>(b);
			return (pa < pb + b_bytes) && (pb < pa + a_bytes);
		}

		bool ranges_overlap(const void* a, const void* b, size_t bytes)
		{
			return ranges_overlap(a, bytes, b, bytes);
		}

		constexpr size_t max_dynamic_lds = 64 * 1024;
		// Below this many tiles a smaller tile is used so that more compute units get work.
		constexpr uint32_t min_tiles_wanted = 1024;
		// From this size on (64 MB per tensor) the smaller tile is used.
		constexpr uint32_t large_tensor_elements = 1u << 24;
		// The grid that stays put is built for groups with one input: it holds two tiles per lane and input (74
		// vector registers with one input, five workgroups per compute unit; 106 with two, where it measured no
		// faster than one tile per workgroup at any size).
		constexpr uint32_t resident_workgroups_per_compute_unit = 8; // of 256 lanes at up to 64 vector registers
		constexpr uint32_t persistent_max_inputs = 1;
		constexpr uint32_t persistent_workgroups_per_compute_unit = 5;
	}

	namespace
	{
		// A group checked and ready to launch: the kernel's arguments and the launch shape chosen for it.
		struct prepared_group
		{
			chain_args a;
			bool nothing_to_do; // zero elements
			int shape;          // index into launch_shapes
			bool direct;
			int program;        // index into known_programs, 0: the layer list is interpreted
			uint32_t input_count;
			uint32_t tiles;
			size_t lds_bytes;
			size_t bytes;       // of one tensor
		};

		// Checks the call's arguments and fills p. single_launch: the group gets a launch of its own, so the grid
		// that stays put is a candidate; as one of several groups of a launch it is not.
		// wanted_shape >= 0: that launch shape and the interpreted layer list, whatever the size suggests (the launch over
		// entries has instances for one shape).
		int prepare_group(const nnf_hip_chain_desc* desc, float* output, const float* const* inputs, const float* const* chunk_ptrs,
			bool single_launch, prepared_group& p, int wanted_shape = -1)
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

			p = prepared_group();
			p.input_count = desc->input_count;
			const uint64_t total64 = static_cast<uint64_t>(desc->entry_count) * desc->feature_map_count * desc->neuron_count_per_feature_map;
			if (total64 == 0)
			{
				p.nothing_to_do = true; // as the reference's loops over zero elements
				return NNF_HIP_OK;
			}
			if (total64 > NNF_HIP_MAX_ELEMENT_COUNT)
				return NNF_HIP_ETOOBIG;
			p.bytes = static_cast<size_t>(total64) * sizeof(float);

			chain_args& a = p.a;
			if (!is_aligned16(output))
				return NNF_HIP_EALIGN;
			for(uint32_t j = 0; j < desc->input_count; ++j)
			{
				if (inputs[j] == nullptr)
					return NNF_HIP_EINVAL;
				if (!is_aligned16(inputs[j]))
					return NNF_HIP_EALIGN;
				const bool exact_alias_of_first = (j == 0) && (inputs[j] == output);
				if (!exact_alias_of_first && ranges_overlap(inputs[j], output, p.bytes))
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
				case NNF_HIP_OP_ABSOLUTE:
				case NNF_HIP_OP_DROPOUT:
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
			auto span_of = [&](int shape) -> uint32_t
			{
				const uint32_t tile = launch_shapes[shape].block * launch_shapes[shape].unroll * 4;
				return (tile + a.plane - 2) / a.plane + 1;
			};
			// weights are read straight from memory when a float4 never straddles planes and a tile
			// touches no feature map twice; otherwise the workgroup stages coefficients in LDS
			auto direct_of = [&](int shape) -> bool
			{
				if (a.slot_count == 0)
					return true; // no layer reads per-feature-map weights: nothing to look up, nothing to stage
				return ((a.plane % 4) == 0) && (span_of(shape) <= a.fm_count);
			};
			auto lds_bytes_of = [&](int shape) -> size_t
			{
				if (direct_of(shape))
					return exp_table_bytes;
				return exp_table_bytes + static_cast<size_t>(a.slot_count) * span_of(shape) * sizeof(float2);
			};
			auto tiles_of = [&](int shape) -> uint32_t
			{
				const uint32_t tile = launch_shapes[shape].block * launch_shapes[shape].unroll * 4;
				return (a.total + tile - 1) / tile;
			};

			const int program = (wanted_shape >= 0) ? 0 : match_known_program(*desc, op_count);
			// the grid that stays put exists for the interpreted layer list with weights read straight from memory
			auto persistent_possible = [&]() -> bool
			{
				return single_launch && (program == 0) && (desc->input_count <= persistent_max_inputs) && direct_of(persistent_shape);
			};
			int shape = (wanted_shape >= 0) ? wanted_shape : forced_shape();
			if ((shape == persistent_shape) && !persistent_possible())
				shape = -1;
			if ((wanted_shape >= 0) && (lds_bytes_of(shape) > max_dynamic_lds))
				return NNF_HIP_EUNSUPPORTED;
			const bool automatic = (shape < 0) || (lds_bytes_of(shape) > max_dynamic_lds);
			if (automatic)
			{
				// Measured on MI355X. One input: tensors of 64 MB and more stream best with two float4s per lane,
				// smaller ones with four, as long as enough workgroups exist to cover the machine. Several inputs:
				// two float4s per lane at every size (4 % faster than four from 10 to 130 MB per tensor).
				// As one of several groups of a launch: the tile size follows the number of inputs alone (four float4s per lane
				// with one input, two with several) - the grid is all the groups' tiles, so a small group need not be cut
				// finer to cover the machine, and groups of one tile size share launches (the 49 groups of the ResNet-50
				// stack at 64 entries, launched together where they can be: 1067-1071 us this way, 1078 with four float4s
				// for all, 1067 with two for all, 1189 with one, 1085 with the sizes chosen as for single launches).
				static const int small_tile_order[] = { 1, 2, 3 };
				static const int any_tile_order[] = { 0, 1, 2, 3 };
				const bool large = (a.total >= large_tensor_elements) || !single_launch;
				const bool small_tiles = (single_launch && large) || (desc->input_count > 1);
				const int* order = small_tiles ? small_tile_order : any_tile_order;
				const int order_count = small_tiles ? 3 : 4;
				shape = -1;
				for(int i = 0; i < order_count; ++i)
				{
					const int s = order[i];
					if (lds_bytes_of(s) > max_dynamic_lds)
						continue;
					if (large || (tiles_of(s) >= min_tiles_wanted) || (i == order_count - 1))
					{
						shape = s;
						break;
					}
				}
				if (shape < 0)
					return NNF_HIP_EUNSUPPORTED;
			}
			if ((program > 0) && (shape == 0))
				shape = 1; // the compile-time programs have no four-float4 instance (smaller tile: LDS still fits)
			// as one of several groups of a launch, a group with one input whose weights go through LDS coefficients takes
			// two float4s per lane: the body chain_batch_mixed_kernel has for it
			if (automatic && !single_launch && (desc->input_count == 1) && (shape == 0) && !direct_of(0))
				shape = 1;
			// One input, four float4s per lane, and more tiles than the device holds workgroups at once (8 per compute
			// unit: above 33 MB per tensor): a second, partial round of workgroups would follow the first and the time per
			// byte jumps (32 MB: 11.0 us, 38.5 MB: 15.5 us). There the grid that stays put takes over, five workgroups
			// per compute unit walking over the tiles with the next tile's loads in flight while the current one is
			// stored (38.5 MB: 13.3 us, 51.4 MB: 18.8 -> 17.3 us). With fewer tiles every workgroup has one tile anyway and
			// the plain grid is as fast or faster (25.7 MB: 9.1 against 9.4 us); from 64 MB on the two are equal.
			if (automatic && (shape == 0) && (tiles_of(0) > compute_unit_count() * resident_workgroups_per_compute_unit) && persistent_possible())
				shape = persistent_shape;
			a.span = span_of(shape);
			a.plane_magic = (a.plane >= 2) ? static_cast<uint32_t>(((1ull << 32) + a.plane - 1) / a.plane) : 0u;
			p.shape = shape;
			p.direct = direct_of(shape);
			p.program = program;
			p.tiles = tiles_of(shape);
			p.lds_bytes = launch_shapes[shape].persistent ? exp_table_bytes : lds_bytes_of(shape);
			return NNF_HIP_OK;
		}

		int launch_group(hipStream_t stream, const prepared_group& p)
		{
			if (p.nothing_to_do)
				return NNF_HIP_OK;
			const launch_shape& shape = launch_shapes[p.shape];
			if (shape.persistent)
			{
				const uint32_t grid = std::min(p.tiles, compute_unit_count() * persistent_workgroups_per_compute_unit);
				NNF_LAUNCH(pick_persistent_kernel(p.input_count), dim3(grid), dim3(shape.block), p.lds_bytes, stream, p.a, p.tiles);
				return launch_status();
			}
			NNF_LAUNCH(pick_kernel(p.input_count, p.shape, p.direct, p.program), dim3(p.tiles), dim3(shape.block), p.lds_bytes, stream, p.a);
			return launch_status();
		}

		typedef void (*chain_batch_kernel_fn)(const chain_batch_args);

		// a group's arguments in the form they take among the arguments of a shared launch (slot_count <= batch_slots)
		chain_batch_group_args batch_group_args_of(const chain_args& a)
		{
			chain_batch_group_args c = {};
			for(int j = 0; j < NNF_HIP_MAX_INPUTS; ++j)
			{
				c.in[j] = a.in[j];
				c.arm_ops[j] = a.arm_ops[j];
			}
			c.out = a.out;
			c.total = a.total;
			c.fm_count = a.fm_count;
			c.plane = a.plane;
			c.plane_magic = a.plane_magic;
			c.span = a.span;
			c.has_add = a.has_add;
			c.alpha = a.alpha;
			c.tail_ops = a.tail_ops;
			c.slot_count = a.slot_count;
			c.need_exp = a.need_exp;
			for(int i = 0; i < NNF_HIP_MAX_OPS; ++i)
				c.ops[i] = a.ops[i];
			for(int i = 0; i < batch_slots; ++i)
				c.slots[i] = a.slots[i];
			return c;
		}

		template<int NIN, int BLOCK, int U>
		chain_batch_kernel_fn pick_batch_kernel_mode(int direct_mode)
		{
			switch (direct_mode)
			{
			case 0: return chain_batch_kernel<NIN, BLOCK, U, 0>;
			case 1: return chain_batch_kernel<NIN, BLOCK, U, 1>;
			default: return chain_batch_kernel<NIN, BLOCK, U, 2>;
			}
		}

		template<int NIN>
		chain_batch_kernel_fn pick_batch_kernel_of(int shape, int direct_mode)
		{
			switch (shape)
			{
			case 0: return pick_batch_kernel_mode<NIN, 256, 4>(direct_mode);
			case 1: return pick_batch_kernel_mode<NIN, 256, 2>(direct_mode);
			case 2: return pick_batch_kernel_mode<NIN, 256, 1>(direct_mode);
			default: return pick_batch_kernel_mode<NIN, 64, 1>(direct_mode);
			}
		}

		chain_batch_kernel_fn pick_batch_mixed_kernel(int direct_mode)
		{
			switch (direct_mode)
			{
			case 0: return chain_batch_mixed_kernel<256, 0>;
			case 1: return chain_batch_mixed_kernel<256, 1>;
			default: return chain_batch_mixed_kernel<256, 2>;
			}
		}

		// the two kinds of group chain_batch_mixed_kernel takes side by side
		bool mixes(const prepared_group& g)
		{
			return ((g.input_count == 1) && (g.shape == (g.direct ? 0 : 1))) || ((g.input_count == 2) && (g.shape == 1));
		}

		chain_batch_kernel_fn pick_batch_kernel(uint32_t input_count, int shape, int direct_mode)
		{
			switch (input_count)
			{
			case 1: return pick_batch_kernel_of<1>(shape, direct_mode);
			case 2: return pick_batch_kernel_of<2>(shape, direct_mode);
			case 3: return pick_batch_kernel_of<3>(shape, direct_mode);
			default: return pick_batch_kernel_of<4>(shape, direct_mode);
			}
		}
	}

	int chain_forward(hipStream_t stream, const nnf_hip_chain_desc* desc, float* output,
		const float* const* inputs, const float* const* chunk_ptrs)
	{
		prepared_group p;
		const int rc = prepare_group(desc, output, inputs, chunk_ptrs, true, p);
		return (rc != NNF_HIP_OK) ? rc : launch_group(stream, p);
	}

	// The launch over entries has instances for one or two inputs and 256 lanes x 2 float4s, and one for groups of one
	// input with weights straight from memory and 4 float4s.
	constexpr int strided_shape = 1;
	constexpr int strided_wide_shape = 0;

	int chain_forward_strided_status(const nnf_hip_chain_desc* desc, uint32_t output_entry_stride)
	{
		if (desc == nullptr)
			return NNF_HIP_EINVAL;
		const uint64_t per_entry = static_cast<uint64_t>(desc->feature_map_count) * desc->neuron_count_per_feature_map;
		if ((per_entry == 0) || (desc->input_count < 1))
			return NNF_HIP_EINVAL;
		if (output_entry_stride < per_entry)
			return NNF_HIP_EINVAL;
		// every entry of the tensors starts on a 16-byte boundary, and at most two inputs
		if (((per_entry % 4) != 0) || ((output_entry_stride % 4) != 0) || (desc->input_count > 2))
			return NNF_HIP_EUNSUPPORTED;
		if (static_cast<uint64_t>(desc->entry_count) * output_entry_stride > NNF_HIP_MAX_ELEMENT_COUNT)
			return NNF_HIP_ETOOBIG;
		return NNF_HIP_OK;
	}

	int chain_forward_strided_batch(hipStream_t stream, uint32_t group_count, const nnf_hip_chain_desc* descs, float* const* outputs,
		const uint32_t* output_entry_strides, const float* const* const* inputs, const float* const* const* chunk_ptrs)
	{
		if (group_count == 0)
			return NNF_HIP_OK;
		if ((descs == nullptr) || (outputs == nullptr) || (output_entry_strides == nullptr) || (inputs == nullptr))
			return NNF_HIP_EINVAL;
		// everything is checked before anything is launched
		const uint32_t entry_count = descs[0].entry_count;
		for(uint32_t i = 0; i < group_count; ++i)
		{
			const int rc = chain_forward_strided_status(&descs[i], output_entry_strides[i]);
			if (rc != NNF_HIP_OK)
				return rc;
			if (descs[i].entry_count != entry_count)
				return NNF_HIP_EINVAL; // the groups of a call go entry by entry together
		}
		if (entry_count == 0)
			return NNF_HIP_OK; // as the reference's loops over zero entries
		std::vector<prepared_group> groups(group_count);
		// planned as groups of one entry: with the wide tiles where all groups of the call are of the one kind that has them
		// and the launch is then one round of workgroups that still covers the machine, with the narrow ones otherwise
		bool wide = group_count <= max_strided_batch;
		for(;;)
		{
			uint64_t tiles = 0;
			bool of_the_kind = true;
			for(uint32_t i = 0; i < group_count; ++i)
			{
				nnf_hip_chain_desc one = descs[i];
				one.entry_count = 1;
				const int rc = prepare_group(&one, outputs[i], inputs[i], (chunk_ptrs == nullptr) ? nullptr : chunk_ptrs[i], false, groups[i],
					wide ? strided_wide_shape : strided_shape);
				if ((rc != NNF_HIP_OK) && !wide)
					return rc;
				of_the_kind = of_the_kind && (rc == NNF_HIP_OK) && groups[i].direct && (groups[i].input_count == 1);
				tiles += groups[i].tiles;
			}
			if (!wide)
				break;
			const uint64_t workgroups = tiles * entry_count;
			if (of_the_kind && (workgroups >= 2ull * compute_unit_count()) && (workgroups <= static_cast<uint64_t>(resident_workgroups_per_compute_unit) * compute_unit_count()))
				break;
			wide = false; // once more, with the narrow tiles
		}
		// What group i writes: entry_count pieces of its entry size, output_entry_strides[i] floats apart. No input of the
		// call may lie inside the span they cover, and the pieces of two groups may not meet: either their spans are
		// apart, or they step alike and their pieces lie side by side inside one step (the parts of one wider tensor).
		for(uint32_t i = 0; i < group_count; ++i)
		{
			const size_t piece_i = groups[i].bytes;
			const size_t span_i = static_cast<size_t>(entry_count - 1) * output_entry_strides[i] * sizeof(float) + piece_i;
			for(uint32_t j = 0; j < group_count; ++j)
			{
				for(uint32_t k = 0; k < groups[j].input_count; ++k)
					if (ranges_overlap(outputs[i], span_i, groups[j].a.in[k], groups[j].bytes * entry_count))
						return NNF_HIP_EOVERLAP;
				if (j <= i)
					continue;
				const size_t piece_j = groups[j].bytes;
				const size_t span_j = static_cast<size_t>(entry_count - 1) * output_entry_strides[j] * sizeof(float) + piece_j;
				if (!ranges_overlap(outputs[i], span_i, outputs[j], span_j))
					continue;
				if (output_entry_strides[i] != output_entry_strides[j])
					return NNF_HIP_EOVERLAP;
				const uintptr_t pi = reinterpret_cast<uintptr_t>(outputs[i]), pj = reinterpret_cast<uintptr_t>(outputs[j]);
				const size_t step = static_cast<size_t>(output_entry_strides[i]) * sizeof(float);
				const size_t low_piece = (pi < pj) ? piece_i : piece_j, high_piece = (pi < pj) ? piece_j : piece_i;
				const size_t gap = (pi < pj) ? (pj - pi) : (pi - pj);
				if ((gap < low_piece) || (gap + high_piece > step))
					return NNF_HIP_EOVERLAP;
			}
		}
		for(uint32_t first = 0; first < group_count; first += max_strided_batch)
		{
			chain_strided_batch_args b = {};
			b.count = std::min(max_strided_batch, group_count - first);
			b.entry_count = entry_count;
			size_t lds_bytes = 0;
			uint32_t tiles = 0;
			for(uint32_t m = 0; m < b.count; ++m)
			{
				const prepared_group& g = groups[first + m];
				b.group[m] = g.a;
				b.direct_mask |= g.direct ? (1u << m) : 0u;
				b.two_input_mask |= (g.input_count == 2) ? (1u << m) : 0u;
				b.out_entry_stride[m] = output_entry_strides[first + m];
				tiles += g.tiles;
				b.tile_end[m] = tiles;
				lds_bytes = std::max(lds_bytes, g.lds_bytes);
			}
			const dim3 grid(tiles, std::min(entry_count, 65535u)), block(launch_shapes[strided_shape].block);
			const bool all_direct = b.direct_mask == ((1u << b.count) - 1u), one_input = b.two_input_mask == 0;
			if (wide) NNF_LAUNCH((chain_entries_batch_kernel<256, true, true, 4>), grid, block, lds_bytes, stream, b);
			else if (all_direct && one_input) NNF_LAUNCH((chain_entries_batch_kernel<256, true, true>), grid, block, lds_bytes, stream, b);
			else if (all_direct) NNF_LAUNCH((chain_entries_batch_kernel<256, true, false>), grid, block, lds_bytes, stream, b);
			else if (one_input) NNF_LAUNCH((chain_entries_batch_kernel<256, false, true>), grid, block, lds_bytes, stream, b);
			else NNF_LAUNCH((chain_entries_batch_kernel<256, false, false>), grid, block, lds_bytes, stream, b);
			const int rc = launch_status();
			if (rc != NNF_HIP_OK)
				return rc;
		}
		return NNF_HIP_OK;
	}

	int chain_forward_strided(hipStream_t stream, const nnf_hip_chain_desc* desc, float* output, uint32_t output_entry_stride,
		const float* const* inputs, const float* const* chunk_ptrs)
	{
		if (desc == nullptr)
			return NNF_HIP_EINVAL;
		float* outputs[1] = { output };
		const float* const* input_lists[1] = { inputs };
		const float* const* chunk_lists[1] = { chunk_ptrs };
		return chain_forward_strided_batch(stream, 1, desc, outputs, &output_entry_stride, input_lists, chunk_lists);
	}

	int chain_forward_batch(hipStream_t stream, uint32_t group_count, const nnf_hip_chain_desc* descs, float* const* outputs,
		const float* const* const* inputs, const float* const* const* chunk_ptrs)
	{
		if (group_count == 0)
			return NNF_HIP_OK;
		if ((descs == nullptr) || (outputs == nullptr) || (inputs == nullptr))
			return NNF_HIP_EINVAL;
		if (group_count == 1)
			return chain_forward(stream, &descs[0], outputs[0], inputs[0], (chunk_ptrs == nullptr) ? nullptr : chunk_ptrs[0]);

		// everything is checked before anything is launched
		std::vector<prepared_group> groups(group_count);
		for(uint32_t i = 0; i < group_count; ++i)
		{
			const int rc = prepare_group(&descs[i], outputs[i], inputs[i], (chunk_ptrs == nullptr) ? nullptr : chunk_ptrs[i], false, groups[i]);
			if (rc != NNF_HIP_OK)
				return rc;
		}
		// the groups run in no particular order, possibly at the same time: what one writes no other may touch
		for(uint32_t i = 0; i < group_count; ++i)
		{
			if (groups[i].nothing_to_do)
				continue;
			for(uint32_t j = 0; j < group_count; ++j)
			{
				if ((j == i) || groups[j].nothing_to_do)
					continue;
				if (ranges_overlap(groups[i].a.out, groups[i].bytes, groups[j].a.out, groups[j].bytes))
					return NNF_HIP_EOVERLAP;
				for(uint32_t k = 0; k < groups[j].input_count; ++k)
					if (ranges_overlap(groups[i].a.out, groups[i].bytes, groups[j].a.in[k], groups[j].bytes))
						return NNF_HIP_EOVERLAP;
			}
		}

		std::vector<bool> launched(group_count, false);
		for(uint32_t first = 0; first < group_count; ++first)
		{
			if (launched[first])
				continue;
			const prepared_group& lead = groups[first];
			launched[first] = true;
			if (lead.nothing_to_do)
				continue;
			// the groups behind it that can share its kernel instance, max_batch to a launch; the compile-time
			// expf programs are bound by the vector ALU, not by launches: they keep their own kernels
			std::vector<uint32_t> members(1, first);
			bool one_kind = true; // all members share the lead's number of inputs and tile size
			if ((lead.program == 0) && (lead.a.slot_count <= static_cast<uint32_t>(batch_slots)))
				for(uint32_t j = first + 1; (j < group_count) && (members.size() < max_batch); ++j)
				{
					const prepared_group& g = groups[j];
					const bool same_kind = (g.input_count == lead.input_count) && (g.shape == lead.shape);
					if (!launched[j] && !g.nothing_to_do && (g.program == 0) && (same_kind || (mixes(lead) && mixes(g)))
						&& (g.a.slot_count <= static_cast<uint32_t>(batch_slots)))
					{
						members.push_back(j);
						launched[j] = true;
						one_kind = one_kind && same_kind;
					}
				}
			if (members.size() == 1)
			{
				const int rc = launch_group(stream, lead);
				if (rc != NNF_HIP_OK)
					return rc;
				continue;
			}
			chain_batch_args b = {};
			b.count = static_cast<uint32_t>(members.size());
			size_t lds_bytes = 0;
			uint64_t tiles = 0;
			for(size_t m = 0; m < members.size(); ++m)
			{
				const prepared_group& g = groups[members[m]];
				b.group[m] = batch_group_args_of(g.a);
				b.direct_mask |= g.direct ? (1u << m) : 0u;
				b.two_input_mask |= (g.input_count == 2) ? (1u << m) : 0u;
				tiles += g.tiles;
				b.tile_end[m] = static_cast<uint32_t>(tiles);
				lds_bytes = std::max(lds_bytes, g.lds_bytes);
			}
			if (tiles > 0x7FFFFFFFull)
				return NNF_HIP_ETOOBIG;
			const uint32_t all_groups = (1u << b.count) - 1u;
			const int direct_mode = (b.direct_mask == all_groups) ? 1 : ((b.direct_mask == 0) ? 0 : 2);
			const chain_batch_kernel_fn kernel = one_kind ? pick_batch_kernel(lead.input_count, lead.shape, direct_mode) : pick_batch_mixed_kernel(direct_mode);
			NNF_LAUNCH(kernel, dim3(static_cast<uint32_t>(tiles)), dim3(launch_shapes[lead.shape].block), lds_bytes, stream, b);
			const int rc = launch_status();
			if (rc != NNF_HIP_OK)
				return rc;
		}
		return NNF_HIP_OK;
	}
}
