// Maximum / minimum over windows (max subsampling) and over groups of feature maps (maxout).
//
// Both reference testers fold the values of a window in a fixed order with std::max / std::min,
// whose result for equal values (+0.0 and -0.0) and for NaN depends on the argument order, and
// max subsampling starts the fold at -1.0e37F / 1.0e37F. The kernels' results equal the reference's bit
// for bit: the staged 2-D kernels take the hardware's maximum of a window and fold it again in the
// reference's order where only that order decides (a result of zero), the others keep the order, the
// argument order and the start value throughout:
//   nnforge/plain/max_subsampling_layer_tester_plain.cpp:175-290  std::max<float>(current, new), x fastest
//   nnforge/plain/maxout_layer_tester_plain.cpp:56-80             std::max(new, current), starts at the first value
#include "nnf_common.h"
#include "nnf_prologue.h"

#include <algorithm>
#include <cstdlib>
#include <type_traits>

namespace nnf
{
	namespace
	{
		constexpr int max_block_size = 256;
		constexpr uint32_t max_dims = NNF_HIP_MAX_SUBSAMPLING_DIMENSIONS;

		// std::max<float>(current, new_val) / std::min<float>(current, new_val)
		template<bool IS_MIN>
		__device__ __forceinline__ float fold(float current, float new_val)
		{
			if (IS_MIN)
				return (new_val < current) ? new_val : current;
			return (current < new_val) ? new_val : current;
		}

		// What the window kernels do with the values of a window, scanned x fastest:
		// maximum, minimum (both from the -/+1.0e37F start value), or their left-to-right sum times a
		// multiplier (average subsampling, nnforge/plain/average_subsampling_layer_tester_plain.cpp:125-145).
		constexpr int window_op_max = 0;
		constexpr int window_op_min = 1;
		constexpr int window_op_sum = 2;

		template<int OP>
		__device__ __forceinline__ float window_fold(float current, float new_val)
		{
			if (OP == window_op_sum)
				return current + new_val;
			return fold<OP == window_op_min>(current, new_val);
		}

		template<int OP>
		__device__ __forceinline__ float window_fold_start()
		{
			if (OP == window_op_sum)
				return 0.0f;
			return (OP == window_op_min) ? 1.0e37f : -1.0e37f;
		}

		// ---- the hardware's maximum / minimum, with the reference's result ------------------------
		// std::max<float>(current, new) from a finite start value never holds a NaN (current < NaN is false), so a
		// window's result is the largest of the start value and the window's numbers - whatever the order of
		// the fold - with one exception: when that largest value is a zero, the fold keeps the first zero it met,
		// -0.0 or +0.0, while v_max_f32 ranks +0.0 above -0.0. The kernels therefore fold with v_max3_f32 /
		// v_min3_f32 (two values per instruction instead of a compare and a select per value) and a lane whose
		// result is a zero folds its window again the reference's way. v_max_f32 passes over a quiet NaN operand but
		// answers a signalling one with a NaN, which the next fold would then pass over together with everything
		// folded so far: the values are made quiet (canonical) once, on their way into LDS.
		__device__ __forceinline__ float quiet(float v)
		{
			return __builtin_canonicalizef(v);
		}

		__device__ __forceinline__ floatx4 quiet(floatx4 v)
		{
			floatx4 q;
			q.x = quiet(v.x); q.y = quiet(v.y); q.z = quiet(v.z); q.w = quiet(v.w);
			return q;
		}

		template<bool IS_MIN>
		__device__ __forceinline__ float hw_fold(float a, float b)
		{
			float d;
			if (IS_MIN)
				asm("v_min_f32 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b));
			else
				asm("v_max_f32 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b));
			return d;
		}

		template<bool IS_MIN>
		__device__ __forceinline__ float hw_fold3(float a, float b, float c)
		{
			float d;
			if (IS_MIN)
				asm("v_min3_f32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "v"(c));
			else
				asm("v_max3_f32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "v"(c));
			return d;
		}

		// The largest (smallest) of the start value and COUNT quiet values: the window's result, unless it is a zero.
		template<int OP, int COUNT>
		__device__ __forceinline__ float fold_values_hw(const float (&v)[COUNT])
		{
			constexpr bool is_min = (OP == window_op_min);
			float current = window_fold_start<OP>();
			#pragma unroll
			for(int i = 0; i + 1 < COUNT; i += 2)
				current = hw_fold3<is_min>(current, v[i], v[i + 1]);
			if (COUNT % 2 != 0)
				current = hw_fold<is_min>(current, v[COUNT - 1]);
			return current;
		}

		// The reference's fold of COUNT values in the order given.
		template<int OP, int COUNT>
		__device__ __forceinline__ float fold_values_in_order(const float (&v)[COUNT])
		{
			float current = window_fold_start<OP>();
			#pragma unroll
			for(int i = 0; i < COUNT; ++i)
				current = window_fold<OP>(current, v[i]);
			return current;
		}

		// One window: the values in scan order (quiet ones, for maximum and minimum).
		template<int OP, int COUNT>
		__device__ __forceinline__ float fold_values(const float (&v)[COUNT])
		{
			if (OP == window_op_sum)
				return fold_values_in_order<OP>(v);
			float current = fold_values_hw<OP>(v);
			if (current == 0.0f)
				current = fold_values_in_order<OP>(v); // which zero: the first one in scan order
			return current;
		}

		// Two windows behind one test, so that the lanes without a zero jump over one block of code instead of
		// stepping through two short ones.
		template<int OP, int COUNT>
		__device__ __forceinline__ void fold_values_twice(float& first_result, float& second_result, const float (&first)[COUNT], const float (&second)[COUNT])
		{
			if (OP == window_op_sum)
			{
				first_result = fold_values_in_order<OP>(first);
				second_result = fold_values_in_order<OP>(second);
				return;
			}
			first_result = fold_values_hw<OP>(first);
			second_result = fold_values_hw<OP>(second);
			if ((first_result == 0.0f) || (second_result == 0.0f))
			{
				first_result = fold_values_in_order<OP>(first);
				second_result = fold_values_in_order<OP>(second);
			}
		}

		// ---- 2-D windows, staged through LDS ------------------------------------------------------
		//
		// A workgroup produces a contiguous run of outputs: either `rows` output rows of one plane
		// (large planes) or all rows of `planes` consecutive planes (small planes). The input it needs
		// is one contiguous range of memory in both cases; it is copied to LDS with aligned float4
		// loads (each input byte is fetched once per workgroup; only the window_height - stride_y rows
		// shared by neighbouring row bands are fetched twice), then every lane scans its windows in LDS.
		struct window2d_args
		{
			float* out;
			const float* in;
			uint32_t total_in;        // floats in the input tensor
			uint32_t plane_count;     // entries * feature maps
			uint32_t in_w, in_h, out_w, out_h;
			uint32_t win_w, win_h, stride_x, stride_y;
			uint32_t planes;          // planes per workgroup (1 when a plane is split into bands)
			uint32_t rows;            // output rows per workgroup (out_h when planes > 1 or the plane is not split)
			uint32_t bands;           // ceil(out_h / rows)
			uint32_t out_w_magic;     // ceil(2^32 / out_w)
			uint32_t band_magic;      // ceil(2^32 / (rows * out_w)): outputs per plane inside a workgroup
			float mult;               // window_op_sum: the sum is multiplied by it
		};

		constexpr int stage_vectors_per_lane = 8; // float4 loads a lane has in flight while staging

		// WIN_W, WIN_H: window size known at compile time, 0: read it from the arguments.
		// TRUNC: windows may reach beyond the input (round up) and are cut off there (maximum and
		// minimum only: repeating a value would change a sum).
		// PROLOGUE: the staged values go through the layers of pro first, with the weights of the feature
		// map each value belongs to (a float4 may straddle two planes when several planes that are not
		// a multiple of four floats long share a workgroup; the host declines planes of under 4 floats).
		// PAIR: a lane takes two neighbouring outputs of a row at a time (stride_x == 2, WIN_W 2 or 3, rows that are a
		// multiple of four floats long and an even number of outputs per row: the host checks). The four columns
		// both windows start in are one 16-byte LDS read, aligned; with three columns per window the fifth is one more
		// read - two LDS reads per window row and pair instead of six, none of them with lanes two words apart (which
		// puts two lanes on every bank), and the two results leave as one 8-byte store. Each window is still folded
		// in the reference's order (x fastest, then y).
		// BN_RELU: the layers are BatchNorm -> ReLU and nothing else (with UNIFORM; apply_known_group)
		// CHUNKED (with BN_RELU): the layers go over the staged float4s two at a time and skip those no lane holds
		template<int OP, int WIN_W, int WIN_H, bool TRUNC, bool PROLOGUE, bool EXP, bool UNIFORM, bool PAIR = false, bool BN_RELU = false, bool CHUNKED = false>
		__device__ __forceinline__ void window2d_body(const window2d_args& a, const window_prologue& pro)
		{
			static_assert(!PAIR || (((WIN_W == 2) || (WIN_W == 3)) && (WIN_H > 0)), "pairs of outputs: windows 2 or 3 wide, height known");
			extern __shared__ __align__(16) float lds_in[];
			__shared__ uint64_t lds_exp[EXP ? exp_lds_entries : 1];
			__shared__ float lds_coef[PROLOGUE ? prologue_coef_floats : 1];
			exp_context exp_ctx = make_exp_context(lds_exp);

			const uint32_t group = blockIdx.x / a.bands;
			const uint32_t band = blockIdx.x - group * a.bands;
			const uint32_t first_plane = group * a.planes;
			const uint32_t planes_here = min(a.planes, a.plane_count - first_plane);
			const uint32_t first_row = band * a.rows;
			const uint32_t rows_here = min(a.rows, a.out_h - first_row);
			const uint32_t in_plane = a.in_w * a.in_h;
			const uint32_t win_w = (WIN_W > 0) ? WIN_W : a.win_w;
			const uint32_t win_h = (WIN_H > 0) ? WIN_H : a.win_h;

			// input rows [in_row0, in_row1) of planes [first_plane, first_plane + planes_here)
			const uint32_t in_row0 = first_row * a.stride_y;
			uint32_t in_row1 = a.in_h;
			if (planes_here == 1)
				in_row1 = min(a.in_h, (first_row + rows_here - 1) * a.stride_y + win_h);
			const uint32_t g0 = first_plane * in_plane + in_row0 * a.in_w;
			const uint32_t g1 = (first_plane + planes_here - 1) * in_plane + in_row1 * a.in_w;
			const uint32_t g0_aligned = g0 & ~3u;
			const uint32_t shift = g0 - g0_aligned;
			const uint32_t vectors = (g1 - g0_aligned + 3) / 4;
			// all loads of a round are issued before the first one is stored to LDS
			constexpr int STAGE = stage_vectors_per_lane;
			// the weights are requested first and looked at once the first round's tensor loads are out
			prologue_weights weights;
			uniform_weights plane_weights;
			float own_coef[prologue_weighted_max][2];
			constexpr bool uniform = PROLOGUE && UNIFORM; // every workgroup of the launch stages (part of) one plane
			if (PROLOGUE)
			{
				if (uniform)
					plane_weights = load_uniform_weights(first_plane % pro.fm_count, pro);
				else
					weights = load_prologue_weights(first_plane % pro.fm_count, planes_here, pro);
			}
			// A round: COUNT float4s per lane from float4 `base` of the range on, up to float4 `limit`. PARTIAL: the
			// round is the tensor's last float4, which ends inside it.
			bool first_round = true;
			auto stage_round = [&](auto count_tag, auto partial_tag, const uint32_t base, const uint32_t limit)
			{
				constexpr int COUNT = decltype(count_tag)::value;
				constexpr bool PARTIAL = decltype(partial_tag)::value;
				floatx4 t[COUNT];
				#pragma unroll
				for(int k = 0; k < COUNT; ++k)
				{
					const uint32_t i = base + k * max_block_size + threadIdx.x;
					if (!PARTIAL)
					{
						// Lanes past the end load the last float4 once more (and do not stage it): without a branch
						// around every load the loads of a round are issued one behind the other. With the branches
						// the compiler formed a load's address in the registers an earlier load was to arrive in,
						// and every load waited for the ones before it.
						t[k] = load_stream(reinterpret_cast<const floatx4*>(a.in + g0_aligned) + min(i, limit - 1));
					}
					else
					{
						t[k].x = t[k].y = t[k].z = t[k].w = 0.0f;
						if (i < limit)
						{
							const uint32_t g = g0_aligned + i * 4;
							t[k].x = a.in[g];
							t[k].y = (g + 1 < a.total_in) ? a.in[g + 1] : 0.0f;
							t[k].z = (g + 2 < a.total_in) ? a.in[g + 2] : 0.0f;
						}
					}
				}
				if (PROLOGUE && first_round)
				{
					first_round = false;
					if (uniform)
						uniform_coefficients(own_coef, plane_weights, pro);
					else
						stage_prologue_coefficients(lds_coef, weights, planes_here, pro);
					if (EXP)
						stage_exp2_table(lds_exp);
					if (EXP || (!uniform && (pro.weighted_count != 0)))
						__syncthreads();
					if (EXP)
						exp_ctx = exp_context_from_lds(lds_exp);
				}
				static_assert(!BN_RELU || UNIFORM || CHUNKED, "several planes per workgroup: the chunked form knows about float4s between planes");
				if (PROLOGUE && BN_RELU && CHUNKED)
				{
					// Straight code, two float4s at a time, and only those the round holds for some lane (a workgroup
					// with a plane of 3025 floats has three float4s per lane to stage, not the eight of a round). A
					// float4 between two planes: every value picks its own plane's coefficients. Not for the bands of
					// large planes, which fill their rounds: 64 x 64 planes of 112 x 112 42.7 us all eight at once,
					// 43.5 us two at a time.
					constexpr int CHUNK = (COUNT >= 2) ? 2 : 1;
					const bool per_plane = !uniform && (planes_here > 1);
					#pragma unroll
					for(int k0 = 0; k0 < COUNT; k0 += CHUNK)
					{
						if (base + k0 * max_block_size < limit)
						{
							float v[CHUNK][4];
							uint32_t off[CHUNK];
							two_plane_offsets<CHUNK> two;
							#pragma unroll
							for(int k = 0; k < CHUNK; ++k)
							{
								const uint32_t i = base + (k0 + k) * max_block_size + threadIdx.x;
								const bool valid = i < limit;
								v[k][0] = t[k0 + k].x; v[k][1] = t[k0 + k].y; v[k][2] = t[k0 + k].z; v[k][3] = t[k0 + k].w;
								// plane, inside the workgroup's range, of the first float of this float4 (floats in front
								// of the range count as plane 0: they are staged but not read)
								const uint32_t first_pos = max(i * 4, shift) - shift;
								const uint32_t p = (per_plane && valid) ? fast_divide(first_pos, in_plane, pro.in_plane_magic) : 0u;
								off[k] = p * (2 * pro.weighted_count);
								two.off2[k] = min(p + 1, planes_here - 1) * (2 * pro.weighted_count); // behind the last plane: values nobody reads
								two.split[k] = (p + 1) * in_plane + shift - i * 4;                    // >= 4: the whole float4 lies in plane p
							}
							if (UNIFORM)
								apply_known_group<CHUNK, known_group_batch_norm_relu, true>(v, v, off, lds_coef, own_coef, pro, exp_ctx);
							else
								apply_known_group<CHUNK, known_group_batch_norm_relu, false, true>(v, v, off, lds_coef, own_coef, pro, exp_ctx, &two);
							#pragma unroll
							for(int k = 0; k < CHUNK; ++k)
							{
								t[k0 + k].x = v[k][0]; t[k0 + k].y = v[k][1]; t[k0 + k].z = v[k][2]; t[k0 + k].w = v[k][3];
							}
						}
					}
				}
				else if (PROLOGUE)
				{
					float v[COUNT][4];
					uint32_t off[COUNT];
					// Planes that are not a multiple of four floats long: a float4 may straddle two of them (never
					// three: the host declines planes of under 4 floats). Bit k: vector k does.
					// which plane a value belongs to matters only to layers with weights, and only with several planes here
					const bool per_plane = !uniform && (planes_here > 1) && (pro.weighted_count != 0);
					const bool straddle = per_plane && ((in_plane & 3u) != 0);
					uint32_t straddling = 0;
					#pragma unroll
					for(int k = 0; k < COUNT; ++k)
					{
						const uint32_t i = base + k * max_block_size + threadIdx.x;
						const bool valid = i < limit;
						// lanes past the end put the values they hold through the layers with the others (whole float4s: the
						// last float4 once more; the partial one: zeros) and store nothing
						v[k][0] = t[k].x; v[k][1] = t[k].y; v[k][2] = t[k].z; v[k][3] = t[k].w;
						// plane, inside the workgroup's range, of the first float of this float4 (floats in front
						// of the range count as plane 0: they are staged but not read)
						const uint32_t first_pos = max(i * 4, shift) - shift;
						const uint32_t p = (per_plane && valid) ? fast_divide(first_pos, in_plane, pro.in_plane_magic) : 0u;
						off[k] = p * (2 * pro.weighted_count);
						// floats from staged position (p + 1) * in_plane + shift on belong to plane p + 1; beyond
						// the last plane of the workgroup they are not read
						if (straddle && valid && (p + 1 < planes_here) && (i * 4 + 3 >= (p + 1) * in_plane + shift))
							straddling |= 1u << k;
					}
					if (BN_RELU)
						apply_known_group<COUNT, known_group_batch_norm_relu, true>(v, v, off, lds_coef, own_coef, pro, exp_ctx);
					else if (uniform)
						apply_prologue<COUNT, EXP, true>(v, off, lds_coef, own_coef, pro, exp_ctx, 0, pro.op_count);
					else
						apply_prologue<COUNT, EXP, false>(v, off, lds_coef, own_coef, pro, exp_ctx, 0, pro.op_count);
					// The floats of the second plane of a straddling float4 were given the first plane's
					// coefficients: they are fetched again and go through the layers with their own.
					while (__any(straddling != 0))
					{
						const int k_mine = (straddling != 0) ? __ffs(straddling) - 1 : 0;
						const bool mine = straddling != 0;
						const uint32_t i = base + k_mine * max_block_size + threadIdx.x;
						const uint32_t first_pos = max(i * 4, shift) - shift;
						const uint32_t p_next = mine ? fast_divide(first_pos, in_plane, pro.in_plane_magic) + 1 : 0u;
						const uint32_t split = mine ? p_next * in_plane + shift - i * 4 : 4u; // 1..3: first float of plane p_next
						float w[1][4];
						#pragma unroll
						for(uint32_t e = 0; e < 4; ++e)
						{
							const uint32_t g = g0_aligned + i * 4 + e;
							w[0][e] = (mine && (e >= split) && (g < a.total_in)) ? a.in[g] : 0.0f;
						}
						const uint32_t off_next[1] = { p_next * (2 * pro.weighted_count) };
						apply_prologue<1, EXP, false>(w, off_next, lds_coef, own_coef, pro, exp_ctx, 0, pro.op_count);
						#pragma unroll
						for(int k = 0; k < COUNT; ++k)
						{
							#pragma unroll
							for(uint32_t e = 1; e < 4; ++e)
							{
								if (mine && (k == k_mine) && (e >= split))
									v[k][e] = w[0][e];
							}
						}
						straddling &= straddling - 1;
					}
					#pragma unroll
					for(int k = 0; k < COUNT; ++k)
					{
						t[k].x = v[k][0]; t[k].y = v[k][1]; t[k].z = v[k][2]; t[k].w = v[k][3];
					}
				}
				#pragma unroll
				for(int k = 0; k < COUNT; ++k)
				{
					const uint32_t i = base + k * max_block_size + threadIdx.x;
					if (i < limit)
						*reinterpret_cast<floatx4*>(lds_in + i * 4) = (OP == window_op_sum) ? t[k] : quiet(t[k]);
				}
			};
			// whole float4s first; only the tensor's last float4 can be partial (in the launch's last workgroup) and gets a
			// round of its own, so that the rounds all others take carry no such case
			const uint32_t whole_vectors = min(vectors, (a.total_in - g0_aligned) / 4);
			for(uint32_t base = 0; base < whole_vectors; base += STAGE * max_block_size)
				stage_round(std::integral_constant<int, STAGE>(), std::false_type(), base, whole_vectors);
			if (whole_vectors < vectors)
				stage_round(std::integral_constant<int, 1>(), std::true_type(), whole_vectors, vectors);
			__syncthreads();

			// A lane's unit of work: one output, or (PAIR) two neighbouring outputs of a row
			const uint32_t units_w = PAIR ? (a.out_w >> 1) : a.out_w;
			const uint32_t unit_stride_x = PAIR ? 2 * a.stride_x : a.stride_x;
			const uint32_t outputs_per_plane = rows_here * units_w;
			const uint32_t outputs_here = planes_here * outputs_per_plane;
			float* dst = a.out + (first_plane * a.out_h + first_row) * a.out_w;

			// A lane takes units tid, tid + 256, ... of the workgroup's run. Where its window starts - column
			// x0 and row y0 of the plane, float index win of the staged copy - is worked out once with
			// divisions and then carried from one unit to the next with additions: 256 units further is
			// step_p planes, step_y rows and step_x columns further, with a carry from columns into rows
			// and from rows into planes (integer multiplications run at a quarter of the rate of additions
			// here, and the scan, not the memory, was what bounded this kernel).
			const uint32_t step_p = max_block_size / outputs_per_plane;
			const uint32_t step_rest = max_block_size - step_p * outputs_per_plane;
			const uint32_t step_y = step_rest / units_w;
			const uint32_t step_x = step_rest - step_y * units_w;
			const uint32_t row_floats = a.stride_y * a.in_w;        // one output row further
			const uint32_t x_limit = units_w * unit_stride_x;       // x0 of the column behind the last one
			const uint32_t y_limit = (first_row + rows_here) * a.stride_y;
			const uint32_t x_advance = step_x * unit_stride_x;
			const uint32_t y_advance = step_y * a.stride_y;
			const uint32_t win_advance = step_p * in_plane + step_y * row_floats + x_advance;
			const uint32_t x_carry_win = row_floats - x_limit;                 // back to column 0, one row down
			const uint32_t y_carry_y = rows_here * a.stride_y;
			const uint32_t y_carry_win = in_plane - rows_here * row_floats;    // back to row 0, one plane on

			uint32_t x0, y0, win;
			{
				// rows_here differs from a.rows only in the last band, where planes_here == 1 and p is 0 anyway
				const uint32_t o = threadIdx.x;
				uint32_t p, oy;
				if (PAIR)
				{
					p = (planes_here > 1) ? o / outputs_per_plane : 0u;
					oy = (o - p * outputs_per_plane) / units_w;
				}
				else
				{
					p = (planes_here > 1) ? fast_divide(o, outputs_per_plane, a.band_magic) : 0u;
					oy = fast_divide(o - p * outputs_per_plane, a.out_w, a.out_w_magic);
				}
				const uint32_t ox = o - p * outputs_per_plane - oy * units_w;
				x0 = ox * unit_stride_x;
				y0 = (first_row + oy) * a.stride_y;
				win = shift + p * in_plane + (y0 - in_row0) * a.in_w + x0;
			}
			for(uint32_t o = threadIdx.x; o < outputs_here; o += max_block_size)
			{
				const float* src = lds_in + win;
				// A window position beyond the input reads the last position inside instead. That value
				// has been folded before (it precedes in scan order) and folding a value twice changes
				// nothing, so this equals skipping the position.
				const uint32_t last_x = TRUNC ? min(win_w, a.in_w - x0) - 1 : 0u;
				const uint32_t last_y = TRUNC ? min(win_h, a.in_h - y0) - 1 : 0u;
				static_assert(!(TRUNC && (OP == window_op_sum)), "a truncated window re-reads values");
				if (PAIR)
				{
					// columns x0 .. x0 + 3 lie inside the row (its length is a multiple of four, as is x0); the second
					// window's third column, x0 + 4, may not
					uint32_t row_offset[WIN_H > 0 ? WIN_H : 1];
					row_offset[0] = 0;
					#pragma unroll
					for(int y = 1; y < WIN_H; ++y)
						row_offset[y] = TRUNC ? row_offset[y - 1] + ((static_cast<uint32_t>(y) <= last_y) ? a.in_w : 0u) : static_cast<uint32_t>(y) * a.in_w;
					const bool fifth_inside = !TRUNC || (x0 + 4 < a.in_w);
					constexpr int count = ((WIN_W > 0) && (WIN_H > 0)) ? WIN_W * WIN_H : 1;
					float first[count], second[count];
					#pragma unroll
					for(int y = 0; y < WIN_H; ++y)
					{
						const float* row = src + row_offset[y];
						const floatx4 v = *reinterpret_cast<const floatx4*>(row);
						if (WIN_W == 2)
						{
							first[y * WIN_W] = v.x; first[y * WIN_W + 1] = v.y;
							second[y * WIN_W] = v.z; second[y * WIN_W + 1] = v.w;
						}
						else
						{
							const float fifth = fifth_inside ? row[4] : v.w;
							first[y * WIN_W] = v.x; first[y * WIN_W + 1] = v.y; first[y * WIN_W + 2] = v.z;
							second[y * WIN_W] = v.z; second[y * WIN_W + 1] = v.w; second[y * WIN_W + 2] = fifth;
						}
					}
					float2 both;
					fold_values_twice<OP>(both.x, both.y, first, second);
					if (OP == window_op_sum)
					{
						both.x *= a.mult;
						both.y *= a.mult;
					}
					*reinterpret_cast<float2*>(dst + 2 * o) = both;
				}
				else
				{
				float current;
				if ((WIN_W > 0) && (WIN_H > 0))
				{
					// min(y, last_y) * in_w and min(x, last_x) without multiplications
					uint32_t row_offset[WIN_H > 0 ? WIN_H : 1], column_offset[WIN_W > 0 ? WIN_W : 1];
					row_offset[0] = 0;
					#pragma unroll
					for(int y = 1; y < WIN_H; ++y)
						row_offset[y] = TRUNC ? row_offset[y - 1] + ((static_cast<uint32_t>(y) <= last_y) ? a.in_w : 0u) : static_cast<uint32_t>(y) * a.in_w;
					#pragma unroll
					for(int x = 0; x < WIN_W; ++x)
						column_offset[x] = TRUNC ? min(static_cast<uint32_t>(x), last_x) : static_cast<uint32_t>(x);
					constexpr int count = ((WIN_W > 0) && (WIN_H > 0)) ? WIN_W * WIN_H : 1;
					float values[count];
					#pragma unroll
					for(int y = 0; y < WIN_H; ++y)
					{
						const float* row = src + row_offset[y];
						#pragma unroll
						for(int x = 0; x < WIN_W; ++x)
							values[y * WIN_W + x] = row[column_offset[x]];
					}
					current = fold_values<OP>(values);
				}
				else
				{
					const uint32_t fit_w = TRUNC ? last_x + 1 : win_w;
					const uint32_t fit_h = TRUNC ? last_y + 1 : win_h;
					current = window_fold_start<OP>();
					const float* row = src;
					if (OP == window_op_sum)
					{
						for(uint32_t y = 0; y < fit_h; ++y, row += a.in_w)
							for(uint32_t x = 0; x < fit_w; ++x)
								current += row[x];
					}
					else
					{
						constexpr bool is_min = (OP == window_op_min);
						for(uint32_t y = 0; y < fit_h; ++y, row += a.in_w)
							for(uint32_t x = 0; x < fit_w; ++x)
								current = hw_fold<is_min>(current, row[x]);
						if (current == 0.0f)
						{
							// which zero: the first one in scan order, as the reference's fold keeps it
							current = window_fold_start<OP>();
							row = src;
							for(uint32_t y = 0; y < fit_h; ++y, row += a.in_w)
								for(uint32_t x = 0; x < fit_w; ++x)
									current = fold<is_min>(current, row[x]);
						}
					}
				}
				dst[o] = (OP == window_op_sum) ? current * a.mult : current;
				}

				// 256 units further
				x0 += x_advance;
				y0 += y_advance;
				win += win_advance;
				if (x0 >= x_limit)
				{
					x0 -= x_limit;
					y0 += a.stride_y;
					win += x_carry_win;
				}
				if (y0 >= y_limit)
				{
					y0 -= y_carry_y;
					win += y_carry_win;
				}
			}
		}

		template<int OP, int WIN_W, int WIN_H, bool TRUNC, bool PAIR = false>
		__global__ void __launch_bounds__(max_block_size) max_window2d_kernel(const window2d_args a)
		{
			window_prologue none; // not read
			window2d_body<OP, WIN_W, WIN_H, TRUNC, false, false, false, PAIR>(a, none);
		}

		// UNIFORM: one plane per workgroup (a.planes == 1). Without expf the layers fit 80 registers per lane,
		// which lets a compute unit hold six workgroups instead of four where their LDS allows it (the two bands of a
		// 112 x 112 plane are 25.6 KB each; BatchNorm + ReLU + 3x3/2 pooling of 64 x 64 such planes: 54 us at four,
		// 46-47 us at five, 43.7 us at six); with expf that would spill, and so would the kernels for several planes per
		// workgroup, which stay at five.
		template<int OP, int WIN_W, int WIN_H, bool TRUNC, bool UNIFORM, bool PAIR = false>
		__global__ void __launch_bounds__(max_block_size) __attribute__((amdgpu_waves_per_eu(UNIFORM ? 6 : 5, UNIFORM ? 6 : 5))) max_window2d_prologue_kernel(const window2d_args a, const window_prologue pro)
		{
			window2d_body<OP, WIN_W, WIN_H, TRUNC, true, false, UNIFORM, PAIR>(a, pro);
		}

		// BatchNorm -> ReLU in front of the windows: the layers as straight code (several planes per workgroup: 77 to 80
		// registers instead of 96; 64 x 256 planes of 27 x 27 20.9 -> 16.6 us, 64 x 128 of 28 x 28 10.2 -> 9.4 us)
		// FILLED: one plane (or band) per workgroup that holds more than four float4s per lane
		template<int OP, int WIN_W, int WIN_H, bool TRUNC, bool PAIR = false, bool UNIFORM = true, bool FILLED = true>
		__global__ void __launch_bounds__(max_block_size) __attribute__((amdgpu_waves_per_eu(UNIFORM ? 6 : 4))) max_window2d_bn_relu_kernel(const window2d_args a, const window_prologue pro)
		{
			static_assert(UNIFORM || !FILLED, "several planes per workgroup go two float4s at a time");
			window2d_body<OP, WIN_W, WIN_H, TRUNC, true, false, UNIFORM, PAIR, true, !FILLED>(a, pro);
		}

		template<int OP, int WIN_W, int WIN_H, bool TRUNC, bool UNIFORM>
		__global__ void __launch_bounds__(max_block_size) max_window2d_exp_prologue_kernel(const window2d_args a, const window_prologue pro)
		{
			window2d_body<OP, WIN_W, WIN_H, TRUNC, true, true, UNIFORM>(a, pro);
		}

		// ---- any window the layer allows: one lane per output, values read from memory ------------
		struct window_nd_args
		{
			float* out;
			const float* in;
			uint32_t output_count;
			uint32_t in_size[max_dims], out_size[max_dims], window[max_dims], stride[max_dims]; // unused dimensions are 1
			uint32_t in_fm, out_fm, fm_window, entry_window, in_plane;
			float mult; // window_op_sum: the sum is multiplied by it
			uint32_t tile_count; // TILING: output entries per input entry, the product of the window sizes
		};

		// TILING: output entry e * tile_count + j holds the windows of input entry e whose grid is shifted by j,
		// taken apart x fastest like the window scan (nnforge/plain/max_subsampling_layer_tester_plain.cpp:78-170)
		template<int OP, bool TILING = false>
		__global__ void __launch_bounds__(max_block_size) window_nd_kernel(const window_nd_args a)
		{
			const uint32_t o = blockIdx.x * max_block_size + threadIdx.x;
			if (o >= a.output_count)
				return;
			uint32_t rem = o;
			uint32_t start[max_dims], fit[max_dims];
			#pragma unroll
			for(uint32_t d = 0; d < max_dims; ++d)
			{
				const uint32_t q = rem / a.out_size[d];
				start[d] = (rem - q * a.out_size[d]) * a.stride[d];
				fit[d] = min(a.window[d], a.in_size[d] - start[d]);
				rem = q;
			}
			const uint32_t out_entry = rem / a.out_fm;
			const uint32_t out_fm_id = rem - out_entry * a.out_fm;
			size_t base;
			if (TILING)
			{
				const uint32_t in_entry = out_entry / a.tile_count;
				uint32_t shift = out_entry - in_entry * a.tile_count;
				#pragma unroll
				for(uint32_t d = 0; d < max_dims; ++d)
				{
					const uint32_t q = shift / a.window[d];
					start[d] += shift - q * a.window[d];
					fit[d] = a.window[d]; // the output sizes leave room for every shift
					shift = q;
				}
				base = (static_cast<size_t>(in_entry) * a.in_fm + out_fm_id) * a.in_plane;
			}
			else
				base = (static_cast<size_t>(out_entry) * a.entry_window * a.in_fm + static_cast<size_t>(out_fm_id) * a.fm_window) * a.in_plane;

			float current = window_fold_start<OP>();
			// scan order of the reference: x fastest, then y, z, w, feature map, entry
			for(uint32_t en = 0; en < a.entry_window; ++en)
			{
				for(uint32_t fm = 0; fm < a.fm_window; ++fm)
				{
					const float* plane = a.in + base + (static_cast<size_t>(en) * a.in_fm + fm) * a.in_plane;
					for(uint32_t w = 0; w < fit[3]; ++w)
					{
						for(uint32_t z = 0; z < fit[2]; ++z)
						{
							for(uint32_t y = 0; y < fit[1]; ++y)
							{
								const float* row = plane + ((static_cast<size_t>(start[3] + w) * a.in_size[2] + start[2] + z) * a.in_size[1] + start[1] + y) * a.in_size[0] + start[0];
								for(uint32_t x = 0; x < fit[0]; ++x)
									current = window_fold<OP>(current, row[x]);
							}
						}
					}
				}
			}
			a.out[o] = (OP == window_op_sum) ? current * a.mult : current;
		}

		// ---- tiling in 1 or 2 dimensions, staged through LDS ---------------------------------------
		// A workgroup stages whole planes (small ones, several) or the input rows of a band of output rows, once, and
		// every lane then takes output positions of that range: at a position it folds the window of each of the
		// win_w * win_h shifted grids out of LDS. The input is read from memory once (twice where bands overlap)
		// instead of once per grid. A band's results are contiguous in every grid's output plane: they are collected
		// in LDS, one run per grid, and leave as aligned float4s (a wavefront's 64 single floats at an odd address,
		// which is what a position per lane gives, cost the write path more than the staging costs: the planes of
		// 55 x 55 outputs that 112 x 112 inputs give start on any 4-byte boundary). Several small planes per
		// workgroup are stored from the lanes directly.
		struct tiling2d_args
		{
			float* out;
			const float* in;
			uint32_t total_in;              // floats in the input tensor
			uint32_t in_w, in_h, out_w, out_h, win_w, win_h;
			uint32_t fm_count, plane_count; // planes = entries * feature maps
			uint32_t planes;                // whole planes per workgroup; 1: bands of `rows` output rows, `bands` per plane
			uint32_t rows, bands;
			uint32_t runs;                  // results leave as one run per grid (bands, or planes of one entry); 0: stored from the scan
			uint32_t in_area;               // runs: LDS floats in front of the grids' output runs
			uint32_t out_pitch;             // runs: LDS floats from one grid's run to the next (a multiple of 4)
			uint32_t together;              // runs: consecutive work items that go to workgroups of one XCD (xcd_grouped)
		};

		// What a workgroup stages: planes [first_plane, first_plane + planes_here), output rows [oy0, oy1) of them
		struct tiling_range
		{
			uint32_t first_plane, planes_here, oy0, oy1;
			uint32_t g0_aligned;   // first float of the aligned float4s around the staged input
			uint32_t shift;        // floats of the first float4 in front of the range
			uint32_t vectors;      // float4s to stage
		};

		__device__ __forceinline__ tiling_range tiling_range_of(const tiling2d_args& a, uint32_t work_id, uint32_t win_h)
		{
			tiling_range r;
			const uint32_t in_plane = a.in_w * a.in_h;
			if (a.planes > 1)
			{
				r.first_plane = work_id * a.planes;
				r.planes_here = min(a.planes, a.plane_count - r.first_plane);
				r.oy0 = 0;
				r.oy1 = a.out_h;
			}
			else
			{
				r.first_plane = work_id / a.bands;
				r.planes_here = 1;
				r.oy0 = (work_id - r.first_plane * a.bands) * a.rows;
				r.oy1 = min(r.oy0 + a.rows, a.out_h);
			}
			// input rows oy0 * win_h .. oy1 * win_h + win_h - 2 of every plane: the last grid's last window ends there
			// (out_h * win_h + win_h - 1 <= in_h by the layer's output size); several planes are staged whole
			const uint32_t first_row = r.oy0 * win_h;
			const uint32_t staged_floats = (a.planes > 1) ? r.planes_here * in_plane : (r.oy1 * win_h + win_h - 1 - first_row) * a.in_w;
			const uint32_t g0 = r.first_plane * in_plane + first_row * a.in_w;
			r.g0_aligned = g0 & ~3u;
			r.shift = g0 - r.g0_aligned;
			r.vectors = (staged_floats + r.shift + 3) / 4;
			return r;
		}

		// The staged input is in LDS (behind a barrier): every lane folds its positions. Bands put their results
		// into the grids' runs in LDS, several planes store them.
		template<int OP, int WIN_W, int WIN_H, int BLOCK>
		__device__ __forceinline__ void tiling_scan(const tiling2d_args& a, const tiling_range& r, float* staged_area)
		{
			const uint32_t win_w = (WIN_W > 0) ? WIN_W : a.win_w, win_h = (WIN_H > 0) ? WIN_H : a.win_h;
			const uint32_t in_plane = a.in_w * a.in_h, out_plane = a.out_w * a.out_h;
			const bool band = a.runs != 0; // positions of the workgroup lie in every grid's output one after the other
			const uint32_t first_plane = r.first_plane, planes_here = r.planes_here;
			const float* staged = staged_area + r.shift;
			const uint32_t rows_here = r.oy1 - r.oy0;
			const uint32_t positions_per_plane = rows_here * a.out_w;
			const uint32_t positions = planes_here * positions_per_plane;
			const uint32_t tiles = win_w * win_h;
			const uint32_t grid_stride = a.fm_count * out_plane; // from one output entry to the next (tensors are indexed with 32 bits)
			// A lane takes positions tid, tid + BLOCK, ...: plane, row and column of the first one by division, the following
			// ones by addition with carries (BLOCK positions further is step_p planes, step_y rows and step_x columns further)
			// instead of divisions and multiplications per position; the same for where its windows start in LDS.
			const uint32_t step_p = BLOCK / positions_per_plane;
			const uint32_t step_rest = BLOCK - step_p * positions_per_plane;
			const uint32_t step_y = step_rest / a.out_w;
			const uint32_t step_x = step_rest - step_y * a.out_w;
			const uint32_t row_floats = win_h * a.in_w;                        // one output row further
			const uint32_t corner_advance = step_p * in_plane + step_y * row_floats + step_x * win_w;
			const uint32_t x_carry_corner = row_floats - a.out_w * win_w;      // back to column 0, one row down
			const uint32_t y_carry_corner = in_plane - rows_here * row_floats; // back to row 0, one plane on
			uint32_t p = (planes_here > 1) ? threadIdx.x / positions_per_plane : 0u;
			uint32_t oy = (threadIdx.x - p * positions_per_plane) / a.out_w;
			uint32_t ox = threadIdx.x - p * positions_per_plane - oy * a.out_w;
			uint32_t corner_offset = p * in_plane + oy * row_floats + ox * win_w;
			// a band: one plane for the whole workgroup, and its positions lie in the output plane one after the other.
			// Grid g's run starts at band_out_index + g * grid_stride; in LDS it is kept at the same offset from a 16-byte
			// boundary as in memory, so that an aligned float4 of the one is an aligned float4 of the other.
			const uint32_t band_entry = first_plane / a.fm_count;
			const uint32_t band_fm = first_plane - band_entry * a.fm_count;
			const uint32_t band_out_index = (band_entry * tiles * a.fm_count + band_fm) * out_plane + r.oy0 * a.out_w;
			float* const runs = staged_area + a.in_area;
			// With the window size known a lane works on several positions at a time: the LDS reads of all of them are
			// out before the first is folded.
			constexpr bool sized = (WIN_W > 0) && (WIN_H > 0);
			constexpr int batch = !sized ? 1 : ((WIN_W * WIN_H <= 4) ? 4 : 2);
			constexpr bool is_min = (OP == window_op_min);
			for(uint32_t pos = threadIdx.x; pos < positions; pos += BLOCK * batch)
			{
				uint32_t out_index[batch], corner_of[batch];
				bool valid[batch];
				#pragma unroll
				for(int b = 0; b < batch; ++b)
				{
					valid[b] = pos + b * BLOCK < positions;
					out_index[b] = pos + b * BLOCK; // bands: inside the run
					if (!band)
					{
						const uint32_t plane_id = first_plane + p;
						const uint32_t entry = plane_id / a.fm_count;
						const uint32_t fm = plane_id - entry * a.fm_count;
						out_index[b] = (entry * tiles * a.fm_count + fm) * out_plane + oy * a.out_w + ox;
					}
					corner_of[b] = valid[b] ? corner_offset : 0u;
					// BLOCK positions further
					ox += step_x;
					oy += step_y;
					p += step_p;
					corner_offset += corner_advance;
					if (ox >= a.out_w)
					{
						ox -= a.out_w;
						++oy;
						corner_offset += x_carry_corner;
					}
					if (oy >= rows_here)
					{
						oy -= rows_here;
						++p;
						corner_offset += y_carry_corner;
					}
				}
				// grids in the order of the window scan: x shift fastest
				if (sized)
				{
					// the (2 * height - 1) x (2 * width - 1) values the grids' windows at a position cover
					constexpr int span_w = sized ? 2 * WIN_W - 1 : 1, span_h = sized ? 2 * WIN_H - 1 : 1;
					constexpr int grids = sized ? WIN_W * WIN_H : 1;
					float near[batch][span_h][span_w];
					#pragma unroll
					for(int b = 0; b < batch; ++b)
					{
						const float* corner = staged + corner_of[b];
						#pragma unroll
						for(int y = 0; y < span_h; ++y)
						{
							#pragma unroll
							for(int x = 0; x < span_w; ++x)
								near[b][y][x] = corner[y * a.in_w + x];
						}
					}
					#pragma unroll
					for(int b = 0; b < batch; ++b)
					{
						float values[grids][grids], result[grids];
						bool any_zero = false;
						#pragma unroll
						for(int g = 0; g < grids; ++g)
						{
							#pragma unroll
							for(int y = 0; y < WIN_H; ++y)
							{
								#pragma unroll
								for(int x = 0; x < WIN_W; ++x)
									values[g][y * WIN_W + x] = near[b][g / WIN_W + y][g % WIN_W + x];
							}
							result[g] = fold_values_hw<OP>(values[g]);
							any_zero = any_zero || (result[g] == 0.0f);
						}
						// which zero: the first one in scan order, as the reference's fold keeps it
						if (any_zero)
						{
							#pragma unroll
							for(int g = 0; g < grids; ++g)
								result[g] = fold_values_in_order<OP>(values[g]);
						}
						if (valid[b])
						{
							#pragma unroll
							for(int g = 0; g < grids; ++g)
							{
								if (band)
									runs[g * a.out_pitch + ((band_out_index + g * grid_stride) & 3u) + out_index[b]] = result[g];
								else
									a.out[out_index[b] + g * grid_stride] = result[g];
							}
						}
					}
				}
				else if (valid[0])
				{
					const float* corner = staged + corner_of[0];
					uint32_t g = 0;
					for(uint32_t sy = 0; sy < win_h; ++sy)
					{
						for(uint32_t sx = 0; sx < win_w; ++sx, ++g)
						{
							float current = window_fold_start<OP>();
							for(uint32_t y = 0; y < win_h; ++y)
								for(uint32_t x = 0; x < win_w; ++x)
									current = hw_fold<is_min>(current, corner[(sy + y) * a.in_w + sx + x]);
							if (current == 0.0f)
							{
								current = window_fold_start<OP>();
								for(uint32_t y = 0; y < win_h; ++y)
									for(uint32_t x = 0; x < win_w; ++x)
										current = fold<is_min>(current, corner[(sy + y) * a.in_w + sx + x]);
							}
							if (band)
								runs[g * a.out_pitch + ((band_out_index + g * grid_stride) & 3u) + out_index[0]] = current;
							else
								a.out[out_index[0] + g * grid_stride] = current;
						}
					}
				}
			}
		}

		// The same for 2 x 2 windows over a band whose rows are a multiple of four floats wide (so that every staged row starts
		// on a 16-byte boundary of LDS): a lane takes a strip of four columns of one output row - the two positions whose
		// windows start in those columns - and reads the three input rows under it as an aligned float4 and the float behind it
		// each: six conflict-free LDS reads for eight results, where a position per lane costs six reads for four results with
		// the lanes two words apart. The largest of two neighbouring rows per column is shared by the windows that hold the
		// column (the hardware's maximum of quiet values does not depend on the order); a strip that holds a zero result is
		// folded again window by window in the reference's order.
		template<int OP, int BLOCK>
		__device__ __forceinline__ void tiling_scan_strips(const tiling2d_args& a, const tiling_range& r, float* staged_area)
		{
			constexpr bool is_min = (OP == window_op_min);
			const uint32_t strips = a.in_w / 4;
			const uint32_t rows_here = r.oy1 - r.oy0;
			const uint32_t tasks = rows_here * strips;
			const uint32_t strips_magic = (strips > 1) ? 0xFFFFFFFFu / strips + 1 : 0u; // ceil(2^32 / strips): exact quotients while task * strips < 2^32
			const uint32_t out_plane = a.out_w * a.out_h;
			const uint32_t grid_stride = a.fm_count * out_plane;
			const uint32_t band_entry = r.first_plane / a.fm_count;
			const uint32_t band_fm = r.first_plane - band_entry * a.fm_count;
			const uint32_t band_out_index = (band_entry * 4 * a.fm_count + band_fm) * out_plane + r.oy0 * a.out_w;
			float* const runs = staged_area + a.in_area;
			const float start = window_fold_start<OP>();
			for(uint32_t task = threadIdx.x; task < tasks; task += BLOCK)
			{
				const uint32_t row = (strips > 1) ? __umulhi(task, strips_magic) : task;
				const uint32_t strip = task - row * strips;
				const float* corner = staged_area + row * 2 * a.in_w + strip * 4;
				float rows3[3][5];
				#pragma unroll
				for(int y = 0; y < 3; ++y)
				{
					const floatx4 four = *reinterpret_cast<const floatx4*>(corner + y * a.in_w);
					rows3[y][0] = four.x; rows3[y][1] = four.y; rows3[y][2] = four.z; rows3[y][3] = four.w;
					rows3[y][4] = corner[y * a.in_w + 4]; // the last strip of a row: the next row's first float, or what lies behind the band; not used then
				}
				// result[grid][position]: grid = 2 * (shift down) + (shift right), as the window scan numbers the shifts
				float result[4][2];
				bool any_zero = false;
				#pragma unroll
				for(int down = 0; down < 2; ++down)
				{
					float column[5];
					#pragma unroll
					for(int c = 0; c < 5; ++c)
						column[c] = hw_fold<is_min>(rows3[down][c], rows3[down + 1][c]);
					#pragma unroll
					for(int right = 0; right < 2; ++right)
					{
						#pragma unroll
						for(int position = 0; position < 2; ++position)
						{
							const float largest = hw_fold3<is_min>(start, column[2 * position + right], column[2 * position + right + 1]);
							result[2 * down + right][position] = largest;
							any_zero = any_zero || (largest == 0.0f);
						}
					}
				}
				if (any_zero)
				{
					#pragma unroll
					for(int down = 0; down < 2; ++down)
					{
						#pragma unroll
						for(int right = 0; right < 2; ++right)
						{
							#pragma unroll
							for(int position = 0; position < 2; ++position)
							{
								const int c = 2 * position + right;
								const float in_scan_order[4] = { rows3[down][c], rows3[down][c + 1], rows3[down + 1][c], rows3[down + 1][c + 1] };
								result[2 * down + right][position] = fold_values_in_order<OP>(in_scan_order);
							}
						}
					}
				}
				const uint32_t ox = strip * 2;
				const bool first = ox < a.out_w, second = ox + 1 < a.out_w; // rows of 4m floats have 2m - 1 positions: the last strip holds one
				const uint32_t in_run = row * a.out_w + ox;
				#pragma unroll
				for(uint32_t g = 0; g < 4; ++g)
				{
					float* to = runs + g * a.out_pitch + ((band_out_index + g * grid_stride) & 3u) + in_run;
					if (first)
						to[0] = result[g][0];
					if (second)
						to[1] = result[g][1];
				}
			}
		}

		// A band's runs are in LDS (behind a barrier) and leave: aligned float4s, and single floats where a run starts
		// or ends inside one.
		template<int BLOCK>
		__device__ __forceinline__ void tiling_write_runs(const tiling2d_args& a, const tiling_range& r, const float* staged_area, uint32_t tiles)
		{
			const uint32_t out_plane = a.out_w * a.out_h;
			const uint32_t grid_stride = a.fm_count * out_plane;
			const uint32_t band_entry = r.first_plane / a.fm_count;
			const uint32_t band_fm = r.first_plane - band_entry * a.fm_count;
			const uint32_t band_out_index = (band_entry * tiles * a.fm_count + band_fm) * out_plane + r.oy0 * a.out_w;
			const uint32_t positions = r.planes_here * (r.oy1 - r.oy0) * a.out_w;
			const float* runs = staged_area + a.in_area;
			for(uint32_t g = 0; g < tiles; ++g)
			{
				const uint32_t run_index = band_out_index + g * grid_stride;   // first float of the run in the output tensor
				const uint32_t lead = run_index & 3u;                          // floats of the first float4 in front of it
				const float* from = runs + g * a.out_pitch;                    // from[lead + i]: float i of the run
				float* to = a.out + (run_index - lead);                        // 16-byte aligned: the tensor's base is
				const uint32_t end = lead + positions;
				for(uint32_t k = threadIdx.x * 4; k < end; k += BLOCK * 4)
				{
					const floatx4 v = *reinterpret_cast<const floatx4*>(from + k);
					if ((k >= lead) && (k + 4 <= end))
						store_stream(reinterpret_cast<floatx4*>(to + k), v);
					else
					{
						if ((k >= lead) && (k < end)) to[k] = v.x;
						if ((k + 1 >= lead) && (k + 1 < end)) to[k + 1] = v.y;
						if ((k + 2 >= lead) && (k + 2 < end)) to[k + 2] = v.z;
						if ((k + 3 >= lead) && (k + 3 < end)) to[k + 3] = v.w;
					}
				}
			}
		}

		// STRIPS: 2 x 2 windows over bands of rows that are a multiple of four floats wide (tiling_scan_strips)
		template<int OP, int WIN_W, int WIN_H, int BLOCK, bool STRIPS = false>
		__global__ void __launch_bounds__(BLOCK) tiling2d_kernel(const tiling2d_args a)
		{
			extern __shared__ __attribute__((aligned(16))) float staged_area[];
			const uint32_t win_w = (WIN_W > 0) ? WIN_W : a.win_w, win_h = (WIN_H > 0) ? WIN_H : a.win_h;
			const uint32_t work_id = a.runs ? xcd_grouped(blockIdx.x, a.together, gridDim.x) : blockIdx.x;
			const tiling_range r = tiling_range_of(a, work_id, win_h);
			// Eight loads in flight per lane before the first LDS store. A band of the usual size is two or three float4s per
			// lane; with sixteen the kernel holds 73 registers per lane and 64 x 64 planes of 112 x 112 with 2 x 2 windows
			// take 78-80 us instead of 73.5.
			constexpr uint32_t in_flight = 8;
			floatx4* staged4 = reinterpret_cast<floatx4*>(staged_area);
			// only the tensor's last float4 can be partial (in the launch's last workgroup): it is staged by one lane, float by float
			const uint32_t whole_vectors = min(r.vectors, (a.total_in - r.g0_aligned) / 4);
			for(uint32_t base = 0; base < whole_vectors; base += BLOCK * in_flight)
			{
				// A stripe of BLOCK float4s is skipped as a whole when it lies past the end (the same for all lanes), and inside
				// the last stripe the lanes past the end load the last float4 once more: no lane-dependent branch around a load,
				// so the loads are issued one behind the other. Rows shared by two bands are wanted twice: no streaming hint.
				floatx4 t[in_flight];
				#pragma unroll
				for(uint32_t k = 0; k < in_flight; ++k)
					if (base + k * BLOCK < whole_vectors)
						t[k] = reinterpret_cast<const floatx4*>(a.in + r.g0_aligned)[min(base + k * BLOCK + threadIdx.x, whole_vectors - 1)];
				#pragma unroll
				for(uint32_t k = 0; k < in_flight; ++k)
					if (base + k * BLOCK + threadIdx.x < whole_vectors)
						staged4[base + k * BLOCK + threadIdx.x] = quiet(t[k]);
			}
			if ((whole_vectors < r.vectors) && (threadIdx.x == 0))
			{
				for(uint32_t g = r.g0_aligned + whole_vectors * 4; g < a.total_in; ++g)
					staged_area[g - r.g0_aligned] = quiet(a.in[g]);
			}
			__syncthreads();
			if (STRIPS)
				tiling_scan_strips<OP, BLOCK>(a, r, staged_area);
			else
				tiling_scan<OP, WIN_W, WIN_H, BLOCK>(a, r, staged_area);
			if (!a.runs)
				return;
			__syncthreads();
			tiling_write_runs<BLOCK>(a, r, staged_area, win_w * win_h);
		}

		// -> true when the staged kernel took the work
		bool launch_tiling2d(hipStream_t stream, bool is_min, float* output, const float* input, uint32_t total_in, uint32_t plane_count, uint32_t fm_count,
			uint32_t in_w, uint32_t in_h, uint32_t out_w, uint32_t out_h, uint32_t win_w, uint32_t win_h)
		{
			constexpr uint32_t lds_floats_max = 15 * 1024;  // what a workgroup may use
			constexpr uint32_t lds_floats_band = 6 * 1024;  // what a band and its output runs should stay under: six workgroups or more to a compute unit
			tiling2d_args a = {};
			a.out = output;
			a.in = input;
			a.total_in = total_in;
			a.in_w = in_w; a.in_h = in_h; a.out_w = out_w; a.out_h = out_h; a.win_w = win_w; a.win_h = win_h;
			a.fm_count = fm_count;
			a.plane_count = plane_count;
			const uint64_t in_plane = static_cast<uint64_t>(in_w) * in_h;
			const uint32_t tiles = win_w * win_h;
			// a band of `rows` output rows: (rows * win_h + win_h - 1) input rows (+ 3 floats in front of an unaligned start),
			// and a run of rows * out_w floats (+ up to 3 in front, rounded up to float4s) per grid
			auto band_floats = [&](uint32_t rows, uint32_t& in_area, uint32_t& out_pitch) -> uint64_t
			{
				const uint64_t in_floats = static_cast<uint64_t>(rows * win_h + win_h - 1) * in_w + 3;
				in_area = static_cast<uint32_t>((in_floats + 3) & ~static_cast<uint64_t>(3));
				out_pitch = (rows * out_w + 3 + 3) & ~3u;
				return static_cast<uint64_t>(in_area) + static_cast<uint64_t>(tiles) * out_pitch;
			};
			uint32_t in_area_one, out_pitch_one;
			if (band_floats(1, in_area_one, out_pitch_one) > lds_floats_max)
				return false;
			uint32_t grid;
			size_t lds_floats;
			a.planes = 1;
			a.runs = 1;
			const uint32_t out_plane = out_w * out_h;
			// several whole planes of one entry: their input (+ 3 floats in front of an unaligned start) and a run of their outputs per grid
			auto planes_floats = [&](uint32_t planes, uint32_t& in_area, uint32_t& out_pitch) -> uint64_t
			{
				in_area = static_cast<uint32_t>((planes * in_plane + 3 + 3) & ~static_cast<uint64_t>(3));
				out_pitch = (planes * out_plane + 3 + 3) & ~3u;
				return static_cast<uint64_t>(in_area) + static_cast<uint64_t>(tiles) * out_pitch;
			};
			// planes of any entries with results stored from the scan: what remains when runs would leave the lanes with too little
			uint32_t planes_without_runs = 1;
			if (in_plane * 2 + 3 <= lds_floats_max)
			{
				const uint32_t wanted = (4 * max_block_size + out_plane - 1) / out_plane;
				planes_without_runs = max(1u, min(min(wanted, static_cast<uint32_t>((lds_floats_max - 3) / in_plane)), plane_count));
			}
			constexpr uint32_t positions_worth_runs = 2 * max_block_size;
			if (planes_floats(1, a.in_area, a.out_pitch) <= lds_floats_band)
			{
				// Planes that fit the budget whole: as many of one entry (so that their outputs are one run in every grid: a
				// divisor of the number of feature maps) as stay within it, until the lanes have four positions each.
				uint32_t in_area, out_pitch;
				for(uint32_t planes = 2; (planes <= fm_count) && ((planes - 1) * out_plane < 4 * max_block_size); ++planes)
				{
					if ((fm_count % planes == 0) && (planes_floats(planes, in_area, out_pitch) <= lds_floats_band))
						a.planes = planes;
				}
				a.rows = out_h;
				a.bands = 1;
				a.together = 4; // neighbouring workgroups' runs meet in cache lines, as the bands of a plane do
			}
			else
			{
				// the highest band within the budget (any band that fits, if none does)
				uint32_t rows = out_h;
				while ((rows > 1) && (band_floats(rows, a.in_area, a.out_pitch) > lds_floats_band))
					rows = (band_floats(rows, a.in_area, a.out_pitch) > 2 * static_cast<uint64_t>(lds_floats_band)) ? (rows + 1) / 2 : rows - 1;
				a.bands = (out_h + rows - 1) / rows;
				// few planes: more, lower bands (not below 4 output rows) until about 1024 workgroups share the work
				const uint32_t bands_wanted = (1024 + plane_count - 1) / plane_count;
				a.bands = max(a.bands, min(bands_wanted, max(1u, out_h / 4)));
				a.rows = (out_h + a.bands - 1) / a.bands; // bands of equal height
				a.bands = (out_h + a.rows - 1) / a.rows;
				a.together = a.bands;
			}
			if ((a.planes * a.rows * out_w < positions_worth_runs) && (planes_without_runs > 1))
			{
				a.planes = planes_without_runs;
				a.runs = 0;
				a.rows = out_h;
				a.bands = 1;
				grid = (plane_count + a.planes - 1) / a.planes;
				lds_floats = a.planes * static_cast<size_t>(in_plane) + 8;
			}
			else if (a.bands == 1)
			{
				grid = (plane_count + a.planes - 1) / a.planes;
				lds_floats = planes_floats(a.planes, a.in_area, a.out_pitch);
			}
			else
			{
				grid = plane_count * a.bands;
				lds_floats = band_floats(a.rows, a.in_area, a.out_pitch);
			}
			const bool strips = a.runs && (a.planes == 1) && (win_w == 2) && (win_h == 2) && (in_w % 4 == 0);
			const size_t lds_bytes = lds_floats * sizeof(float);
			constexpr int block = max_block_size;
			const bool w2 = (win_w == 2) && (win_h == 2), w3 = (win_w == 3) && (win_h == 3);
			const dim3 g(grid), b(block);
			if (is_min)
			{
				if (strips) NNF_LAUNCH((tiling2d_kernel<window_op_min, 2, 2, block, true>), g, b, lds_bytes, stream, a);
				else if (w2) NNF_LAUNCH((tiling2d_kernel<window_op_min, 2, 2, block>), g, b, lds_bytes, stream, a);
				else if (w3) NNF_LAUNCH((tiling2d_kernel<window_op_min, 3, 3, block>), g, b, lds_bytes, stream, a);
				else NNF_LAUNCH((tiling2d_kernel<window_op_min, 0, 0, block>), g, b, lds_bytes, stream, a);
			}
			else
			{
				if (strips) NNF_LAUNCH((tiling2d_kernel<window_op_max, 2, 2, block, true>), g, b, lds_bytes, stream, a);
				else if (w2) NNF_LAUNCH((tiling2d_kernel<window_op_max, 2, 2, block>), g, b, lds_bytes, stream, a);
				else if (w3) NNF_LAUNCH((tiling2d_kernel<window_op_max, 3, 3, block>), g, b, lds_bytes, stream, a);
				else NNF_LAUNCH((tiling2d_kernel<window_op_max, 0, 0, block>), g, b, lds_bytes, stream, a);
			}
			return true;
		}

		// ---- windows over feature maps and entries only: whole rows folded with float4 ------------
		// Spatial windows of 1: output row r (a plane, or a whole entry when there is no window over feature maps)
		// is the fold of the input rows (entry e * entry_window + en, row fo * fm_window + fm), feature maps inside
		// entries as in the reference's scan. Rows are multiples of 4 floats; a lane folds one float4 of a row.
		struct window_rows_args
		{
			float* out;
			const float* in;
			uint32_t row_vectors;      // float4s per row
			uint32_t out_rows;         // output entries * rows_per_out_entry
			uint32_t rows_per_out_entry, rows_per_in_entry;
			uint32_t fm_window, entry_window;
			float mult;
		};

		template<int OP>
		__global__ void __launch_bounds__(max_block_size) window_rows_kernel(const window_rows_args a)
		{
			const uint32_t j = blockIdx.x * max_block_size + threadIdx.x;
			if (j >= a.row_vectors)
				return;
			for(uint32_t r = blockIdx.y; r < a.out_rows; r += gridDim.y)
			{
				const uint32_t entry = r / a.rows_per_out_entry;
				const uint32_t row = r - entry * a.rows_per_out_entry;
				const floatx4* src = reinterpret_cast<const floatx4*>(a.in)
					+ (static_cast<size_t>(entry) * a.entry_window * a.rows_per_in_entry + static_cast<size_t>(row) * a.fm_window) * a.row_vectors + j;
				const float start = window_fold_start<OP>();
				floatx4 current = { start, start, start, start };
				for(uint32_t en = 0; en < a.entry_window; ++en)
				{
					for(uint32_t fm = 0; fm < a.fm_window; ++fm)
					{
						const floatx4 v = load_stream(src + (static_cast<size_t>(en) * a.rows_per_in_entry + fm) * a.row_vectors);
						current.x = window_fold<OP>(current.x, v.x);
						current.y = window_fold<OP>(current.y, v.y);
						current.z = window_fold<OP>(current.z, v.z);
						current.w = window_fold<OP>(current.w, v.w);
					}
				}
				if (OP == window_op_sum)
				{
					current.x *= a.mult;
					current.y *= a.mult;
					current.z *= a.mult;
					current.w *= a.mult;
				}
				store_stream(reinterpret_cast<floatx4*>(a.out) + static_cast<size_t>(r) * a.row_vectors + j, current);
			}
		}

		// rows shorter than this leave most lanes of a workgroup idle: the one-lane-per-output kernel does better
		constexpr uint32_t window_rows_min_vectors = 64;

		// -> true when the rows kernel took the work
		bool launch_window_rows(hipStream_t stream, int op, float mult, float* output, const float* input, uint32_t output_entry_count,
			uint32_t in_fm, uint32_t out_fm, uint64_t plane, uint32_t fm_window, uint32_t entry_window)
		{
			window_rows_args a = {};
			const uint64_t row_floats = (fm_window == 1) ? static_cast<uint64_t>(in_fm) * plane : plane;
			if ((row_floats % 4 != 0) || (row_floats / 4 < window_rows_min_vectors))
				return false;
			a.out = output;
			a.in = input;
			a.row_vectors = static_cast<uint32_t>(row_floats / 4);
			a.rows_per_out_entry = (fm_window == 1) ? 1 : out_fm;
			a.rows_per_in_entry = (fm_window == 1) ? 1 : in_fm;
			a.out_rows = output_entry_count * a.rows_per_out_entry;
			a.fm_window = fm_window;
			a.entry_window = entry_window;
			a.mult = mult;
			const dim3 grid((a.row_vectors + max_block_size - 1) / max_block_size, min(a.out_rows, 65535u));
			if (op == window_op_sum)
				NNF_LAUNCH(window_rows_kernel<window_op_sum>, grid, dim3(max_block_size), 0, stream, a);
			else if (op == window_op_min)
				NNF_LAUNCH(window_rows_kernel<window_op_min>, grid, dim3(max_block_size), 0, stream, a);
			else
				NNF_LAUNCH(window_rows_kernel<window_op_max>, grid, dim3(max_block_size), 0, stream, a);
			return true;
		}

		// ---- maxout ------------------------------------------------------------------------------
		// Per entry the output is `group` floats and output j folds the inputs j, j + group, j + 2*group, ...
		// std::max(new_val, current) = (new_val < current) ? current : new_val
		__device__ __forceinline__ float maxout_fold(float current, float new_val)
		{
			return (new_val < current) ? current : new_val;
		}

		// group is a multiple of 4, two feature maps folded into one: a lane folds four float4s of outputs, all eight loads
		// out before the first fold; 4 KB of an entry's outputs per wavefront instruction. hold_ticks: read_phase_ticks.
		constexpr int maxout_pair_unroll = 4;
		__global__ void __launch_bounds__(max_block_size) maxout_pairs_kernel(float* out, const float* in, uint32_t entry_count, uint32_t group, uint32_t hold_ticks)
		{
			const uint64_t started = (hold_ticks != 0) ? wall_clock64() : 0;
			const uint32_t first = blockIdx.x * (max_block_size * maxout_pair_unroll) + threadIdx.x; // in float4s of an entry's outputs
			const uint32_t vectors = group / 4;
			for(uint32_t entry = blockIdx.y; entry < entry_count; entry += gridDim.y)
			{
				const floatx4* src = reinterpret_cast<const floatx4*>(in + static_cast<size_t>(entry) * group * 2);
				floatx4 a[maxout_pair_unroll], b[maxout_pair_unroll];
				#pragma unroll
				for(int k = 0; k < maxout_pair_unroll; ++k)
				{
					const uint32_t j = min(first + k * max_block_size, vectors - 1); // past the end: the last one again, stored by nobody
					a[k] = load_stream(src + j);
					b[k] = load_stream(src + vectors + j);
				}
				#pragma unroll
				for(int k = 0; k < maxout_pair_unroll; ++k)
				{
					a[k].x = maxout_fold(a[k].x, b[k].x);
					a[k].y = maxout_fold(a[k].y, b[k].y);
					a[k].z = maxout_fold(a[k].z, b[k].z);
					a[k].w = maxout_fold(a[k].w, b[k].w);
				}
				if ((hold_ticks != 0) && (entry == blockIdx.y))
				{
					#pragma unroll
					for(int k = 0; k < maxout_pair_unroll; ++k)
						asm volatile("" : "+v"(a[k]));
					hold_until(started, hold_ticks);
				}
				#pragma unroll
				for(int k = 0; k < maxout_pair_unroll; ++k)
				{
					const uint32_t j = first + k * max_block_size;
					if (j < vectors)
						store_stream(reinterpret_cast<floatx4*>(out + static_cast<size_t>(entry) * group) + j, a[k]);
				}
			}
		}

		// group is a multiple of 4: a lane folds four neighbouring outputs
		__global__ void __launch_bounds__(max_block_size) maxout_vec4_kernel(float* out, const float* in, uint32_t entry_count, uint32_t group, uint32_t fold_count)
		{
			const uint32_t j = (blockIdx.x * max_block_size + threadIdx.x) * 4;
			if (j >= group)
				return;
			for(uint32_t entry = blockIdx.y; entry < entry_count; entry += gridDim.y)
			{
				const float* src = in + static_cast<size_t>(entry) * group * fold_count + j;
				floatx4 current = load_stream(reinterpret_cast<const floatx4*>(src));
				for(uint32_t i = 1; i < fold_count; ++i)
				{
					const floatx4 new_val = load_stream(reinterpret_cast<const floatx4*>(src + static_cast<size_t>(i) * group));
					current.x = maxout_fold(current.x, new_val.x);
					current.y = maxout_fold(current.y, new_val.y);
					current.z = maxout_fold(current.z, new_val.z);
					current.w = maxout_fold(current.w, new_val.w);
				}
				store_stream(reinterpret_cast<floatx4*>(out + static_cast<size_t>(entry) * group + j), current);
			}
		}

		__global__ void __launch_bounds__(max_block_size) maxout_scalar_kernel(float* out, const float* in, uint32_t entry_count, uint32_t group, uint32_t fold_count)
		{
			const uint32_t j = blockIdx.x * max_block_size + threadIdx.x;
			if (j >= group)
				return;
			for(uint32_t entry = blockIdx.y; entry < entry_count; entry += gridDim.y)
			{
				const float* src = in + static_cast<size_t>(entry) * group * fold_count + j;
				float current = src[0];
				for(uint32_t i = 1; i < fold_count; ++i)
					current = maxout_fold(current, src[static_cast<size_t>(i) * group]);
				out[static_cast<size_t>(entry) * group + j] = current;
			}
		}

		bool overlap(const void* a, uint64_t a_bytes, const void* b, uint64_t b_bytes)
		{
			const uintptr_t pa = reinterpret_cast<uintptr_t>(a), pb = reinterpret_cast<uintptr_t>(b);
			return (pa < pb + b_bytes) && (pb < pa + a_bytes);
		}

		// Shapes the kernels take two outputs per lane at a time for (window2d_body's PAIR): every staged row starts on
		// a 16-byte boundary of LDS and holds whole float4s, and a row's outputs pair up.
		bool pairs_of_outputs(const window2d_args& a)
		{
			return (a.stride_x == 2) && ((a.in_w % 4) == 0) && ((a.out_w % 2) == 0) && (a.out_w >= 2);
		}

		template<int OP, bool TRUNC, bool UNIFORM>
		void launch_window2d_prologue(hipStream_t stream, const window2d_args& a, uint32_t grid, size_t lds_bytes, const window_prologue& pro)
		{
			const dim3 g(grid), b(max_block_size);
			const bool w3 = (a.win_w == 3) && (a.win_h == 3), w2 = (a.win_w == 2) && (a.win_h == 2);
			if (pro.need_exp)
			{
				if (w3) NNF_LAUNCH((max_window2d_exp_prologue_kernel<OP, 3, 3, TRUNC, UNIFORM>), g, b, lds_bytes, stream, a, pro);
				else if (w2) NNF_LAUNCH((max_window2d_exp_prologue_kernel<OP, 2, 2, TRUNC, UNIFORM>), g, b, lds_bytes, stream, a, pro);
				else NNF_LAUNCH((max_window2d_exp_prologue_kernel<OP, 0, 0, TRUNC, UNIFORM>), g, b, lds_bytes, stream, a, pro);
			}
			else if (known_group_of(pro) == known_group_batch_norm_relu)
			{
				const bool pair = pairs_of_outputs(a);
				// the floats a workgroup stages, as lds_bytes counts them
				const bool filled = UNIFORM && (lds_bytes / sizeof(float) > 4u * 4u * max_block_size);
				if (filled)
				{
					if (w3 && pair) NNF_LAUNCH((max_window2d_bn_relu_kernel<OP, 3, 3, TRUNC, true>), g, b, lds_bytes, stream, a, pro);
					else if (w2 && pair) NNF_LAUNCH((max_window2d_bn_relu_kernel<OP, 2, 2, TRUNC, true>), g, b, lds_bytes, stream, a, pro);
					else if (w3) NNF_LAUNCH((max_window2d_bn_relu_kernel<OP, 3, 3, TRUNC>), g, b, lds_bytes, stream, a, pro);
					else if (w2) NNF_LAUNCH((max_window2d_bn_relu_kernel<OP, 2, 2, TRUNC>), g, b, lds_bytes, stream, a, pro);
					else NNF_LAUNCH((max_window2d_bn_relu_kernel<OP, 0, 0, TRUNC>), g, b, lds_bytes, stream, a, pro);
				}
				else if (w3 && pair) NNF_LAUNCH((max_window2d_bn_relu_kernel<OP, 3, 3, TRUNC, true, UNIFORM, false>), g, b, lds_bytes, stream, a, pro);
				else if (w2 && pair) NNF_LAUNCH((max_window2d_bn_relu_kernel<OP, 2, 2, TRUNC, true, UNIFORM, false>), g, b, lds_bytes, stream, a, pro);
				else if (w3) NNF_LAUNCH((max_window2d_bn_relu_kernel<OP, 3, 3, TRUNC, false, UNIFORM, false>), g, b, lds_bytes, stream, a, pro);
				else if (w2) NNF_LAUNCH((max_window2d_bn_relu_kernel<OP, 2, 2, TRUNC, false, UNIFORM, false>), g, b, lds_bytes, stream, a, pro);
				else NNF_LAUNCH((max_window2d_bn_relu_kernel<OP, 0, 0, TRUNC, false, UNIFORM, false>), g, b, lds_bytes, stream, a, pro);
			}
			else
			{
				const bool pair = pairs_of_outputs(a);
				if (w3 && pair) NNF_LAUNCH((max_window2d_prologue_kernel<OP, 3, 3, TRUNC, UNIFORM, true>), g, b, lds_bytes, stream, a, pro);
				else if (w2 && pair) NNF_LAUNCH((max_window2d_prologue_kernel<OP, 2, 2, TRUNC, UNIFORM, true>), g, b, lds_bytes, stream, a, pro);
				else if (w3) NNF_LAUNCH((max_window2d_prologue_kernel<OP, 3, 3, TRUNC, UNIFORM>), g, b, lds_bytes, stream, a, pro);
				else if (w2) NNF_LAUNCH((max_window2d_prologue_kernel<OP, 2, 2, TRUNC, UNIFORM>), g, b, lds_bytes, stream, a, pro);
				else NNF_LAUNCH((max_window2d_prologue_kernel<OP, 0, 0, TRUNC, UNIFORM>), g, b, lds_bytes, stream, a, pro);
			}
		}

		template<int OP, bool TRUNC>
		void launch_window2d(hipStream_t stream, const window2d_args& a, uint32_t grid, size_t lds_bytes, const window_prologue* pro)
		{
			if (pro != nullptr)
			{
				if (a.planes == 1)
					launch_window2d_prologue<OP, TRUNC, true>(stream, a, grid, lds_bytes, *pro);
				else
					launch_window2d_prologue<OP, TRUNC, false>(stream, a, grid, lds_bytes, *pro);
				return;
			}
			const bool pair = pairs_of_outputs(a);
			if ((a.win_w == 3) && (a.win_h == 3) && pair)
				NNF_LAUNCH((max_window2d_kernel<OP, 3, 3, TRUNC, true>), dim3(grid), dim3(max_block_size), lds_bytes, stream, a);
			else if ((a.win_w == 2) && (a.win_h == 2) && pair)
				NNF_LAUNCH((max_window2d_kernel<OP, 2, 2, TRUNC, true>), dim3(grid), dim3(max_block_size), lds_bytes, stream, a);
			else if ((a.win_w == 3) && (a.win_h == 3))
				NNF_LAUNCH((max_window2d_kernel<OP, 3, 3, TRUNC>), dim3(grid), dim3(max_block_size), lds_bytes, stream, a);
			else if ((a.win_w == 2) && (a.win_h == 2))
				NNF_LAUNCH((max_window2d_kernel<OP, 2, 2, TRUNC>), dim3(grid), dim3(max_block_size), lds_bytes, stream, a);
			else
				NNF_LAUNCH((max_window2d_kernel<OP, 0, 0, TRUNC>), dim3(grid), dim3(max_block_size), lds_bytes, stream, a);
		}

		// LDS floats a workgroup of the 2-D kernel stages (measured best of 2048 ... 12288 on the ResNet stem's pooling)
		constexpr uint32_t staging_floats = 8u * 1024u;
	}

	// Plans and launches the LDS-staged 2-D window kernel. op: 0 maximum, 1 minimum, 2 maximum with
	// windows cut off at the input edge (round up), 3 minimum likewise, 4 sum times mult. Returns
	// false (nothing launched) when the shape does not suit the kernel: more than 65535 outputs per
	// plane, or a single band of window_height input rows that does not fit LDS.
	bool window2d_launch(hipStream_t stream, int op, float mult, float* output, const float* input, uint32_t input_total, uint32_t plane_count,
		uint32_t in_w, uint32_t in_h, uint32_t out_w, uint32_t out_h, uint32_t win_w, uint32_t win_h, uint32_t stride_x, uint32_t stride_y)
	{
		return window2d_launch_with_prologue(stream, op, mult, output, input, input_total, plane_count, in_w, in_h, out_w, out_h,
			win_w, win_h, stride_x, stride_y, nullptr, nullptr, 0, false);
	}

	// NNF_HIP_OK when desc describes layers a subsampling kernel can apply to its input: one input, no
	// Add (with allow_join also: two inputs joined by an Add), 1..NNF_HIP_MAX_OPS known layers, every weight
	// pointer they name present (NNF_HIP_EINVAL otherwise), at most two of them with weights (NNF_HIP_EUNSUPPORTED).
	int prologue_status(const nnf_hip_chain_desc& desc, const float* const* chunk_ptrs, bool allow_join)
	{
		window_prologue pro = {};
		if (!fill_prologue(pro, desc, chunk_ptrs, std::max(1u, desc.feature_map_count), std::max(1u, desc.neuron_count_per_feature_map), allow_join))
			return NNF_HIP_EINVAL;
		return (pro.weighted_count > prologue_weighted_max) ? NNF_HIP_EUNSUPPORTED : NNF_HIP_OK;
	}

	// As window2d_launch; with prologue != null the layers of that single-input group are applied to the
	// input on its way into LDS (feature_map_count: feature maps of the input). plan_only: nothing is
	// launched, the return value tells whether this shape would run (with the prologue, if one is given).
	bool window2d_launch_with_prologue(hipStream_t stream, int op, float mult, float* output, const float* input, uint32_t input_total, uint32_t plane_count,
		uint32_t in_w, uint32_t in_h, uint32_t out_w, uint32_t out_h, uint32_t win_w, uint32_t win_h, uint32_t stride_x, uint32_t stride_y,
		const nnf_hip_chain_desc* prologue, const float* const* chunk_ptrs, uint32_t feature_map_count, bool plan_only)
	{
		const uint32_t lds_floats_wanted = staging_floats;
		constexpr uint32_t lds_floats_max = 15 * 1024;
		if (static_cast<uint64_t>(out_w) * out_h >= (1u << 16))
			return false;
		window2d_args a = {};
		a.out = output;
		a.in = input;
		a.total_in = input_total;
		a.plane_count = plane_count;
		a.in_w = in_w; a.in_h = in_h;
		a.out_w = out_w; a.out_h = out_h;
		a.win_w = win_w; a.win_h = win_h;
		a.stride_x = stride_x; a.stride_y = stride_y;
		a.mult = mult;
		const uint32_t plane = a.in_w * a.in_h;
		bool fits = true;
		if (plane <= lds_floats_wanted)
		{
			// whole planes; enough of them for a few outputs per lane, few enough to keep the grid wide
			a.planes = std::max(1u, std::min(lds_floats_wanted / plane, (4u * max_block_size + a.out_w * a.out_h - 1) / (a.out_w * a.out_h)));
			a.rows = a.out_h;
		}
		else
		{
			a.planes = 1;
			// rows per band: input rows needed = (rows - 1) * stride_y + win_h
			const uint32_t rows_in = lds_floats_wanted / a.in_w;
			a.rows = (rows_in >= a.win_h) ? (rows_in - a.win_h) / a.stride_y + 1 : 0;
			if (a.rows == 0)
			{
				a.rows = 1;
				fits = static_cast<uint64_t>(a.win_h) * a.in_w + 4 <= lds_floats_max;
			}
			a.rows = std::min(a.rows, a.out_h);
			// bands of equal height
			const uint32_t bands = (a.out_h + a.rows - 1) / a.rows;
			a.rows = (a.out_h + bands - 1) / bands;
		}
		if (!fits)
			return false;
		window_prologue pro = {};
		if (prologue != nullptr)
		{
			// a float4 of a workgroup's range may straddle two planes, not three
			if ((a.planes > 1) && (plane < 4))
				return false;
			if (!plan_only && (!fill_prologue(pro, *prologue, chunk_ptrs, feature_map_count, plane) || (pro.weighted_count > prologue_weighted_max)))
				return false;
			// the planes of a workgroup keep their coefficients in LDS
			a.planes = std::min(a.planes, std::min(prologue_planes_max, prologue_coef_floats / (2 * prologue_weighted_max)));
			// Layers with weights over planes this large: one plane per workgroup, whose coefficients come through the scalar
			// cache into registers - no table in LDS, no barrier in front of the layers, no float4 between two planes
			// (BatchNorm -> ReLU -> 3 x 3 every 2 on 64 x 96 planes of 55 x 55: 21.6 -> 19.8 us, of 51 x 51 19.5 -> 18.6 us,
			// 2 x 2 on 56 x 56 14.9 -> 13.4 us; equal on 45 x 45 and 48 x 48; 64 x 128 planes of 40 x 40 the other way,
			// 15.4 -> 18.2 us, 35 x 35 18.9 -> 24.1 us).
			if ((a.planes > 1) && (pro.weighted_count != 0) && (plane >= 2500u))
				a.planes = 1;
			// Layers that call expf are what such a launch waits for, and a workgroup takes every round of eight float4s per
			// lane through them whole: as many small planes as fill the rounds, not as few as give every lane four outputs
			// (TanH -> Absolute -> average over 2 x 2 on 1024 x 38 planes of 28 x 28: six planes, 4.6 float4s per lane,
			// 63.2 us; ten planes, 7.7 per lane, 46.6 us; 1024 x 96 planes of 10 x 10 26.9 -> 19.2 us).
			if (pro.need_exp && (plane <= lds_floats_wanted))
				a.planes = std::max(1u, std::min(lds_floats_wanted / plane, std::min(prologue_planes_max, prologue_coef_floats / (2 * prologue_weighted_max))));
		}
		if (plan_only)
			return true;
		a.bands = (a.out_h + a.rows - 1) / a.rows;
		a.out_w_magic = magic_of(a.out_w);
		a.band_magic = magic_of(a.rows * a.out_w);
		const uint32_t rows_in = (a.planes > 1 || a.bands == 1) ? a.in_h : std::min(a.in_h, (a.rows - 1) * a.stride_y + a.win_h);
		const size_t lds_bytes = (static_cast<size_t>(a.planes - 1) * plane + static_cast<size_t>(rows_in) * a.in_w + 8) * sizeof(float);
		const uint32_t grid = ((a.plane_count + a.planes - 1) / a.planes) * a.bands;
		const window_prologue* use = (prologue != nullptr) ? &pro : nullptr;
		switch (op)
		{
		case 0: launch_window2d<window_op_max, false>(stream, a, grid, lds_bytes, use); break;
		case 1: launch_window2d<window_op_min, false>(stream, a, grid, lds_bytes, use); break;
		case 2: launch_window2d<window_op_max, true>(stream, a, grid, lds_bytes, use); break;
		case 3: launch_window2d<window_op_min, true>(stream, a, grid, lds_bytes, use); break;
		default: launch_window2d<window_op_sum, false>(stream, a, grid, lds_bytes, use); break;
		}
		return true;
	}

	// prologue != null: the layers of that group are applied to the input first (LDS-staged kernel only:
	// NNF_HIP_EUNSUPPORTED for shapes it does not take). plan_only: nothing is launched and no pointer is
	// looked at; NNF_HIP_OK means the call would run.
	int max_subsampling_forward_with_prologue(hipStream_t stream, float* output, const float* input,
		uint32_t output_entry_count, uint32_t input_feature_map_count, uint32_t dimension_count,
		const uint32_t* input_sizes, const uint32_t* subsampling_sizes, const uint32_t* strides, const uint32_t* round_ups,
		uint32_t feature_map_subsampling_size, uint32_t entry_subsampling_size, int32_t is_min,
		const nnf_hip_chain_desc* prologue, const float* const* chunk_ptrs, bool plan_only)
	{
		if (plan_only)
		{
			// planning looks at shapes only: stand-ins that pass the pointer checks below, never dereferenced
			output = reinterpret_cast<float*>(static_cast<uintptr_t>(16));
			input = reinterpret_cast<const float*>(static_cast<uintptr_t>(1) << 46);
		}
		if ((output == nullptr) || (input == nullptr) || (input_sizes == nullptr) || (subsampling_sizes == nullptr))
			return NNF_HIP_EINVAL;
		if ((dimension_count < 1) || (dimension_count > max_dims))
			return NNF_HIP_EUNSUPPORTED; // the reference's testers stop at 4 dimensions as well
		if ((input_feature_map_count == 0) || (feature_map_subsampling_size == 0) || (entry_subsampling_size == 0))
			return NNF_HIP_EINVAL;
		if (!is_aligned16(output) || !is_aligned16(input))
			return NNF_HIP_EALIGN;

		window_nd_args nd = {};
		uint64_t in_plane = 1, out_plane = 1;
		bool round_up_anywhere = false;
		bool identity_in_plane = true; // windows of one element at every position
		for(uint32_t d = 0; d < max_dims; ++d)
		{
			nd.in_size[d] = nd.out_size[d] = nd.window[d] = nd.stride[d] = 1;
			if (d >= dimension_count)
				continue;
			const uint32_t size = input_sizes[d], window = subsampling_sizes[d];
			const uint32_t stride = (strides != nullptr) ? strides[d] : window;
			identity_in_plane = identity_in_plane && (window == 1) && (stride == 1);
			const bool round_up = (round_ups != nullptr) && (round_ups[d] != 0);
			if ((size == 0) || (window == 0) || (stride == 0))
				return NNF_HIP_EINVAL;
			// nnforge/max_subsampling_layer.cpp:135-139
			const int64_t out_size = (static_cast<int64_t>(size) + stride - window + (round_up ? window - 1 : 0)) / stride;
			if (out_size <= 0)
				return NNF_HIP_EINVAL; // "produces 0 output size"
			nd.in_size[d] = size;
			nd.out_size[d] = static_cast<uint32_t>(out_size);
			nd.window[d] = window;
			nd.stride[d] = stride;
			in_plane *= size;
			out_plane *= static_cast<uint64_t>(out_size);
			round_up_anywhere = round_up_anywhere || round_up;
		}
		const uint32_t out_fm = input_feature_map_count / feature_map_subsampling_size;
		if (out_fm == 0)
			return NNF_HIP_EINVAL;
		const uint64_t input_total = static_cast<uint64_t>(output_entry_count) * entry_subsampling_size * input_feature_map_count * in_plane;
		const uint64_t output_total = static_cast<uint64_t>(output_entry_count) * out_fm * out_plane;
		if (output_total == 0)
			return NNF_HIP_OK;
		if ((input_total > NNF_HIP_MAX_ELEMENT_COUNT) || (output_total > NNF_HIP_MAX_ELEMENT_COUNT))
			return NNF_HIP_ETOOBIG;
		if (overlap(output, output_total * sizeof(float), input, input_total * sizeof(float)))
			return NNF_HIP_EOVERLAP;

		// 2-D (or 1-D) windows within a feature map: stage through LDS
		const bool within_plane = (feature_map_subsampling_size == 1) && (entry_subsampling_size == 1) && (dimension_count <= 2);
		if (within_plane)
		{
			const int op = is_min ? (round_up_anywhere ? 3 : 1) : (round_up_anywhere ? 2 : 0);
			if (window2d_launch_with_prologue(stream, op, 0.0f, output, input, static_cast<uint32_t>(input_total), output_entry_count * input_feature_map_count,
				nd.in_size[0], nd.in_size[1], nd.out_size[0], nd.out_size[1], nd.window[0], nd.window[1], nd.stride[0], nd.stride[1],
				prologue, chunk_ptrs, input_feature_map_count, plan_only))
				return plan_only ? NNF_HIP_OK : launch_status();
		}
		if (prologue != nullptr)
			return NNF_HIP_EUNSUPPORTED; // only the LDS-staged kernel applies a prologue
		if (plan_only)
			return NNF_HIP_OK;

		// windows over feature maps and entries only
		if (identity_in_plane && launch_window_rows(stream, is_min ? window_op_min : window_op_max, 0.0f, output, input, output_entry_count,
			input_feature_map_count, out_fm, in_plane, feature_map_subsampling_size, entry_subsampling_size))
			return launch_status();

		nd.out = output;
		nd.in = input;
		nd.output_count = static_cast<uint32_t>(output_total);
		nd.in_fm = input_feature_map_count;
		nd.out_fm = out_fm;
		nd.fm_window = feature_map_subsampling_size;
		nd.entry_window = entry_subsampling_size;
		nd.in_plane = static_cast<uint32_t>(in_plane);
		const dim3 grid((nd.output_count + max_block_size - 1) / max_block_size);
		if (is_min)
			NNF_LAUNCH(window_nd_kernel<window_op_min>, grid, dim3(max_block_size), 0, stream, nd);
		else
			NNF_LAUNCH(window_nd_kernel<window_op_max>, grid, dim3(max_block_size), 0, stream, nd);
		return launch_status();
	}

	// Max subsampling with tiling (nnforge/plain/max_subsampling_layer_tester_plain.cpp:78-170): windows every
	// window-size elements, once per shift of the window grid; input entry e gives the output entries
	// e * T .. e * T + T - 1, T = product of the window sizes. Output size = (input - (window - 1)) / window
	// (nnforge/max_subsampling_layer.cpp:113-121). One lane per output; the shifted grids read the same input
	// T times over, out of the caches.
	int max_subsampling_tiling_forward(hipStream_t stream, float* output, const float* input,
		uint32_t input_entry_count, uint32_t feature_map_count, uint32_t dimension_count,
		const uint32_t* input_sizes, const uint32_t* subsampling_sizes, int32_t is_min)
	{
		if ((output == nullptr) || (input == nullptr) || (input_sizes == nullptr) || (subsampling_sizes == nullptr))
			return NNF_HIP_EINVAL;
		if ((dimension_count < 1) || (dimension_count > max_dims))
			return NNF_HIP_EUNSUPPORTED;
		if (feature_map_count == 0)
			return NNF_HIP_EINVAL;
		if (!is_aligned16(output) || !is_aligned16(input))
			return NNF_HIP_EALIGN;
		window_nd_args nd = {};
		uint64_t in_plane = 1, out_plane = 1, tile_count = 1;
		for(uint32_t d = 0; d < max_dims; ++d)
		{
			nd.in_size[d] = nd.out_size[d] = nd.window[d] = nd.stride[d] = 1;
			if (d >= dimension_count)
				continue;
			const uint32_t size = input_sizes[d], window = subsampling_sizes[d];
			if ((window == 0) || (static_cast<uint64_t>(size) + 1 < static_cast<uint64_t>(window) * 2))
				return NNF_HIP_EINVAL; // "smaller than subsampling size * 2 - 1"
			nd.in_size[d] = size;
			nd.window[d] = nd.stride[d] = window;
			nd.out_size[d] = (size - (window - 1)) / window;
			in_plane *= size;
			out_plane *= nd.out_size[d];
			tile_count *= window;
			if (tile_count > 0xFFFFull)
				return NNF_HIP_ETOOBIG;
		}
		const uint64_t input_total = static_cast<uint64_t>(input_entry_count) * feature_map_count * in_plane;
		const uint64_t output_total = static_cast<uint64_t>(input_entry_count) * tile_count * feature_map_count * out_plane;
		if (output_total == 0)
			return NNF_HIP_OK;
		if ((input_total > NNF_HIP_MAX_ELEMENT_COUNT) || (output_total > NNF_HIP_MAX_ELEMENT_COUNT))
			return NNF_HIP_ETOOBIG;
		if (overlap(output, output_total * sizeof(float), input, input_total * sizeof(float)))
			return NNF_HIP_EOVERLAP;
		if ((dimension_count <= 2) && launch_tiling2d(stream, is_min != 0, output, input, static_cast<uint32_t>(input_total), input_entry_count * feature_map_count, feature_map_count,
			nd.in_size[0], nd.in_size[1], nd.out_size[0], nd.out_size[1], nd.window[0], nd.window[1]))
			return launch_status();
		nd.out = output;
		nd.in = input;
		nd.output_count = static_cast<uint32_t>(output_total);
		nd.in_fm = nd.out_fm = feature_map_count;
		nd.fm_window = nd.entry_window = 1;
		nd.in_plane = static_cast<uint32_t>(in_plane);
		nd.tile_count = static_cast<uint32_t>(tile_count);
		const dim3 grid((nd.output_count + max_block_size - 1) / max_block_size);
		if (is_min)
			NNF_LAUNCH((window_nd_kernel<window_op_min, true>), grid, dim3(max_block_size), 0, stream, nd);
		else
			NNF_LAUNCH((window_nd_kernel<window_op_max, true>), grid, dim3(max_block_size), 0, stream, nd);
		return launch_status();
	}

	// Average subsampling in the reference's full form (nnforge/plain/average_subsampling_layer_tester_plain.cpp:34-148):
	// 1 to 4 spatial dimensions, windows over feature maps and over entries, every output the left-to-right fp32
	// sum of its window - x fastest, then the further dimensions, feature maps, entries - times mult. Output size =
	// input size / window size rounded down per dimension; a margin is not read. Plain 1-D / 2-D windows go to
	// the staged kernels of average_subsampling_forward; everything else takes one lane per output.
	int average_subsampling_nd_forward(hipStream_t stream, float* output, const float* input,
		uint32_t output_entry_count, uint32_t input_feature_map_count, uint32_t dimension_count,
		const uint32_t* input_sizes, const uint32_t* subsampling_sizes,
		uint32_t feature_map_subsampling_size, uint32_t entry_subsampling_size, float mult)
	{
		if ((output == nullptr) || (input == nullptr) || (input_sizes == nullptr) || (subsampling_sizes == nullptr))
			return NNF_HIP_EINVAL;
		if ((dimension_count < 1) || (dimension_count > max_dims))
			return NNF_HIP_EUNSUPPORTED;
		if ((input_feature_map_count == 0) || (feature_map_subsampling_size == 0) || (entry_subsampling_size == 0))
			return NNF_HIP_EINVAL;
		if ((dimension_count <= 2) && (feature_map_subsampling_size == 1) && (entry_subsampling_size == 1))
			return average_subsampling_forward(stream, output, input, output_entry_count, input_feature_map_count,
				input_sizes[0], (dimension_count > 1) ? input_sizes[1] : 1u, subsampling_sizes[0], (dimension_count > 1) ? subsampling_sizes[1] : 1u, mult);
		if (!is_aligned16(output) || !is_aligned16(input))
			return NNF_HIP_EALIGN;
		window_nd_args nd = {};
		uint64_t in_plane = 1, out_plane = 1;
		for(uint32_t d = 0; d < max_dims; ++d)
		{
			nd.in_size[d] = nd.out_size[d] = nd.window[d] = nd.stride[d] = 1;
			if (d >= dimension_count)
				continue;
			if ((input_sizes[d] == 0) || (subsampling_sizes[d] == 0) || (input_sizes[d] < subsampling_sizes[d]))
				return NNF_HIP_EINVAL; // nnforge/average_subsampling_layer.cpp:82-87
			nd.in_size[d] = input_sizes[d];
			nd.window[d] = nd.stride[d] = subsampling_sizes[d];
			nd.out_size[d] = input_sizes[d] / subsampling_sizes[d];
			in_plane *= nd.in_size[d];
			out_plane *= nd.out_size[d];
		}
		const uint32_t out_fm = input_feature_map_count / feature_map_subsampling_size;
		if (out_fm == 0)
			return NNF_HIP_EINVAL;
		const uint64_t input_total = static_cast<uint64_t>(output_entry_count) * entry_subsampling_size * input_feature_map_count * in_plane;
		const uint64_t output_total = static_cast<uint64_t>(output_entry_count) * out_fm * out_plane;
		if (output_total == 0)
			return NNF_HIP_OK;
		if ((input_total > NNF_HIP_MAX_ELEMENT_COUNT) || (output_total > NNF_HIP_MAX_ELEMENT_COUNT))
			return NNF_HIP_ETOOBIG;
		if (overlap(output, output_total * sizeof(float), input, input_total * sizeof(float)))
			return NNF_HIP_EOVERLAP;
		nd.out = output;
		nd.in = input;
		nd.output_count = static_cast<uint32_t>(output_total);
		nd.in_fm = input_feature_map_count;
		nd.out_fm = out_fm;
		nd.fm_window = feature_map_subsampling_size;
		nd.entry_window = entry_subsampling_size;
		nd.in_plane = static_cast<uint32_t>(in_plane);
		nd.mult = mult;
		// windows over feature maps and entries only
		bool identity_in_plane = true;
		for(uint32_t d = 0; d < max_dims; ++d)
			identity_in_plane = identity_in_plane && (nd.window[d] == 1);
		if (identity_in_plane && launch_window_rows(stream, window_op_sum, mult, output, input, output_entry_count,
			input_feature_map_count, out_fm, in_plane, feature_map_subsampling_size, entry_subsampling_size))
			return launch_status();
		const dim3 grid((nd.output_count + max_block_size - 1) / max_block_size);
		NNF_LAUNCH(window_nd_kernel<window_op_sum>, grid, dim3(max_block_size), 0, stream, nd);
		return launch_status();
	}

	int max_subsampling_forward(hipStream_t stream, float* output, const float* input,
		uint32_t output_entry_count, uint32_t input_feature_map_count, uint32_t dimension_count,
		const uint32_t* input_sizes, const uint32_t* subsampling_sizes, const uint32_t* strides, const uint32_t* round_ups,
		uint32_t feature_map_subsampling_size, uint32_t entry_subsampling_size, int32_t is_min)
	{
		return max_subsampling_forward_with_prologue(stream, output, input, output_entry_count, input_feature_map_count, dimension_count,
			input_sizes, subsampling_sizes, strides, round_ups, feature_map_subsampling_size, entry_subsampling_size, is_min, nullptr, nullptr, false);
	}

	int maxout_forward(hipStream_t stream, float* output, const float* input,
		uint32_t entry_count, uint32_t output_feature_map_count, uint32_t neuron_count_per_feature_map,
		uint32_t feature_map_subsampling_size)
	{
		if ((output == nullptr) || (input == nullptr))
			return NNF_HIP_EINVAL;
		// nnforge/maxout_layer.cpp:36-40
		if ((feature_map_subsampling_size < 2) || (output_feature_map_count == 0) || (neuron_count_per_feature_map == 0))
			return NNF_HIP_EINVAL;
		if (!is_aligned16(output) || !is_aligned16(input))
			return NNF_HIP_EALIGN;
		const uint64_t group64 = static_cast<uint64_t>(output_feature_map_count) * neuron_count_per_feature_map;
		const uint64_t output_total = group64 * entry_count;
		const uint64_t input_total = output_total * feature_map_subsampling_size;
		if (output_total == 0)
			return NNF_HIP_OK;
		if (input_total > NNF_HIP_MAX_ELEMENT_COUNT)
			return NNF_HIP_ETOOBIG;
		if (overlap(output, output_total * sizeof(float), input, input_total * sizeof(float)))
			return NNF_HIP_EOVERLAP;
		const uint32_t group = static_cast<uint32_t>(group64);
		const uint32_t rows = std::min(entry_count, 65535u);
		const uint32_t pair_blocks = (group / 4 + max_block_size * maxout_pair_unroll - 1) / (max_block_size * maxout_pair_unroll);
		// four float4s per lane where that still leaves two workgroups per compute unit (24 entries of 256 x 14 x 14 outputs, 312
		// such workgroups: 4.4 against 3.8 us with one float4 per lane; 48 entries: 5.9 against 6.4 us)
		if (((group % 4) == 0) && (feature_map_subsampling_size == 2) && (static_cast<uint64_t>(pair_blocks) * rows >= 2ull * compute_unit_count()))
		{
			const dim3 grid(pair_blocks, rows);
			const uint32_t hold = (rows == entry_count) ? read_phase_ticks(static_cast<uint64_t>(grid.x) * grid.y, 8, input_total * sizeof(float)) : 0;
			NNF_LAUNCH(maxout_pairs_kernel, grid, dim3(max_block_size), 0, stream, output, input, entry_count, group, hold);
		}
		else if ((group % 4) == 0)
		{
			const dim3 grid((group / 4 + max_block_size - 1) / max_block_size, rows);
			NNF_LAUNCH(maxout_vec4_kernel, grid, dim3(max_block_size), 0, stream, output, input, entry_count, group, feature_map_subsampling_size);
		}
		else
		{
			const dim3 grid((group + max_block_size - 1) / max_block_size, rows);
			NNF_LAUNCH(maxout_scalar_kernel, grid, dim3(max_block_size), 0, stream, output, input, entry_count, group, feature_map_subsampling_size);
		}
		return launch_status();
	}
}
