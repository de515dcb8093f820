// 2-D average subsampling with non-overlapping windows
// (nnforge/plain/average_subsampling_layer_tester_plain.cpp:125-145): every output is the
// left-to-right fp32 sum of its window (x fastest, then y) multiplied by mult. All kernels keep
// that summation order, so results equal the reference's bit for bit. Windows smaller than the
// plane go through the LDS-staged 2-D window kernel shared with max subsampling (nnf_max.hip);
// the one-lane-per-output kernel below remains for the shapes that kernel declines.
#include "nnf_common.h"
#include "nnf_prologue.h"

#include <algorithm>
#include <cstdlib>
#include <type_traits>

namespace nnf
{
	namespace
	{
		constexpr int pool_block_size = 256;
		constexpr uint32_t global_pool_planes = 64;    // most planes a workgroup of the global pooling kernel takes
		constexpr uint32_t global_pool_max_plane = 240; // 64 planes * 241 floats of padded LDS = 60 KB
		constexpr uint32_t global_pool_lds_floats = 4096; // a workgroup stages about this much: more, smaller workgroups per compute unit

		// Window == whole plane (global pooling, e.g. 7x7 -> 1x1). A workgroup reduces planes_per_group
		// (a multiple of 4, at most 64) consecutive planes: its 256 lanes copy them to LDS with coalesced
		// float4 loads, then lane t of the first wavefront sums plane t front to back. Planes are stored with an odd stride so that the 64 lanes
		// hit distinct banks. Many small workgroups: the load, barrier and summation phases of
		// different workgroups on a compute unit overlap.
		__global__ void __launch_bounds__(pool_block_size) global_pool_kernel(float* out, const float* in, uint32_t plane_count, uint32_t plane, uint32_t plane_magic, float mult, uint32_t planes_per_group)
		{
			extern __shared__ __align__(16) float lds_planes[];
			const uint32_t stride = plane | 1u;
			const uint32_t first_plane = blockIdx.x * planes_per_group;
			const uint32_t planes_here = min(planes_per_group, plane_count - first_plane);
			const uint32_t floats_here = planes_here * plane; // multiple of 4 except possibly in the last workgroup
			const float* src = in + static_cast<size_t>(first_plane) * plane; // 16-byte aligned: first_plane is a multiple of 4

			const uint32_t vectors = floats_here / 4;
			// four loads in flight per lane before the first value goes to LDS (a workgroup stages about 4096 floats)
			constexpr int stage = 4;
			for(uint32_t base = 0; base < vectors; base += stage * pool_block_size)
			{
				// No branch around a load (lanes past the end load the last float4 once more and do not stage it): with one,
				// every load of a round waited for the one before it.
				floatx4 t[stage];
				#pragma unroll
				for(int k = 0; k < stage; ++k)
					t[k] = load_stream(reinterpret_cast<const floatx4*>(src) + min(base + k * pool_block_size + threadIdx.x, vectors - 1));
				#pragma unroll
				for(int k = 0; k < stage; ++k)
				{
					const uint32_t i = base + k * pool_block_size + threadIdx.x;
					if (i < vectors)
					{
						const float vals[4] = {t[k].x, t[k].y, t[k].z, t[k].w};
						// floats_here * plane < 2^32: the multiplication by ceil(2^32 / plane) divides exactly
						uint32_t p = __umulhi(i * 4, plane_magic);
						uint32_t r = i * 4 - p * plane;
						#pragma unroll
						for(int e = 0; e < 4; ++e)
						{
							lds_planes[p * stride + r] = vals[e];
							if (++r == plane)
							{
								r = 0;
								++p;
							}
						}
					}
				}
			}
			for(uint32_t f = vectors * 4 + threadIdx.x; f < floats_here; f += pool_block_size)
			{
				const uint32_t p = f / plane;
				lds_planes[p * stride + (f - p * plane)] = src[f];
			}
			__syncthreads();

			if (threadIdx.x < planes_here)
			{
				const float* my_plane = lds_planes + threadIdx.x * stride;
				float sum = 0.0f;
				#pragma unroll 8
				for(uint32_t i = 0; i < plane; ++i)
					sum += my_plane[i];
				out[first_plane + threadIdx.x] = sum * mult;
			}
		}

		// The same with the element-wise layers in front of the subsampling layer applied to the values between
		// the load and the LDS store. Lane p works out the coefficients of plane p of the workgroup (at most
		// 64 planes) into an LDS table. A float4 may hold the end of one plane and the start of the next
		// (planes of 49 floats): then it goes through the layers twice, once with each plane's
		// coefficients, and every float keeps the result that is its own.
		// JOIN: the group has two inputs (in, in2: same shape) that an Add sums after each one's own layers.
		// GROUP: one of the groups of apply_known_group (nnf_prologue.h), compiled as straight code (77 to 92 registers per
		// lane instead of 107 to 124). With the loads of a round issued without a branch around each as well: BatchNorm -> ReLU
		// in front of the average over 64 x 2048 planes of 8 x 8 11.7 -> 8.2 us, 64 x 1024 of 14 x 14 16.6 -> 11.9 us,
		// 256 x 1024 of 4 x 4 13.2 -> 7.7 us; the residual block (two inputs) 16.1 -> 12.8 us, 24.0 -> 19.6 us and
		// 8.9 -> 6.6 us (256 x 512 of 4 x 4). The loads alone, any group: 16.0 -> 13.5 us and 23.9 -> 20.3 us.
		template<bool EXP, bool JOIN, int GROUP = known_group_none>
		__global__ void __launch_bounds__(pool_block_size) global_pool_prologue_kernel(float* out, const float* in, const float* in2, uint32_t plane_count, uint32_t plane,
			uint32_t plane_magic, float mult, uint32_t planes_per_group, const window_prologue pro)
		{
			extern __shared__ __align__(16) float lds_planes[];
			__shared__ uint64_t lds_exp[EXP ? exp_lds_entries : 1];
			__shared__ float lds_coef[global_pool_planes * 2 * prologue_weighted_max];
			exp_context exp_ctx = make_exp_context(lds_exp);
			const float none[prologue_weighted_max][2] = {};

			const uint32_t stride = plane | 1u;
			const uint32_t first_plane = blockIdx.x * planes_per_group;
			const uint32_t planes_here = min(planes_per_group, plane_count - first_plane);
			const uint32_t floats_here = planes_here * plane;
			const float* src = in + static_cast<size_t>(first_plane) * plane;
			const float* src2 = JOIN ? in2 + static_cast<size_t>(first_plane) * plane : nullptr;
			const uint32_t coef_stride = 2 * pro.weighted_count;

			const prologue_weights weights = load_prologue_weights(first_plane % pro.fm_count, planes_here, pro);
			const uint32_t vectors = floats_here / 4;
			constexpr int stage = 4; // a workgroup stages about 4096 floats: one round
			for(uint32_t base = 0; base < vectors; base += stage * pool_block_size)
			{
				floatx4 t[stage], t2[stage]; // t2, u: unused without JOIN
				#pragma unroll
				for(int k = 0; k < stage; ++k)
				{
					// no branch around a load: lanes past the end take the last float4 through the layers once more and do not stage it
					const uint32_t i = min(base + k * pool_block_size + threadIdx.x, vectors - 1);
					t[k] = load_stream(reinterpret_cast<const floatx4*>(src) + i);
					if (JOIN)
						t2[k] = load_stream(reinterpret_cast<const floatx4*>(src2) + i);
				}
				if (base == 0)
				{
					stage_prologue_coefficients(lds_coef, weights, planes_here, pro);
					if (EXP)
						stage_exp2_table(lds_exp);
					__syncthreads();
					if (EXP)
						exp_ctx = exp_context_from_lds(lds_exp);
				}
				float v[stage][4], u[stage][4];
				uint32_t first_plane_of[stage], off[stage];
				bool straddles = false;
				#pragma unroll
				for(int k = 0; k < stage; ++k)
				{
					const uint32_t i = min(base + k * pool_block_size + threadIdx.x, vectors - 1);
					v[k][0] = t[k].x; v[k][1] = t[k].y; v[k][2] = t[k].z; v[k][3] = t[k].w;
					if (JOIN)
					{
						u[k][0] = t2[k].x; u[k][1] = t2[k].y; u[k][2] = t2[k].z; u[k][3] = t2[k].w;
					}
					// floats_here * plane < 2^32: the multiplication by ceil(2^32 / plane) divides exactly
					first_plane_of[k] = __umulhi(i * 4, plane_magic);
					off[k] = first_plane_of[k] * coef_stride;
					straddles = straddles || (i * 4 + 3 >= (first_plane_of[k] + 1) * plane);
				}
				if (GROUP != known_group_none)
					apply_known_group<stage, (GROUP != known_group_none) ? GROUP : known_group_batch_norm_relu, false>(v, u, off, lds_coef, none, pro, exp_ctx);
				else
					apply_prologue_group<stage, EXP, JOIN>(v, u, off, lds_coef, none, pro, exp_ctx);
				if (__any(straddles))
				{
					// one float4 at a time: the copies that go through the layers a second time stay few
					#pragma unroll
					for(int k = 0; k < stage; ++k)
					{
						const uint32_t i = min(base + k * pool_block_size + threadIdx.x, vectors - 1);
						float w[1][4] = { { t[k].x, t[k].y, t[k].z, t[k].w } };
						float w2[1][4] = { { 0.0f, 0.0f, 0.0f, 0.0f } };
						if (JOIN)
						{
							w2[0][0] = t2[k].x; w2[0][1] = t2[k].y; w2[0][2] = t2[k].z; w2[0][3] = t2[k].w;
						}
						const uint32_t next_off[1] = { min(first_plane_of[k] + 1, planes_here - 1) * coef_stride }; // beyond the last plane: not stored
						if (GROUP != known_group_none)
							apply_known_group<1, (GROUP != known_group_none) ? GROUP : known_group_batch_norm_relu, false>(w, w2, next_off, lds_coef, none, pro, exp_ctx);
						else
							apply_prologue_group<1, EXP, JOIN>(w, w2, next_off, lds_coef, none, pro, exp_ctx);
						#pragma unroll
						for(uint32_t e = 1; e < 4; ++e)
						{
							if (i * 4 + e >= (first_plane_of[k] + 1) * plane)
								v[k][e] = w[0][e];
						}
					}
				}
				#pragma unroll
				for(int k = 0; k < stage; ++k)
				{
					const uint32_t i = base + k * pool_block_size + threadIdx.x;
					if (i < vectors)
					{
						uint32_t p = first_plane_of[k];
						uint32_t r = i * 4 - p * plane;
						#pragma unroll
						for(int e = 0; e < 4; ++e)
						{
							lds_planes[p * stride + r] = v[k][e];
							if (++r == plane)
							{
								r = 0;
								++p;
							}
						}
					}
				}
			}
			// the up to three floats behind the last whole float4 (last workgroup of a plane count that is no multiple of 4)
			for(uint32_t f = vectors * 4 + threadIdx.x; f < floats_here; f += pool_block_size)
			{
				const uint32_t p = f / plane;
				float one[1][4] = { { src[f], 0.0f, 0.0f, 0.0f } };
				float one2[1][4] = { { JOIN ? src2[f] : 0.0f, 0.0f, 0.0f, 0.0f } };
				const uint32_t one_off[1] = { p * coef_stride };
				if (GROUP != known_group_none)
					apply_known_group<1, (GROUP != known_group_none) ? GROUP : known_group_batch_norm_relu, false>(one, one2, one_off, lds_coef, none, pro, exp_ctx);
				else
					apply_prologue_group<1, EXP, JOIN>(one, one2, one_off, lds_coef, none, pro, exp_ctx);
				lds_planes[p * stride + (f - p * plane)] = one[0][0];
			}
			__syncthreads();

			if (threadIdx.x < planes_here)
			{
				const float* my_plane = lds_planes + threadIdx.x * stride;
				float sum = 0.0f;
				#pragma unroll 8
				for(uint32_t i = 0; i < plane; ++i)
					sum += my_plane[i];
				out[first_plane + threadIdx.x] = sum * mult;
			}
		}

		// Whole-plane windows over planes of an odd number of floats (7x7, the end of a ResNet). Every wavefront works
		// alone on linear_planes_per_wave consecutive planes: it copies them to its own part of LDS as they lie in memory
		// (float4 loads four at a time, float4 LDS stores; an odd plane size puts the planes of different lanes on
		// different banks), then lane t sums plane t front to back. No workgroup barrier, no index arithmetic per value.
		// With a group folded in (PROLOGUE), the layers are applied to the float4s between the load and the LDS store,
		// by all lanes. Lane p works out the coefficients of the wavefront's plane p into a small LDS table of the
		// wavefront's own; a float4 that holds the end of one plane and the start of the next takes both planes'
		// coefficients and every value picks its own. JOIN: two inputs, each through its own layers, summed by the
		// group's Add, the layers behind it applied to the sum.
		// Measured on 64 x 2048 x 7 x 7 (25.7 MB): 6.2 us against 8.9 us for the kernel above; 64 planes per wavefront 6.8 us,
		// all thirteen float4s of a lane loaded before the first LDS store 9.0 us (all seven of 32 planes: 6.3 us, no change). With BatchNorm + ReLU folded in 8.9 us, with a
		// joined block 14.0 us (16 planes per wavefront: 9.8 and 14.5 us; 64: 10.3 and 13.2 us).
		// GROUP: the folded layers are one of the groups of nnf_prologue.h's apply_known_group, compiled as straight code
		// (68 registers per lane instead of 127), with rounds of two float4s per lane and input and the next round requested
		// before the layers are applied to this one. Same shape: BatchNorm -> ReLU folded in 8.6 -> 7.2 us, the joined
		// block 13.2 -> 10.8 us (128 entries: 21.7 -> 18.1 us; 32 x 1024 planes of 11 x 11: 12.6 -> 8.8 us). Rounds of
		// one, three and four float4s: 10.8 / 11.7 / 11.7 us for the joined block, 7.4 / 8.1 / 7.6 us for BatchNorm -> ReLU.
		constexpr uint32_t linear_planes_per_wave = 32;
		constexpr int linear_waves = 4;
		constexpr size_t linear_lds_bytes_max = 64 * 1024;

		// (Four wavefronts per SIMD for every instance: 64 x 2048 planes are 1024 workgroups, which 256 compute units hold all
		// at once at four each - every load of the launch is then requested in its first microsecond. The instance with two
		// inputs and no expf took 132 registers, three workgroups per compute unit and a second round for the last quarter;
		// with two inputs and expf it takes 152 and would spill 45 of them, so that one stays at three.)
		template<bool PROLOGUE, bool EXP, bool JOIN, int GROUP = known_group_none>
		__global__ void __launch_bounds__(linear_waves * wave_size) __attribute__((amdgpu_waves_per_eu((EXP && JOIN) ? 3 : 4))) global_pool_linear_kernel(float* out, const float* in, const float* in2,
			uint32_t plane_count, uint32_t plane, uint32_t plane_magic, float mult, const window_prologue pro)
		{
			extern __shared__ __align__(16) float lds_planes[];
			__shared__ uint64_t lds_exp[EXP ? linear_waves * exp_lds_entries : 1];
			__shared__ float lds_coef[PROLOGUE ? linear_waves * linear_planes_per_wave * 2 * prologue_weighted_max : 1];
			const uint32_t lane = threadIdx.x % wave_size;
			const uint32_t wave = threadIdx.x / wave_size;
			const uint32_t first_plane = (blockIdx.x * linear_waves + wave) * linear_planes_per_wave;
			if (first_plane >= plane_count)
				return; // wavefronts never wait for each other
			const uint32_t planes_here = min(linear_planes_per_wave, plane_count - first_plane);
			const uint32_t floats_here = planes_here * plane; // a multiple of 4 except possibly in the last wavefront
			const size_t first_float = static_cast<size_t>(first_plane) * plane; // 16-byte aligned: first_plane is a multiple of 4
			const float* src = in + first_float;
			const float* src2 = JOIN ? in2 + first_float : nullptr;
			float* mine = lds_planes + wave * (linear_planes_per_wave * plane);
			float* my_coef = lds_coef + wave * (linear_planes_per_wave * 2 * prologue_weighted_max);
			const uint32_t coef_stride = 2 * pro.weighted_count;
			const float none[prologue_weighted_max][2] = {};

			// the weights of plane `lane` of this wavefront and the lane's share of the expf table: requested before the
			// tensor, looked at after its first loads are out
			float w[prologue_weighted_max][4] = {};
			if (PROLOGUE && (lane < planes_here))
			{
				const uint32_t fm = (first_plane + lane) % pro.fm_count;
				#pragma unroll
				for(uint32_t j = 0; j < prologue_weighted_max; ++j)
				{
					if (j < pro.weighted_count)
					{
						w[j][0] = pro.weights[j][0][fm];
						if (pro.weighted_kind[j] == NNF_HIP_OP_BATCH_NORM)
						{
							#pragma unroll
							for(int c = 1; c < 4; ++c)
								w[j][c] = pro.weights[j][c][fm];
						}
					}
				}
			}
			uint64_t exp_entry = 0;
			if (EXP)
				exp_entry = load_exp2_table_entry();
			exp_context exp_ctx = make_exp_context(lds_exp);

			const uint32_t vectors = floats_here / 4;
			constexpr int stage = (GROUP != known_group_none) ? 2 : 4; // float4s per lane, input and round
			constexpr uint32_t step = stage * wave_size;
			// a round of a lane's float4s: requested ...
			auto request = [&](floatx4 (&t)[stage], floatx4 (&t2)[stage], const uint32_t base)
			{
				#pragma unroll
				for(int k = 0; k < stage; ++k)
				{
					// beyond the last float4: the last one again (taken through the layers with the rest, stored by nobody)
					const uint32_t i = min(base + k * wave_size + lane, vectors - 1);
					t[k] = load_stream(reinterpret_cast<const floatx4*>(src) + i);
					if (JOIN)
						t2[k] = load_stream(reinterpret_cast<const floatx4*>(src2) + i);
				}
			};
			// the coefficient table and the expf table of this wavefront, while the first loads are in flight
			auto prepare_tables = [&]()
			{
				#pragma unroll
				for(uint32_t j = 0; j < prologue_weighted_max; ++j)
				{
					#pragma unroll
					for(int c = 0; c < 4; ++c)
						asm volatile("" : "+v"(w[j][c])); // not looked at (nor waited for) before this point
				}
				#pragma unroll
				for(uint32_t j = 0; j < prologue_weighted_max; ++j)
				{
					if ((j < pro.weighted_count) && (lane < planes_here))
					{
						float* dst = my_coef + (lane * pro.weighted_count + j) * 2;
						if (pro.weighted_kind[j] == NNF_HIP_OP_BATCH_NORM)
							nnf_batch_norm_coefficients(w[j][0], w[j][1], w[j][2], w[j][3], dst[0], dst[1]);
						else
							dst[0] = w[j][0];
					}
				}
				if (EXP)
					exp_ctx = stage_exp2_table_per_wavefront(lds_exp, exp_entry);
				__builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
				__builtin_amdgcn_wave_barrier();
				__builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
			};
			// ... and the first COUNT of them taken through the layers into LDS
			auto through_layers = [&](auto count, floatx4 (&t)[stage], floatx4 (&t2)[stage], const uint32_t base)
			{
				constexpr int COUNT = decltype(count)::value;
				if (PROLOGUE)
				{
					float v[COUNT][4], u[COUNT][4];
					uint32_t off[COUNT];
					two_plane_offsets<COUNT> two;
					#pragma unroll
					for(int k = 0; k < COUNT; ++k)
					{
						const uint32_t i = min(base + k * wave_size + lane, vectors - 1);
						v[k][0] = t[k].x; v[k][1] = t[k].y; v[k][2] = t[k].z; v[k][3] = t[k].w;
						u[k][0] = JOIN ? t2[k].x : 0.0f; u[k][1] = JOIN ? t2[k].y : 0.0f; u[k][2] = JOIN ? t2[k].z : 0.0f; u[k][3] = JOIN ? t2[k].w : 0.0f;
						// floats_here * plane < 2^32: the multiplication by ceil(2^32 / plane) divides exactly
						const uint32_t p = __umulhi(i * 4, plane_magic);
						off[k] = p * coef_stride;
						two.off2[k] = min(p + 1, planes_here - 1) * coef_stride; // behind the last plane: values nobody stores
						two.split[k] = (p + 1) * plane - i * 4;                  // >= 4: the whole float4 lies in plane p
					}
					if (GROUP != known_group_none)
						apply_known_group<COUNT, (GROUP != known_group_none) ? GROUP : known_group_batch_norm_relu, false, true>(v, u, off, my_coef, none, pro, exp_ctx, &two);
					else
						apply_prologue_group<COUNT, EXP, JOIN, false, true>(v, u, off, my_coef, none, pro, exp_ctx, &two);
					#pragma unroll
					for(int k = 0; k < COUNT; ++k)
					{
						t[k].x = v[k][0]; t[k].y = v[k][1]; t[k].z = v[k][2]; t[k].w = v[k][3];
					}
				}
				#pragma unroll
				for(int k = 0; k < COUNT; ++k)
				{
					const uint32_t i = base + k * wave_size + lane;
					if (i < vectors)
						reinterpret_cast<floatx4*>(mine)[i] = t[k];
				}
			};
			auto finish = [&](floatx4 (&t)[stage], floatx4 (&t2)[stage], const uint32_t base)
			{
				if (PROLOGUE && (base == 0))
					prepare_tables();
				if (GROUP == known_group_none)
				{
					through_layers(std::integral_constant<int, stage>(), t, t2, base);
					return;
				}
				// the wavefront's last round: only as many float4s per lane as some lane has left
				static_assert((GROUP == known_group_none) || (stage == 2), "a round of the known groups is whole or half");
				if (__builtin_amdgcn_readfirstlane(vectors - base) > wave_size)
					through_layers(std::integral_constant<int, stage>(), t, t2, base);
				else
					through_layers(std::integral_constant<int, 1>(), t, t2, base);
			};
			if (GROUP != known_group_none)
			{
				// Two sets of registers take turns: the next round is on its way while the layers are applied to this one
				// (every request unconditional and clamped: no join of two paths between a request and the wait for an
				// earlier one, where the compiler would wait for everything outstanding). The request behind the last
				// round asks for the wavefront's last float4 in every lane and is looked at by nobody. (vectors >= 1: the
				// host folds a group in over planes of four floats or more only.)
				floatx4 a[stage], a2[stage], b[stage], b2[stage];
				request(a, a2, 0);
				for(uint32_t base = 0; ; )
				{
					request(b, b2, base + step);
					finish(a, a2, base);
					base += step;
					if (base >= vectors)
						break;
					request(a, a2, base + step);
					finish(b, b2, base);
					base += step;
					if (base >= vectors)
						break;
				}
			}
			else
			{
				for(uint32_t base = 0; base < vectors; base += step)
				{
					floatx4 t[stage], t2[stage];
					request(t, t2, base);
					finish(t, t2, base);
				}
			}
			// the up to three floats behind the last whole float4 (last wavefront of a plane count that is no multiple of 4)
			for(uint32_t f = vectors * 4 + lane; f < floats_here; f += wave_size)
			{
				float one[1][4] = { { src[f], 0.0f, 0.0f, 0.0f } };
				if (PROLOGUE)
				{
					float one2[1][4] = { { JOIN ? src2[f] : 0.0f, 0.0f, 0.0f, 0.0f } };
					const uint32_t one_off[1] = { (f / plane) * coef_stride };
					apply_prologue_group<1, EXP, JOIN>(one, one2, one_off, my_coef, none, pro, exp_ctx);
				}
				mine[f] = one[0][0];
			}
			// what the other lanes of this wavefront stored is read below
			__builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
			__builtin_amdgcn_wave_barrier();
			__builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

			if (lane < planes_here)
			{
				const float* my_plane = mine + lane * plane;
				float sum = 0.0f;
				#pragma unroll 8
				for(uint32_t i = 0; i < plane; ++i)
					sum += my_plane[i];
				out[first_plane + lane] = sum * mult;
			}
		}

		// whether the kernel above takes this plane size; its launch
		bool global_pool_linear_fits(uint32_t plane)
		{
			return ((plane & 1u) != 0) && (plane >= 3) && (static_cast<size_t>(linear_waves) * linear_planes_per_wave * plane * sizeof(float) <= linear_lds_bytes_max);
		}

		void launch_global_pool_linear(hipStream_t stream, float* output, const float* input, const float* input2, uint32_t plane_count, uint32_t plane, float mult,
			const window_prologue* pro)
		{
			const bool join = (pro != nullptr) && (pro->join != 0);
			const size_t lds_bytes = static_cast<size_t>(linear_waves) * linear_planes_per_wave * plane * sizeof(float);
			const uint32_t planes_per_group = linear_waves * linear_planes_per_wave;
			const uint32_t plane_magic = static_cast<uint32_t>(((1ull << 32) + plane - 1) / plane);
			const dim3 grid((plane_count + planes_per_group - 1) / planes_per_group);
			const dim3 block(linear_waves * wave_size);
			if (pro == nullptr)
			{
				const window_prologue none = {};
				NNF_LAUNCH((global_pool_linear_kernel<false, false, false>), grid, block, lds_bytes, stream, output, input, input2, plane_count, plane, plane_magic, mult, none);
				return;
			}
			auto kernel = global_pool_linear_kernel<true, false, false>;
			const int group = known_group_of(*pro);
			if (pro->need_exp)
				kernel = join ? global_pool_linear_kernel<true, true, true> : global_pool_linear_kernel<true, true, false>;
			else if (group == known_group_batch_norm_relu)
				kernel = global_pool_linear_kernel<true, false, false, known_group_batch_norm_relu>;
			else if (group == known_group_batch_norm_shortcut_add_relu)
				kernel = global_pool_linear_kernel<true, false, true, known_group_batch_norm_shortcut_add_relu>;
			else if (group == known_group_shortcut_batch_norm_add_relu)
				kernel = global_pool_linear_kernel<true, false, true, known_group_shortcut_batch_norm_add_relu>;
			else if (join)
				kernel = global_pool_linear_kernel<true, false, true>;
			NNF_LAUNCH(kernel, grid, block, lds_bytes, stream, output, input, input2, plane_count, plane, plane_magic, mult, *pro);
		}

		// 64 planes of 7x7; fewer of larger planes, so that a compute unit holds several workgroups
		uint32_t global_pool_planes_per_group(uint32_t plane)
		{
			return std::min(global_pool_planes, std::max(8u, (global_pool_lds_floats / plane) & ~3u));
		}

		// General case: one lane per output neuron, window read straight from memory.
		__global__ void __launch_bounds__(pool_block_size) window_pool_kernel(
			float* out, const float* in, uint32_t output_count,
			uint32_t input_width, uint32_t input_height, uint32_t output_width, uint32_t output_height,
			uint32_t window_width, uint32_t window_height, float mult)
		{
			const uint32_t o = blockIdx.x * pool_block_size + threadIdx.x;
			if (o >= output_count)
				return;
			const uint32_t ox = o % output_width;
			const uint32_t oy = (o / output_width) % output_height;
			const uint32_t plane_id = o / (output_width * output_height);
			const float* src = in + static_cast<size_t>(plane_id) * input_width * input_height
				+ static_cast<size_t>(oy) * window_height * input_width + static_cast<size_t>(ox) * window_width;
			float sum = 0.0f;
			for(uint32_t wy = 0; wy < window_height; ++wy)
			{
				for(uint32_t wx = 0; wx < window_width; ++wx)
					sum += src[wy * input_width + wx];
			}
			out[o] = sum * mult;
		}
	}

	int average_subsampling_forward(hipStream_t stream, float* output, const float* input,
		uint32_t entry_count, uint32_t feature_map_count, uint32_t input_width, uint32_t input_height,
		uint32_t window_width, uint32_t window_height, float mult)
	{
		return average_subsampling_forward_with_prologue(stream, output, input, nullptr, entry_count, feature_map_count, input_width, input_height,
			window_width, window_height, mult, nullptr, nullptr, false);
	}

	// prologue != null: the layers of that group are applied to the input first (the LDS-staged kernels only:
	// whole-plane averages and 2-D windows; NNF_HIP_EUNSUPPORTED for shapes they do not take). A group of two
	// inputs joined by an Add (input2: its second input, same shape as input) goes with whole-plane averages
	// only. plan_only: nothing is launched and no pointer is looked at; NNF_HIP_OK means the call would run.
	int average_subsampling_forward_with_prologue(hipStream_t stream, float* output, const float* input, const float* input2,
		uint32_t entry_count, uint32_t feature_map_count, uint32_t input_width, uint32_t input_height,
		uint32_t window_width, uint32_t window_height, float mult,
		const nnf_hip_chain_desc* prologue, const float* const* chunk_ptrs, bool plan_only)
	{
		const bool join = (prologue != nullptr) && (prologue->input_count == 2);
		if (plan_only)
		{
			// planning looks at shapes only: stand-ins that pass the pointer checks below, never dereferenced
			output = reinterpret_cast<float*>(static_cast<uintptr_t>(16));
			input = reinterpret_cast<const float*>(static_cast<uintptr_t>(1) << 46);
			input2 = join ? reinterpret_cast<const float*>(static_cast<uintptr_t>(1) << 47) : nullptr;
		}
		if ((output == nullptr) || (input == nullptr) || (join != (input2 != nullptr)))
			return NNF_HIP_EINVAL;
		if ((feature_map_count == 0) || (input_width == 0) || (input_height == 0) || (window_width == 0) || (window_height == 0))
			return NNF_HIP_EINVAL;
		// nnforge/average_subsampling_layer.cpp:82-87: the input may not be smaller than the window; the
		// output size is the quotient rounded down and a leftover right/bottom margin is not read
		if ((input_width < window_width) || (input_height < window_height))
			return NNF_HIP_EINVAL;
		if (!is_aligned16(output) || !is_aligned16(input) || !is_aligned16(input2))
			return NNF_HIP_EALIGN;

		const uint32_t output_width = input_width / window_width;
		const uint32_t output_height = input_height / window_height;
		const uint64_t input_total = static_cast<uint64_t>(entry_count) * feature_map_count * input_width * input_height;
		if (input_total == 0)
			return NNF_HIP_OK;
		if (input_total > NNF_HIP_MAX_ELEMENT_COUNT)
			return NNF_HIP_ETOOBIG;
		const uint32_t plane_count = entry_count * feature_map_count;
		const uint32_t output_count = plane_count * output_width * output_height;
		{
			const uintptr_t a = reinterpret_cast<uintptr_t>(output), b = reinterpret_cast<uintptr_t>(input);
			if ((a < b + input_total * sizeof(float)) && (b < a + static_cast<uint64_t>(output_count) * sizeof(float)))
				return NNF_HIP_EOVERLAP; // the tester cannot run in place: get_input_index_layer_can_write is -1 for it
			const uintptr_t c = reinterpret_cast<uintptr_t>(input2);
			if (join && (a < c + input_total * sizeof(float)) && (c < a + static_cast<uint64_t>(output_count) * sizeof(float)))
				return NNF_HIP_EOVERLAP;
		}

		const uint32_t plane = input_width * input_height;
		if (prologue != nullptr)
		{
			const bool whole_plane = (window_width == input_width) && (window_height == input_height) && (plane >= 2) && (plane <= global_pool_max_plane);
			if (whole_plane)
			{
				// a float4 may straddle two planes, not three
				if (plane < 4)
					return NNF_HIP_EUNSUPPORTED;
				if (plan_only)
					return NNF_HIP_OK;
				window_prologue pro = {};
				if (!fill_prologue(pro, *prologue, chunk_ptrs, feature_map_count, plane, true) || (pro.weighted_count > prologue_weighted_max))
					return NNF_HIP_EUNSUPPORTED;
				if (global_pool_linear_fits(plane))
				{
					launch_global_pool_linear(stream, output, input, input2, plane_count, plane, mult, &pro);
					return launch_status();
				}
				const uint32_t planes_per_group = global_pool_planes_per_group(plane);
				const size_t lds_bytes = static_cast<size_t>(planes_per_group) * (plane | 1u) * sizeof(float);
				const dim3 grid((plane_count + planes_per_group - 1) / planes_per_group);
				const uint32_t plane_magic = static_cast<uint32_t>(((1ull << 32) + plane - 1) / plane);
				auto kernel = global_pool_prologue_kernel<false, false>;
				const int group = known_group_of(pro);
				if (pro.need_exp)
					kernel = join ? global_pool_prologue_kernel<true, true> : global_pool_prologue_kernel<true, false>;
				else if (group == known_group_batch_norm_relu)
					kernel = global_pool_prologue_kernel<false, false, known_group_batch_norm_relu>;
				else if (group == known_group_batch_norm_shortcut_add_relu)
					kernel = global_pool_prologue_kernel<false, true, known_group_batch_norm_shortcut_add_relu>;
				else if (group == known_group_shortcut_batch_norm_add_relu)
					kernel = global_pool_prologue_kernel<false, true, known_group_shortcut_batch_norm_add_relu>;
				else if (join)
					kernel = global_pool_prologue_kernel<false, true>;
				NNF_LAUNCH(kernel, grid, dim3(pool_block_size), lds_bytes, stream, output, input, input2, plane_count, plane, plane_magic, mult, planes_per_group, pro);
				return launch_status();
			}
			if (join)
				return NNF_HIP_EUNSUPPORTED; // the window kernels take single-input groups
			if (!window2d_launch_with_prologue(stream, 4, mult, output, input, static_cast<uint32_t>(input_total), plane_count,
				input_width, input_height, output_width, output_height, window_width, window_height, window_width, window_height,
				prologue, chunk_ptrs, feature_map_count, plan_only))
				return NNF_HIP_EUNSUPPORTED;
			return plan_only ? NNF_HIP_OK : launch_status();
		}
		if (plan_only)
			return NNF_HIP_OK;
		if ((window_width == input_width) && (window_height == input_height) && global_pool_linear_fits(plane))
			launch_global_pool_linear(stream, output, input, nullptr, plane_count, plane, mult, nullptr);
		else if ((window_width == input_width) && (window_height == input_height) && (plane >= 2) && (plane <= global_pool_max_plane))
		{
			const uint32_t planes_per_group = global_pool_planes_per_group(plane);
			const size_t lds_bytes = static_cast<size_t>(planes_per_group) * (plane | 1u) * sizeof(float);
			const dim3 grid((plane_count + planes_per_group - 1) / planes_per_group);
			// plane >= 2 here: a 1x1 window over a 1x1 plane takes the general kernel
			const uint32_t plane_magic = static_cast<uint32_t>(((1ull << 32) + plane - 1) / plane);
			NNF_LAUNCH(global_pool_kernel, grid, dim3(pool_block_size), lds_bytes, stream, output, input, plane_count, plane, plane_magic, mult, planes_per_group);
		}
		else if (window2d_launch(stream, 4, mult, output, input, static_cast<uint32_t>(input_total), plane_count,
			input_width, input_height, output_width, output_height, window_width, window_height, window_width, window_height))
		{
			// staged through LDS by the 2-D window kernel: contiguous float4 reads, windows summed x fastest
		}
		else
		{
			const dim3 grid((output_count + pool_block_size - 1) / pool_block_size);
			NNF_LAUNCH(window_pool_kernel, grid, dim3(pool_block_size), 0, stream, output, input, output_count,
				input_width, input_height, output_width, output_height, window_width, window_height, mult);
		}
		return launch_status();
	}
}
