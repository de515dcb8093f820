/*
 * nnf_oracle.c - CPU restatement of nnForge's plain (CPU) layer testers for the inference path.
 *
 * TEST INFRASTRUCTURE ONLY. Nothing the library ships calls this file: it exists so that the
 * parity tests, the smoke check and the benchmark's cpu_baseline leg have the reference's
 * arithmetic to compare against and to time. The product path is the HIP library and fails
 * loudly when that library is missing.
 *
 * Every function follows one reference tester, cited next to it, with the same operation order,
 * the same fp32 roundings (one per operation; built with -ffp-contract=off -fno-fast-math) and
 * the same libm expf the reference calls. Loops are parallelised the way the reference does it:
 * "#pragma omp parallel for schedule(guided)" over elements or over (entry, feature map) planes.
 *
 * What pins this restatement (the reference has no tests, golden vectors or fixtures of its own,
 * and its sources cannot be compiled in this image: every tester includes Boost and protobuf-
 * generated headers that are absent): tests/test_oracle.py checks each function against an
 * independent numpy evaluation (per-operation fp32 for the exactly reproducible layers, fp64
 * closed forms expm1 / logistic / tanh / softmax with error budgets for the ones that call expf),
 * plus identities (identity batch norm, PReLU(a=1) = x, PReLU(a=0) = ReLU(0), Add(x, 0) = alpha*x,
 * softmax rows sum to 1 and are shift invariant, pooling of a constant) and brute-force index
 * checks on tiny shapes with distinct values per element. The layers next to that path are pinned
 * the same way: absolute / dropout / concat against numpy's abs, identity and concatenate; maxout
 * against a reshape-and-max that fails for the wrong feature-map grouping, plus a Python fold of
 * std::max for the order-dependent cases (+0.0 / -0.0, NaN); max subsampling against numpy sliding
 * windows in 1, 2 and 3 dimensions with strides, padded windows for round up, a reshape-and-max for
 * feature-map / entry windows, the start value, tie and NaN cases, and a brute-force loop for tiling;
 * the statistics against two-pass fp64 numpy (mean, population variance, fp32 rounding before the
 * square root), packet invariance, a large-offset case, and the batch norm refresh against its two
 * fp32 formulas and the closed loop (refreshed weights give mean 0, deviation 1). The libm expf this file calls
 * is itself checked against recorded values (tests/golden/expf_vectors.npy: glibc 2.35 on 8192 inputs), so a host
 * whose expf differs is noticed. Not pinned by anything: the bit pattern
 * of the reference *as shipped* (built with -ffast-math -O3 -march=native, Settings.mk:26-28),
 * which depends on the compiler's contraction and vector-libm choices - "parity unpinned" for that;
 * this file states the source-level semantics.
 *
 * Layout: fp32, [entry][feature_map][y][x], x fastest (nnforge/layer_configuration_specific.cpp:62-73).
 */
#include <math.h>
#include <stddef.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define NNF_ORACLE_API __attribute__((visibility("default")))

static int thread_count(int requested)
{
#ifdef _OPENMP
	return requested > 0 ? requested : omp_get_max_threads();
#else
	(void)requested;
	return 1;
#endif
}

/* number of hardware threads OpenMP would use by default (plain_running_configuration's default,
 * nnforge/plain/factory_generator_plain.cpp:71) */
NNF_ORACLE_API int nnf_oracle_max_threads(void)
{
	return thread_count(0);
}

/* nnforge/plain/batch_norm_layer_tester_plain.cpp:43-74. data chunks: gamma, beta, mean, inverse
 * sigma (nnforge/batch_norm_layer.cpp:96-106); epsilon plays no part at inference. */
NNF_ORACLE_API void nnf_oracle_batch_norm(
	float* out, const float* in,
	const float* gamma, const float* beta, const float* mean, const float* inverse_sigma,
	unsigned int entry_count, unsigned int feature_map_count, unsigned int neuron_count_per_feature_map,
	int threads)
{
	const int total_workload = (int)(entry_count * feature_map_count);
	const unsigned int neuron_count = neuron_count_per_feature_map * feature_map_count;
	int workload_id;
	#pragma omp parallel for schedule(guided) num_threads(thread_count(threads))
	for (workload_id = 0; workload_id < total_workload; ++workload_id)
	{
		const int entry_id = workload_id / (int)feature_map_count;
		const int fm = workload_id - entry_id * (int)feature_map_count;
		const float mult = gamma[fm] * inverse_sigma[fm];
		const float add = beta[fm] - mult * mean[fm];
		const size_t offset = (size_t)entry_id * neuron_count + (size_t)fm * neuron_count_per_feature_map;
		const float* src = in + offset;
		float* dst = out + offset;
		unsigned int i;
		for (i = 0; i < neuron_count_per_feature_map; ++i)
			dst[i] = src[i] * mult + add;
	}
}

/* nnforge/plain/rectified_linear_layer_tester_plain.cpp:45-55 */
NNF_ORACLE_API void nnf_oracle_rectified_linear(float* out, const float* in, float negative_slope, long long elem_count, int threads)
{
	long long i;
	#pragma omp parallel for schedule(guided) num_threads(thread_count(threads))
	for (i = 0; i < elem_count; ++i)
	{
		const float x = in[i];
		out[i] = x >= 0.0F ? x : x * negative_slope;
	}
}

/* nnforge/plain/parametric_rectified_linear_layer_tester_plain.cpp:43-70; data chunk 0 = one slope
 * per feature map (nnforge/parametric_rectified_linear_layer.cpp:87-94) */
NNF_ORACLE_API void nnf_oracle_parametric_rectified_linear(
	float* out, const float* in, const float* slopes,
	unsigned int entry_count, unsigned int feature_map_count, unsigned int neuron_count_per_feature_map,
	int threads)
{
	const int total_workload = (int)(entry_count * feature_map_count);
	const unsigned int neuron_count = neuron_count_per_feature_map * feature_map_count;
	int workload_id;
	#pragma omp parallel for schedule(guided) num_threads(thread_count(threads))
	for (workload_id = 0; workload_id < total_workload; ++workload_id)
	{
		const int entry_id = workload_id / (int)feature_map_count;
		const int fm = workload_id - entry_id * (int)feature_map_count;
		const float a = slopes[fm];
		const size_t offset = (size_t)entry_id * neuron_count + (size_t)fm * neuron_count_per_feature_map;
		const float* src = in + offset;
		float* dst = out + offset;
		unsigned int i;
		for (i = 0; i < neuron_count_per_feature_map; ++i)
		{
			const float x = src[i];
			dst[i] = x * (x >= 0.0F ? 1.0F : a);
		}
	}
}

/* nnforge/plain/exponential_linear_layer_tester_plain.cpp:43-52 (expf(x) - 1, not expm1f) */
NNF_ORACLE_API void nnf_oracle_exponential_linear(float* out, const float* in, long long elem_count, int threads)
{
	long long i;
	#pragma omp parallel for schedule(guided) num_threads(thread_count(threads))
	for (i = 0; i < elem_count; ++i)
	{
		const float x = in[i];
		out[i] = x >= 0.0F ? x : (expf(x) - 1.0F);
	}
}

/* nnforge/plain/sigmoid_layer_tester_plain.cpp:43-53 */
NNF_ORACLE_API void nnf_oracle_sigmoid(float* out, const float* in, long long elem_count, int threads)
{
	long long i;
	#pragma omp parallel for schedule(guided) num_threads(thread_count(threads))
	for (i = 0; i < elem_count; ++i)
	{
		const float x = in[i];
		out[i] = 1.0F / (expf(-x) + 1.0F);
	}
}

/* nnforge/plain/hyperbolic_tangent_layer_tester_plain.cpp:43-58 */
NNF_ORACLE_API void nnf_oracle_hyperbolic_tangent(float* out, const float* in, float scale, float steepness, long long elem_count, int threads)
{
	const float steepness2 = steepness * 2.0F;
	long long i;
	#pragma omp parallel for schedule(guided) num_threads(thread_count(threads))
	for (i = 0; i < elem_count; ++i)
	{
		const float x = in[i];
		const float e = expf(x * steepness2);
		out[i] = (e - 1.0F) / (e + 1.0F) * scale;
	}
}

/* nnforge/plain/add_layer_tester_plain.cpp:45-61 */
NNF_ORACLE_API void nnf_oracle_add(float* out, const float* const* inputs, int input_count, float alpha, long long elem_count, int threads)
{
	long long i;
	#pragma omp parallel for schedule(guided) num_threads(thread_count(threads))
	for (i = 0; i < elem_count; ++i)
	{
		float sum = 0.0F;
		int j;
		for (j = 0; j < input_count; ++j)
			sum += inputs[j][i];
		out[i] = sum * alpha;
	}
}

/* nnforge/plain/softmax_layer_tester_plain.cpp:47-89 */
NNF_ORACLE_API void nnf_oracle_softmax(
	float* out, const float* in,
	unsigned int entry_count, unsigned int feature_map_count, unsigned int neuron_count_per_feature_map,
	int threads)
{
	const unsigned int neuron_count = neuron_count_per_feature_map * feature_map_count;
	const int total_workload = (int)(entry_count * neuron_count_per_feature_map);
	int workload_id;
	#pragma omp parallel for schedule(guided) num_threads(thread_count(threads))
	for (workload_id = 0; workload_id < total_workload; ++workload_id)
	{
		const int entry_id = workload_id / (int)neuron_count_per_feature_map;
		const int neuron_id = workload_id - entry_id * (int)neuron_count_per_feature_map;
		const float* src = in + (size_t)entry_id * neuron_count + neuron_id;
		float* dst = out + (size_t)entry_id * neuron_count + neuron_id;
		float max_val = -1.0e+37F;
		float sum = 0.0F;
		float mult;
		unsigned int fm;
		for (fm = 0; fm < feature_map_count; ++fm)
		{
			const float val = src[(size_t)fm * neuron_count_per_feature_map];
			max_val = (max_val < val) ? val : max_val; /* std::max(max_val, val) */
		}
		for (fm = 0; fm < feature_map_count; ++fm)
		{
			const float val = expf(src[(size_t)fm * neuron_count_per_feature_map] - max_val);
			sum += val;
			dst[(size_t)fm * neuron_count_per_feature_map] = val;
		}
		mult = 1.0F / sum;
		for (fm = 0; fm < feature_map_count; ++fm)
			dst[(size_t)fm * neuron_count_per_feature_map] *= mult;
	}
}

/*
 * nnforge/plain/average_subsampling_layer_tester_plain.cpp:47-147, all of it: any number of spatial
 * dimensions (dimension 0 = x is fastest), feature-map subsampling and entry subsampling. The
 * window of an output neuron is walked x fastest, then the further spatial dimensions, then
 * feature maps, then entries, summed left to right in fp32 and multiplied by mult.
 *   input_sizes / output_sizes / window_sizes: dimension_count values each.
 *   mult: the caller passes what the tester would compute (see nnf_oracle_average_subsampling_plain_mult).
 * entry_count is the number of OUTPUT entries.
 */
NNF_ORACLE_API void nnf_oracle_average_subsampling(
	float* out, const float* in,
	unsigned int entry_count,
	unsigned int input_feature_map_count, unsigned int output_feature_map_count,
	int dimension_count, const unsigned int* input_sizes, const unsigned int* output_sizes, const unsigned int* window_sizes,
	unsigned int feature_map_window, unsigned int entry_window,
	float mult, int threads)
{
	enum { max_dims = 6 };
	unsigned int sub_sizes[max_dims + 2];
	unsigned int slices[max_dims + 2];
	unsigned int in_plane = 1, out_plane = 1, window_elems = 1;
	int sub_count, d;
	unsigned int* offsets;
	const int total_workload = (int)(entry_count * output_feature_map_count);
	int workload_id;

	if (dimension_count < 1 || dimension_count > max_dims)
		return;
	for (d = 0; d < dimension_count; ++d)
	{
		sub_sizes[d] = window_sizes[d];
		in_plane *= input_sizes[d];
		out_plane *= output_sizes[d];
	}
	sub_sizes[dimension_count] = feature_map_window;
	sub_sizes[dimension_count + 1] = entry_window;
	sub_count = dimension_count + 2;
	slices[0] = 1;
	for (d = 0; d < sub_count - 1; ++d)
		slices[d + 1] = slices[d] * (d < dimension_count ? input_sizes[d] : input_feature_map_count);
	for (d = 0; d < sub_count; ++d)
		window_elems *= sub_sizes[d];

	/* input offset of every window element relative to the window's first element, odometer order */
	offsets = (unsigned int*)calloc(window_elems, sizeof(unsigned int));
	{
		unsigned int pos[max_dims + 2];
		unsigned int i;
		memset(pos, 0, sizeof(pos));
		for (i = 1; i < window_elems; ++i)
		{
			for (d = 0; d < sub_count; ++d)
			{
				if (++pos[d] < sub_sizes[d])
					break;
				pos[d] = 0;
			}
			offsets[i] = 0;
			for (d = 0; d < sub_count; ++d)
				offsets[i] += pos[d] * slices[d];
		}
	}

	#pragma omp parallel for schedule(guided) num_threads(thread_count(threads))
	for (workload_id = 0; workload_id < total_workload; ++workload_id)
	{
		const int out_entry = workload_id / (int)output_feature_map_count;
		const int out_fm = workload_id - out_entry * (int)output_feature_map_count;
		const float* src_base = in
			+ (size_t)out_entry * entry_window * in_plane * input_feature_map_count
			+ (size_t)out_fm * feature_map_window * in_plane;
		float* dst = out + ((size_t)out_entry * output_feature_map_count + out_fm) * out_plane;
		unsigned int out_pos[max_dims];
		unsigned int o;
		memset(out_pos, 0, sizeof(out_pos));
		for (o = 0; o < out_plane; ++o)
		{
			size_t first = 0;
			float sum = 0.0F;
			unsigned int i;
			int dd;
			for (dd = 0; dd < dimension_count; ++dd)
				first += (size_t)out_pos[dd] * sub_sizes[dd] * slices[dd];
			for (i = 0; i < window_elems; ++i)
				sum += src_base[first + offsets[i]];
			dst[o] = sum * mult;
			for (dd = 0; dd < dimension_count; ++dd)
			{
				if (++out_pos[dd] < output_sizes[dd])
					break;
				out_pos[dd] = 0;
			}
		}
	}
	free(offsets);
}

/*
 * The multiplier the PLAIN tester ends up with when the schema sets no alpha
 * (nnforge/plain/average_subsampling_layer_tester_plain.cpp:82): it hands the two feature-map
 * COUNTS to get_effective_alpha(const layer_configuration_specific&, const layer_configuration_specific&)
 * (nnforge/average_subsampling_layer.h:82-84); each count converts through the one-argument
 * constructor (nnforge/layer_configuration_specific.h:32) into a configuration without spatial
 * dimensions, so the loop over dimensions in nnforge/average_subsampling_layer.cpp:295-296 runs
 * zero times and only the feature-map and entry factors divide: 1 / (fm_window * entry_window).
 * With an explicit alpha the tester returns alpha itself.
 */
NNF_ORACLE_API float nnf_oracle_average_subsampling_plain_mult(unsigned int feature_map_window, unsigned int entry_window, int has_alpha, float alpha)
{
	if (has_alpha)
		return alpha;
	return 1.0F / (float)(feature_map_window * entry_window);
}

/*
 * The multiplier of average_subsampling_layer::get_effective_alpha when it is given the full
 * configurations (nnforge/average_subsampling_layer.cpp:287-303), as the CUDA tester does
 * (nnforge/cuda/average_subsampling_layer_tester_cuda.cuh:279): 1 / number of window elements.
 */
NNF_ORACLE_API float nnf_oracle_average_subsampling_full_mult(int dimension_count, const unsigned int* window_sizes,
	unsigned int feature_map_window, unsigned int entry_window, int has_alpha, float alpha)
{
	unsigned int elems = feature_map_window * entry_window;
	int d;
	if (has_alpha)
		return alpha;
	for (d = 0; d < dimension_count; ++d)
		elems *= window_sizes[d];
	return 1.0F / (float)elems;
}

/* ---- neighbouring inference testers of the same chains ----------------------------------- */

/* nnforge/plain/absolute_layer_tester_plain.cpp:43-49: out = fabs(in) */
NNF_ORACLE_API void nnf_oracle_absolute(float* out, const float* in, size_t elem_count, int threads)
{
	const long long count = (long long)elem_count;
	long long i;
	#pragma omp parallel for schedule(guided) num_threads(thread_count(threads))
	for (i = 0; i < count; ++i)
		out[i] = fabsf(in[i]);
}

/* nnforge/plain/dropout_layer_tester_plain.cpp:45-48: at inference the layer passes its input on
 * unchanged (a copy unless it runs in place) */
NNF_ORACLE_API void nnf_oracle_dropout(float* out, const float* in, size_t elem_count)
{
	if (out != in)
		memcpy(out, in, elem_count * sizeof(float));
}

/* nnforge/plain/concat_layer_tester_plain.cpp:45-58: per entry, the inputs' neurons one after the
 * other (feature maps of input 0, then of input 1, ...) */
NNF_ORACLE_API void nnf_oracle_concat(float* out, const float* const* inputs, const unsigned int* input_neuron_counts,
	int input_count, unsigned int entry_count)
{
	size_t output_neuron_count = 0;
	unsigned int entry_id;
	int i;
	for (i = 0; i < input_count; ++i)
		output_neuron_count += input_neuron_counts[i];
	for (entry_id = 0; entry_id < entry_count; ++entry_id)
	{
		float* dst = out + (size_t)entry_id * output_neuron_count;
		for (i = 0; i < input_count; ++i)
		{
			memcpy(dst, inputs[i] + (size_t)entry_id * input_neuron_counts[i], (size_t)input_neuron_counts[i] * sizeof(float));
			dst += input_neuron_counts[i];
		}
	}
}

/* std::max(a, b) and std::min(a, b) as the C++ library defines them: the first argument wins ties
 * and unordered comparisons */
static inline float std_max(float a, float b) { return (a < b) ? b : a; }
static inline float std_min(float a, float b) { return (b < a) ? b : a; }

/* nnforge/plain/maxout_layer_tester_plain.cpp:56-80: output feature map o is the maximum over the
 * input feature maps o, o + out_fm, o + 2*out_fm, ...; starts from the first value and folds with
 * std::max(new_val, current_max) */
NNF_ORACLE_API void nnf_oracle_maxout(float* out, const float* in, unsigned int entry_count, unsigned int output_feature_map_count,
	unsigned int plane, unsigned int feature_map_subsampling_size, int threads)
{
	const size_t output_neuron_count = (size_t)output_feature_map_count * plane;
	const size_t input_neuron_count = output_neuron_count * feature_map_subsampling_size;
	const int total_workload = (int)(entry_count * output_feature_map_count);
	int workload_id;
	#pragma omp parallel for schedule(guided) num_threads(thread_count(threads))
	for (workload_id = 0; workload_id < total_workload; ++workload_id)
	{
		const int entry_id = workload_id / (int)output_feature_map_count;
		const int fm = workload_id - entry_id * (int)output_feature_map_count;
		const float* src = in + (size_t)entry_id * input_neuron_count + (size_t)fm * plane;
		float* dst = out + (size_t)entry_id * output_neuron_count + (size_t)fm * plane;
		unsigned int p, i;
		for (p = 0; p < plane; ++p)
		{
			float current_max = src[p];
			for (i = 1; i < feature_map_subsampling_size; ++i)
				current_max = std_max(src[p + (size_t)i * output_neuron_count], current_max);
			dst[p] = current_max;
		}
	}
}

/*
 * nnforge/plain/max_subsampling_layer_tester_plain.cpp:175-290 (test_non_tiling): windows of
 * window_sizes[d] elements every strides[d] elements over the spatial dimensions, then over
 * feature_map_window neighbouring feature maps and entry_window neighbouring entries; the window is
 * scanned x fastest, ..., feature map, entry, starting from -1.0e37F (maximum) or 1.0e37F (minimum)
 * and folding with std::max<float>(current, new) / std::min<float>(current, new).
 * The plain tester refuses round_up; `truncate` restates what the CUDA tester does for it
 * (nnforge/cuda/max_subsampling_layer_tester_cuda.cuh:97-116, TRUNCATION): window elements that
 * lie beyond the input in a spatial dimension are skipped. output_sizes come from
 * nnforge/max_subsampling_layer.cpp:131-141.
 */
NNF_ORACLE_API void nnf_oracle_max_subsampling(float* out, const float* in, unsigned int output_entry_count,
	unsigned int input_feature_map_count, unsigned int output_feature_map_count,
	int dimension_count, const unsigned int* input_sizes, const unsigned int* output_sizes,
	const unsigned int* window_sizes, const unsigned int* strides,
	unsigned int feature_map_window, unsigned int entry_window, int is_min, int truncate, int threads)
{
	enum { max_dims = 6 };
	unsigned int sub_sizes[max_dims + 2];
	size_t slices[max_dims + 2];
	size_t in_plane = 1, out_plane = 1;
	unsigned int window_elems = 1;
	int sub_count, d;
	size_t* offsets;
	unsigned int* positions; /* window element -> its position in every spatial dimension */
	const int total_workload = (int)(output_entry_count * output_feature_map_count);
	int workload_id;

	if (dimension_count < 1 || dimension_count > max_dims)
		return;
	for (d = 0; d < dimension_count; ++d)
	{
		sub_sizes[d] = window_sizes[d];
		in_plane *= input_sizes[d];
		out_plane *= output_sizes[d];
	}
	sub_sizes[dimension_count] = feature_map_window;
	sub_sizes[dimension_count + 1] = entry_window;
	sub_count = dimension_count + 2;
	slices[0] = 1;
	for (d = 0; d < sub_count - 1; ++d)
		slices[d + 1] = slices[d] * (d < dimension_count ? input_sizes[d] : input_feature_map_count);
	for (d = 0; d < sub_count; ++d)
		window_elems *= sub_sizes[d];

	offsets = (size_t*)calloc(window_elems, sizeof(size_t));
	positions = (unsigned int*)calloc((size_t)window_elems * max_dims, sizeof(unsigned int));
	{
		unsigned int pos[max_dims + 2];
		unsigned int i;
		memset(pos, 0, sizeof(pos));
		for (i = 1; i < window_elems; ++i)
		{
			for (d = 0; d < sub_count; ++d)
			{
				if (++pos[d] < sub_sizes[d])
					break;
				pos[d] = 0;
			}
			for (d = 0; d < sub_count; ++d)
				offsets[i] += pos[d] * slices[d];
			for (d = 0; d < dimension_count; ++d)
				positions[(size_t)i * max_dims + d] = pos[d];
		}
	}

	#pragma omp parallel for schedule(guided) num_threads(thread_count(threads))
	for (workload_id = 0; workload_id < total_workload; ++workload_id)
	{
		const int out_entry = workload_id / (int)output_feature_map_count;
		const int out_fm = workload_id - out_entry * (int)output_feature_map_count;
		const float* src_base = in
			+ (size_t)out_entry * entry_window * in_plane * input_feature_map_count
			+ (size_t)out_fm * feature_map_window * in_plane;
		float* dst = out + ((size_t)out_entry * output_feature_map_count + out_fm) * out_plane;
		unsigned int out_pos[max_dims];
		size_t o;
		memset(out_pos, 0, sizeof(out_pos));
		for (o = 0; o < out_plane; ++o)
		{
			size_t first = 0;
			float current = is_min ? 1.0e37F : -1.0e37F;
			unsigned int i;
			int dd;
			for (dd = 0; dd < dimension_count; ++dd)
				first += (size_t)out_pos[dd] * strides[dd] * slices[dd];
			for (i = 0; i < window_elems; ++i)
			{
				float new_val;
				if (truncate)
				{
					int inside = 1;
					for (dd = 0; dd < dimension_count; ++dd)
						if (out_pos[dd] * strides[dd] + positions[(size_t)i * max_dims + dd] >= input_sizes[dd])
							inside = 0;
					if (!inside)
						continue;
				}
				new_val = src_base[first + offsets[i]];
				current = is_min ? std_min(current, new_val) : std_max(current, new_val);
			}
			dst[o] = current;
			for (dd = 0; dd < dimension_count; ++dd)
			{
				if (++out_pos[dd] < output_sizes[dd])
					break;
				out_pos[dd] = 0;
			}
		}
	}
	free(offsets);
	free(positions);
}

/*
 * nnforge/plain/max_subsampling_layer_tester_plain.cpp:78-170 (test_tiling): every input entry gives
 * prod(window_sizes) output entries, one per shift of the window grid (shifts in the same x-fastest
 * order as the window scan); output entry e*T + j at position o is the fold over the window that
 * starts at o*window + shift_j. Output sizes are (input - (window - 1)) / window
 * (nnforge/max_subsampling_layer.cpp:119-128).
 */
NNF_ORACLE_API void nnf_oracle_max_subsampling_tiling(float* out, const float* in, unsigned int input_entry_count,
	unsigned int feature_map_count, int dimension_count, const unsigned int* input_sizes, const unsigned int* output_sizes,
	const unsigned int* window_sizes, int is_min, int threads)
{
	enum { max_dims = 6 };
	size_t slices[max_dims];
	size_t in_plane = 1, out_plane = 1;
	unsigned int window_elems = 1;
	size_t* offsets;
	const int total_workload = (int)(input_entry_count * feature_map_count);
	int workload_id, d;

	if (dimension_count < 1 || dimension_count > max_dims)
		return;
	slices[0] = 1;
	for (d = 0; d < dimension_count; ++d)
	{
		if (d + 1 < dimension_count)
			slices[d + 1] = slices[d] * input_sizes[d];
		in_plane *= input_sizes[d];
		out_plane *= output_sizes[d];
		window_elems *= window_sizes[d];
	}
	offsets = (size_t*)calloc(window_elems, sizeof(size_t));
	{
		unsigned int pos[max_dims];
		unsigned int i;
		memset(pos, 0, sizeof(pos));
		for (i = 1; i < window_elems; ++i)
		{
			for (d = 0; d < dimension_count; ++d)
			{
				if (++pos[d] < window_sizes[d])
					break;
				pos[d] = 0;
			}
			for (d = 0; d < dimension_count; ++d)
				offsets[i] += pos[d] * slices[d];
		}
	}
	{
		const size_t output_neuron_count = out_plane * feature_map_count;
		#pragma omp parallel for schedule(guided) num_threads(thread_count(threads))
		for (workload_id = 0; workload_id < total_workload; ++workload_id)
		{
			const int entry_id = workload_id / (int)feature_map_count;
			const int fm = workload_id - entry_id * (int)feature_map_count;
			const float* src_base = in + ((size_t)entry_id * feature_map_count + fm) * in_plane;
			float* dst_base = out + (size_t)entry_id * window_elems * output_neuron_count + (size_t)fm * out_plane;
			unsigned int out_pos[max_dims];
			size_t o;
			memset(out_pos, 0, sizeof(out_pos));
			for (o = 0; o < out_plane; ++o)
			{
				size_t first = 0;
				unsigned int i, j;
				int dd;
				for (dd = 0; dd < dimension_count; ++dd)
					first += (size_t)out_pos[dd] * window_sizes[dd] * slices[dd];
				for (j = 0; j < window_elems; ++j)
				{
					float current = is_min ? 1.0e37F : -1.0e37F;
					for (i = 0; i < window_elems; ++i)
					{
						const float new_val = src_base[first + offsets[j] + offsets[i]];
						current = is_min ? std_min(current, new_val) : std_max(current, new_val);
					}
					dst_base[(size_t)j * output_neuron_count + o] = current;
				}
				for (dd = 0; dd < dimension_count; ++dd)
				{
					if (++out_pos[dd] < output_sizes[dd])
						break;
					out_pos[dd] = 0;
				}
			}
		}
	}
	free(offsets);
}

/* ---- per-feature-map statistics and the batch norm refresh built on them ------------------- */

/* nnforge/stat_data_bunch_writer.h:45-63: the running state of one feature map */
typedef struct nnf_oracle_running_stat
{
	double n;
	double mean;
	double m2;
	float min_val;
	float max_val;
} nnf_oracle_running_stat;

NNF_ORACLE_API void nnf_oracle_feature_map_stat_init(nnf_oracle_running_stat* stats, unsigned int feature_map_count)
{
	unsigned int f;
	for (f = 0; f < feature_map_count; ++f)
	{
		stats[f].n = 0.0;
		stats[f].mean = 0.0;
		stats[f].m2 = 0.0;
		stats[f].min_val = 3.402823466e+38F;  /* std::numeric_limits<float>::max() */
		stats[f].max_val = -3.402823466e+38F;
	}
}

/*
 * nnforge/stat_data_bunch_writer.cpp:45-79, for entry_count entries one after the other: every value
 * of a feature map, in memory order, updates min (std::min(current, val)), max (std::max(current, val))
 * and the single-pass mean / sum of squared deviations in double precision. Feature maps do not
 * interact, so they run in parallel here; each one sees its values in the reference's order.
 */
NNF_ORACLE_API void nnf_oracle_feature_map_stat_write(nnf_oracle_running_stat* stats, const float* data,
	unsigned int entry_count, unsigned int feature_map_count, unsigned int plane, int threads)
{
	int f;
	#pragma omp parallel for schedule(guided) num_threads(thread_count(threads))
	for (f = 0; f < (int)feature_map_count; ++f)
	{
		nnf_oracle_running_stat s = stats[f];
		unsigned int e, i;
		for (e = 0; e < entry_count; ++e)
		{
			const float* src = data + ((size_t)e * feature_map_count + (size_t)f) * plane;
			for (i = 0; i < plane; ++i)
			{
				const float val = src[i];
				double val_d, delta, delta2;
				s.min_val = std_min(s.min_val, val);
				s.max_val = std_max(s.max_val, val);
				s.n += 1.0;
				val_d = (double)val;
				delta = val_d - s.mean;
				s.mean += delta / s.n;
				delta2 = val_d - s.mean;
				s.m2 += delta * delta2;
			}
		}
		stats[f] = s;
	}
}

/* nnforge/stat_data_bunch_writer.cpp:92-106: average = (float)mean, std_dev = sqrtf((float)(m2 / n)) */
NNF_ORACLE_API void nnf_oracle_feature_map_stat_get(const nnf_oracle_running_stat* stats, unsigned int feature_map_count,
	float* min_val, float* max_val, float* average, float* std_dev)
{
	unsigned int f;
	for (f = 0; f < feature_map_count; ++f)
	{
		average[f] = (float)stats[f].mean;
		std_dev[f] = sqrtf((float)(stats[f].m2 / stats[f].n));
		min_val[f] = stats[f].min_val;
		max_val[f] = stats[f].max_val;
	}
}

/*
 * nnforge/toolset.cpp:1608-1617: the statistics were taken on the layer's output with gamma 1 and
 * beta 0, i.e. on (x - mean) * inv_sigma; the new weights make that output have mean 0 and
 * deviation 1:  inv_sigma' = inv_sigma / std_dev,  mean' = mean + average / inv_sigma  (fp32).
 */
NNF_ORACLE_API void nnf_oracle_update_bn_weights(float* mean, float* inverse_sigma, const float* average, const float* std_dev,
	unsigned int feature_map_count)
{
	unsigned int f;
	for (f = 0; f < feature_map_count; ++f)
	{
		const float old_mean = mean[f];
		const float old_invsigma = inverse_sigma[f];
		const float new_invsigma = old_invsigma / std_dev[f];
		const float new_mean = old_mean + average[f] / old_invsigma;
		mean[f] = new_mean;
		inverse_sigma[f] = new_invsigma;
	}
}
