/*
 * nnforge_hip.h - C ABI of the gfx950 (MI355X) inference kernels behind nnForge's layer_tester surface.
 *
 * Every entry point is extern "C", takes plain pointers and sizes, never throws and never
 * synchronises unless its name says so. Return value: 0 = success, > 0 = a hipError_t reported by
 * the HIP runtime, < 0 = one of the NNF_HIP_E* codes below. nnf_hip_error_string() explains both.
 *
 * Tensor layout is nnForge's: fp32, [entry][feature_map][y][x] with x fastest
 * (nnforge/layer_configuration_specific.cpp:62-73); a "plane" is one feature map of one entry,
 * neuron_count_per_feature_map floats long. Device pointers handed to the kernels must be
 * 16-byte aligned at their base (any hipMalloc / nnf_hip_malloc result is). The output may alias
 * inputs[0] exactly (in-place), as every one of the reference testers on this path allows
 * (e.g. nnforge/plain/batch_norm_layer_tester_plain.cpp:77-84); partial overlap is not supported.
 *
 * Arithmetic contract: every layer is evaluated in fp32 with the reference's own operation order
 * and one rounding per operation (no contraction, no reassociation, no cross-layer algebra), so a
 * fused chain produces the same bits as the same layers run one after another.
 */
#ifndef NNFORGE_HIP_H
#define NNFORGE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NNF_HIP_API __attribute__((visibility("default")))

/* ---- error codes (negative; positive values are hipError_t) -------------------------------- */
#define NNF_HIP_OK 0
#define NNF_HIP_EINVAL (-1)      /* null pointer, zero feature maps, malformed descriptor       */
#define NNF_HIP_EUNSUPPORTED (-2) /* shape or option outside what the kernels implement          */
#define NNF_HIP_EALIGN (-3)      /* a tensor base pointer is not 16-byte aligned                 */
#define NNF_HIP_EOVERLAP (-4)    /* output overlaps an input other than "out == inputs[0]"      */
#define NNF_HIP_ETOOBIG (-5)     /* element count does not fit the kernels' index range          */
#define NNF_HIP_ESCRATCH (-6)    /* shape beyond what the library's static scratch array holds   */

/* The kernels index tensors with 32 bits: a tensor (an input, an output) of more elements than this makes
 * an entry point return NNF_HIP_ETOOBIG. Callers that split their work into batches size them to it. */
#define NNF_HIP_MAX_ELEMENT_COUNT 0xFFFF0000ull

#define NNF_HIP_MAX_OPS 8
/* nnf_hip_chain_forward_strided_batch: most groups one kernel launch takes */
#define NNF_HIP_MAX_STRIDED_GROUPS_PER_LAUNCH 6
#define NNF_HIP_MAX_INPUTS 4
/* nnf_hip_chain_forward_batch: most groups one kernel launch takes (what fits into 4 KB of kernel arguments) */
#define NNF_HIP_MAX_GROUPS_PER_LAUNCH 11

/* Layer kinds of the element-wise chain kernel. The names in comments are nnForge's layer type
 * names (the keys of layer_tester_plain_factory, nnforge/plain/layer_tester_plain_factory.cpp:27-51). */
typedef enum nnf_hip_op_kind
{
	NNF_HIP_OP_BATCH_NORM = 1, /* "BatchNorm": mult = gamma*inv_sigma; add = beta - mult*mean; y = x*mult + add
	                              (nnforge/plain/batch_norm_layer_tester_plain.cpp:54-74)                       */
	NNF_HIP_OP_RELU = 2,       /* "ReLU": y = x >= 0 ? x : x*negative_slope
	                              (nnforge/plain/rectified_linear_layer_tester_plain.cpp:50-55)                 */
	NNF_HIP_OP_PRELU = 3,      /* "PReLU": y = x * (x >= 0 ? 1 : a[feature_map])
	                              (nnforge/plain/parametric_rectified_linear_layer_tester_plain.cpp:51-70)      */
	NNF_HIP_OP_ELU = 4,        /* "ELU": y = x >= 0 ? x : expf(x) - 1
	                              (nnforge/plain/exponential_linear_layer_tester_plain.cpp:47-52)               */
	NNF_HIP_OP_SIGMOID = 5,    /* "Sigmoid": y = 1 / (expf(-x) + 1)
	                              (nnforge/plain/sigmoid_layer_tester_plain.cpp:47-53)                          */
	NNF_HIP_OP_TANH = 6,       /* "TanH": e = expf(x * (steepness*2)); y = (e - 1)/(e + 1) * scale
	                              (nnforge/plain/hyperbolic_tangent_layer_tester_plain.cpp:48-58)               */
	NNF_HIP_OP_ABSOLUTE = 7,   /* "Absolute": y = fabs(x) (nnforge/plain/absolute_layer_tester_plain.cpp:43-49)  */
	NNF_HIP_OP_DROPOUT = 8     /* "Dropout" at inference: y = x (nnforge/plain/dropout_layer_tester_plain.cpp:45-48);
	                              costs nothing inside a group                                                  */
} nnf_hip_op_kind;

/* One element-wise layer of a chain. */
typedef struct nnf_hip_op
{
	int32_t kind;   /* nnf_hip_op_kind */
	int32_t chunk;  /* BATCH_NORM: index into chunk_ptrs of gamma; beta, mean, inverse sigma follow at
	                   chunk+1..chunk+3 (chunk order of nnforge/batch_norm_layer.cpp:96-106).
	                   PRELU: index into chunk_ptrs of the per-feature-map slopes
	                   (nnforge/parametric_rectified_linear_layer.cpp:87-94). Others: ignored.        */
	float f0;       /* RELU: negative_slope. TANH: scale. Others: ignored.                           */
	float f1;       /* TANH: steepness. Others: ignored.                                             */
} nnf_hip_op;

/*
 * A fused group of layers evaluated in one pass over the tensor: up to NNF_HIP_MAX_INPUTS input
 * tensors ("arms"), each optionally run through its own element-wise layers, joined by at most one
 * "Add" layer (sum = 0; sum += arm_j in input order; v = sum*alpha -
 * nnforge/plain/add_layer_tester_plain.cpp:54-61), followed by the layers after the join.
 * Without an Add there is exactly one input and arm_op_count[0] + tail_op_count layers applied in order.
 * All tensors share one shape: entry_count x feature_map_count x neuron_count_per_feature_map.
 */
typedef struct nnf_hip_chain_desc
{
	uint32_t entry_count;
	uint32_t feature_map_count;
	uint32_t neuron_count_per_feature_map;
	uint32_t input_count;                       /* 1..NNF_HIP_MAX_INPUTS; > 1 requires has_add      */
	uint32_t has_add;                           /* 0 or 1                                           */
	float add_alpha;                            /* add_layer::alpha (nnforge/add_layer.h:27)        */
	uint32_t arm_op_count[NNF_HIP_MAX_INPUTS];  /* layers applied to input j before the join        */
	uint32_t tail_op_count;                     /* layers applied after the join                    */
	nnf_hip_op ops[NNF_HIP_MAX_OPS];            /* arm 0's layers, arm 1's, ..., then the tail's    */
} nnf_hip_chain_desc;

/* ---- the hot path -------------------------------------------------------------------------- */

/* One environment variable is read by the library, once per process, for profiling launch shapes against each other:
 * NNF_HIP_CHAIN_SHAPE = 0 | 1 | 2 | 3 | 4 makes nnf_hip_chain_forward (and the single-layer entry points built on it) use
 * 256 lanes x 4 float4s, 256 x 2, 256 x 1, 64 x 1 per workgroup, or (4) the grid that stays put, walking over tiles of
 * 256 x 4, instead of choosing by tensor size. A shape that does not fit the call (coefficient tables beyond LDS; 4 with
 * more than one input, with planes that are not float4-aligned or with one of the compile-time expf groups) is ignored.
 * Results do not depend on it. Unset or empty: automatic. */

/* Fused element-wise group. Replaces one run_forward_propagation call per layer of the group
 * (nnforge/plain/forward_propagation_plain.cpp:137-186 calls them one by one). inputs[] holds
 * input_count device pointers in the Add layer's input order; chunk_ptrs[] holds device pointers
 * to the weight chunks the ops refer to (may be null when no op uses a chunk). */
NNF_HIP_API int nnf_hip_chain_forward(void* stream, const nnf_hip_chain_desc* desc, float* output,
	const float* const* inputs, const float* const* chunk_ptrs);

/* group_count fused groups that have nothing to do with each other, in as few launches as possible: groups that share a
 * kernel instance (same number of inputs and same tile size, or any mix of groups with one input and groups with two; at most
 * three layers with weights) go NNF_HIP_MAX_GROUPS_PER_LAUNCH to a launch, whose grid is their tiles one after the other. Same results as group_count calls of nnf_hip_chain_forward with descs[i],
 * outputs[i], inputs[i], chunk_ptrs[i] (chunk_ptrs, or an entry of it, may be null where no layer has weights); what a
 * launch loses while the device fills and drains is paid once per launch instead of once per group. The groups run in
 * no particular order and possibly at the same time: the output of a group may overlap no other group's output or
 * inputs (NNF_HIP_EOVERLAP, nothing launched; within a group output == inputs[0] stays allowed). Every group is checked
 * before the first launch. In the reference the driver loop calls one tester after the other
 * (nnforge/plain/forward_propagation_plain.cpp:137-186); independent actions on separate streams are what
 * nnforge/cuda/forward_propagation_cuda.cpp:414-423 does about it. */
NNF_HIP_API int nnf_hip_chain_forward_batch(void* stream, uint32_t group_count, const nnf_hip_chain_desc* descs,
	float* const* outputs, const float* const* const* inputs, const float* const* const* chunk_ptrs);

/* A fused group whose result is a part of a wider tensor: entry e of the result is written output_entry_stride floats behind
 * entry e - 1 (the inputs are ordinary tensors, entry behind entry). With `output` pointing at the group's feature maps
 * inside the first entry of a Concat layer's output and output_entry_stride that layer's neuron count, the group writes
 * where nnforge/plain/concat_layer_tester_plain.cpp:45-58 would copy its result to, and the copy is not needed. Same bits as
 * nnf_hip_chain_forward followed by that copy. One or two inputs; the neuron count of an entry and the stride must be
 * multiples of 4 (every entry then starts on a 16-byte boundary): NNF_HIP_EUNSUPPORTED otherwise, and
 * nnf_hip_chain_forward_strided_status tells so from the shapes alone. The written range may overlap no input. */
NNF_HIP_API int nnf_hip_chain_forward_strided(void* stream, const nnf_hip_chain_desc* desc, float* output, uint32_t output_entry_stride,
	const float* const* inputs, const float* const* chunk_ptrs);
NNF_HIP_API int nnf_hip_chain_forward_strided_status(const nnf_hip_chain_desc* desc, uint32_t output_entry_stride);
/* group_count such groups over the same number of entries - the branches in front of one Concat layer, say - in one launch per
 * NNF_HIP_MAX_STRIDED_GROUPS_PER_LAUNCH groups. Same results as group_count calls of nnf_hip_chain_forward_strided. What one group
 * writes may touch no input of the call and no other group's result (NNF_HIP_EOVERLAP, nothing launched); results that step
 * alike may lie side by side inside one step, as the parts of one wider tensor do. */
NNF_HIP_API int nnf_hip_chain_forward_strided_batch(void* stream, uint32_t group_count, const nnf_hip_chain_desc* descs,
	float* const* outputs, const uint32_t* output_entry_strides, const float* const* const* inputs, const float* const* const* chunk_ptrs);

/* Single-layer entry points, one per reference tester (same arithmetic as the chain kernel). */
NNF_HIP_API int nnf_hip_batch_norm_forward(void* stream, float* output, const float* input,
	const float* gamma, const float* beta, const float* mean, const float* inverse_sigma,
	uint32_t entry_count, uint32_t feature_map_count, uint32_t neuron_count_per_feature_map);
	/* nnforge/plain/batch_norm_layer_tester_plain.cpp:30-75 */
NNF_HIP_API int nnf_hip_rectified_linear_forward(void* stream, float* output, const float* input,
	float negative_slope, uint64_t elem_count);
	/* nnforge/plain/rectified_linear_layer_tester_plain.cpp:30-56 */
NNF_HIP_API int nnf_hip_parametric_rectified_linear_forward(void* stream, float* output, const float* input,
	const float* slopes, uint32_t entry_count, uint32_t feature_map_count, uint32_t neuron_count_per_feature_map);
	/* nnforge/plain/parametric_rectified_linear_layer_tester_plain.cpp:30-71 */
NNF_HIP_API int nnf_hip_exponential_linear_forward(void* stream, float* output, const float* input, uint64_t elem_count);
	/* nnforge/plain/exponential_linear_layer_tester_plain.cpp:30-53 */
NNF_HIP_API int nnf_hip_sigmoid_forward(void* stream, float* output, const float* input, uint64_t elem_count);
	/* nnforge/plain/sigmoid_layer_tester_plain.cpp:30-54 */
NNF_HIP_API int nnf_hip_hyperbolic_tangent_forward(void* stream, float* output, const float* input,
	float scale, float steepness, uint64_t elem_count);
	/* nnforge/plain/hyperbolic_tangent_layer_tester_plain.cpp:30-59 */
NNF_HIP_API int nnf_hip_add_forward(void* stream, float* output, const float* const* inputs, uint32_t input_count,
	float alpha, uint64_t elem_count);
	/* nnforge/plain/add_layer_tester_plain.cpp:32-62; any input_count >= 1 (launched in groups of
	   NNF_HIP_MAX_INPUTS, which keeps the reference's left-to-right summation order) */

NNF_HIP_API int nnf_hip_absolute_forward(void* stream, float* output, const float* input, uint64_t elem_count);
	/* nnforge/plain/absolute_layer_tester_plain.cpp:30-50 */
NNF_HIP_API int nnf_hip_dropout_forward(void* stream, float* output, const float* input, uint64_t elem_count);
	/* nnforge/plain/dropout_layer_tester_plain.cpp:33-49: the inference pass copies the input; with
	   output == input nothing is launched */

/* Softmax across feature maps at every (entry, spatial position):
 * nnforge/plain/softmax_layer_tester_plain.cpp:34-91 (max, expf(x - max), sum, multiply by 1/sum). */
NNF_HIP_API int nnf_hip_softmax_forward(void* stream, float* output, const float* input,
	uint32_t entry_count, uint32_t feature_map_count, uint32_t neuron_count_per_feature_map);

/* 2-D average subsampling with non-overlapping window_width x window_height windows (output size =
 * input size / window size rounded down; a leftover right/bottom margin is not read,
 * nnforge/average_subsampling_layer.cpp:80-87), window values summed x-fastest then multiplied by mult:
 * nnforge/plain/average_subsampling_layer_tester_plain.cpp:34-148 restricted to two spatial
 * dimensions, no feature-map/entry subsampling. The caller passes the multiplier the tester would
 * use (average_subsampling_layer::get_effective_alpha, nnforge/average_subsampling_layer.cpp:287-303). */
NNF_HIP_API int nnf_hip_average_subsampling_forward(void* stream, float* output, const float* input,
	uint32_t entry_count, uint32_t feature_map_count, uint32_t input_width, uint32_t input_height,
	uint32_t window_width, uint32_t window_height, float mult);

/* Concatenation along feature maps: per entry the neurons of input 0, then of input 1, ...
 * (nnforge/plain/concat_layer_tester_plain.cpp:33-59). input_neuron_counts[i] = feature maps * neurons
 * per feature map of input i. */
NNF_HIP_API int nnf_hip_concat_forward(void* stream, float* output, const float* const* inputs,
	const uint32_t* input_neuron_counts, uint32_t input_count, uint32_t entry_count);
/* The same with some inputs already where they belong: input i with inputs_in_place[i] != 0 was written into its part of
 * `output` by whoever made it (nnf_hip_chain_forward_strided) and is not copied - its pointer is not looked at; the others
 * are copied to their parts as above. With every input in place nothing is launched. */
NNF_HIP_API int nnf_hip_concat_forward_partial(void* stream, float* output, const float* const* inputs,
	const uint32_t* input_neuron_counts, const uint8_t* inputs_in_place, uint32_t input_count, uint32_t entry_count);

/* Maxout: output feature map o = maximum over the input feature maps o, o + output_feature_map_count,
 * o + 2*output_feature_map_count, ... (feature_map_subsampling_size of them), folded with
 * std::max(new, current) from the first value on (nnforge/plain/maxout_layer_tester_plain.cpp:33-81). */
NNF_HIP_API int nnf_hip_maxout_forward(void* stream, float* output, const float* input,
	uint32_t entry_count, uint32_t output_feature_map_count, uint32_t neuron_count_per_feature_map,
	uint32_t feature_map_subsampling_size);

/* Max (or min) subsampling without tiling: windows of subsampling_sizes[d] every strides[d] elements
 * (strides null: the window sizes) in up to NNF_HIP_MAX_SUBSAMPLING_DIMENSIONS spatial dimensions
 * (x first), then over feature_map_subsampling_size neighbouring feature maps and
 * entry_subsampling_size neighbouring entries; the fold starts at -1.0e37F (1.0e37F for min) and scans
 * the window x fastest with std::max<float>(current, new)
 * (nnforge/plain/max_subsampling_layer_tester_plain.cpp:175-290). Output size per dimension:
 * (input + stride - window + (round_up ? window - 1 : 0)) / stride
 * (nnforge/max_subsampling_layer.cpp:131-141); with round_ups[d] != 0 the part of a window beyond the
 * input is skipped (nnforge/cuda/max_subsampling_layer_tester_cuda.cuh:97-116; the plain tester
 * refuses round up). The input holds output_entry_count * entry_subsampling_size entries. The tiling
 * variant of the layer is nnf_hip_max_subsampling_tiling_forward. */
#define NNF_HIP_MAX_SUBSAMPLING_DIMENSIONS 4
NNF_HIP_API int nnf_hip_max_subsampling_forward(void* stream, float* output, const float* input,
	uint32_t output_entry_count, uint32_t input_feature_map_count, uint32_t dimension_count,
	const uint32_t* input_sizes, const uint32_t* subsampling_sizes, const uint32_t* strides, const uint32_t* round_ups,
	uint32_t feature_map_subsampling_size, uint32_t entry_subsampling_size, int32_t is_min);

/* Max (or min) subsampling with tiling (nnforge/plain/max_subsampling_layer_tester_plain.cpp:78-170):
 * windows of subsampling_sizes[d] every subsampling_sizes[d] elements, computed once per shift of the
 * window grid by 0 .. subsampling_sizes[d] - 1 elements in every dimension. Input entry e gives the output
 * entries e * T + j, T = product of the window sizes, j = the shifts taken together x fastest; each holds
 * feature_map_count feature maps of (input_sizes[d] - (subsampling_sizes[d] - 1)) / subsampling_sizes[d]
 * elements per dimension (nnforge/max_subsampling_layer.cpp:113-121; input sizes below
 * 2 * subsampling size - 1 are refused). The fold is that of nnf_hip_max_subsampling_forward. */
NNF_HIP_API int nnf_hip_max_subsampling_tiling_forward(void* stream, float* output, const float* input,
	uint32_t input_entry_count, uint32_t feature_map_count, uint32_t dimension_count,
	const uint32_t* input_sizes, const uint32_t* subsampling_sizes, int32_t is_min);

/* Average subsampling in the reference's full form: 1 to NNF_HIP_MAX_SUBSAMPLING_DIMENSIONS spatial
 * dimensions (input_sizes / subsampling_sizes: x first), windows over feature maps and over entries
 * (output feature maps = input_feature_map_count / feature_map_subsampling_size; the input holds
 * output_entry_count * entry_subsampling_size entries). Every output is the left-to-right fp32 sum of its
 * window - x fastest, then the further dimensions, then feature maps, then entries - times mult:
 * nnforge/plain/average_subsampling_layer_tester_plain.cpp:34-148. Output size per dimension = input size /
 * window size rounded down (nnforge/average_subsampling_layer.cpp:80-87). 1-D and 2-D windows within a
 * feature map take the kernels of nnf_hip_average_subsampling_forward. */
NNF_HIP_API int nnf_hip_average_subsampling_nd_forward(void* stream, float* output, const float* input,
	uint32_t output_entry_count, uint32_t input_feature_map_count, uint32_t dimension_count,
	const uint32_t* input_sizes, const uint32_t* subsampling_sizes,
	uint32_t feature_map_subsampling_size, uint32_t entry_subsampling_size, float mult);

/* Subsampling with the element-wise layers in front of it folded in: `prologue` describes a
 * single-input group without Add (input_count 1, has_add 0; its arm 0 and tail layers are applied in
 * order; its feature_map_count and neuron_count_per_feature_map must be the subsampling input's) whose
 * result feeds the subsampling layer and nothing else. The layers are applied to the input values on
 * their way into the workgroup's staging buffer, so the group's result - what
 * nnforge/plain/forward_propagation_plain.cpp:137-186 would store between the two testers - is never
 * written to memory; the output carries the same bits as the layers run one after another. Other
 * arguments as for nnf_hip_max_subsampling_forward / nnf_hip_average_subsampling_forward. Only the
 * LDS-staged kernels (2-D windows, whole-plane averages) apply a prologue: NNF_HIP_EUNSUPPORTED
 * (nothing launched) for windows over feature maps or entries, more than two spatial dimensions,
 * planes of fewer than four floats, more than 65535 outputs per plane, and groups with more than two
 * layers that carry weights (batch norm, PReLU). The *_fusable functions answer that from the shapes
 * alone (NNF_HIP_OK / NNF_HIP_EUNSUPPORTED; no device needed). */
NNF_HIP_API int nnf_hip_max_subsampling_fused_forward(void* stream, float* output, const float* input,
	const nnf_hip_chain_desc* prologue, const float* const* chunk_ptrs,
	uint32_t output_entry_count, uint32_t input_feature_map_count, uint32_t dimension_count,
	const uint32_t* input_sizes, const uint32_t* subsampling_sizes, const uint32_t* strides, const uint32_t* round_ups,
	uint32_t feature_map_subsampling_size, uint32_t entry_subsampling_size, int32_t is_min);
NNF_HIP_API int nnf_hip_average_subsampling_fused_forward(void* stream, float* output, const float* input,
	const nnf_hip_chain_desc* prologue, const float* const* chunk_ptrs,
	uint32_t entry_count, uint32_t feature_map_count, uint32_t input_width, uint32_t input_height,
	uint32_t window_width, uint32_t window_height, float mult);
NNF_HIP_API int nnf_hip_max_subsampling_fusable(uint32_t output_entry_count, uint32_t input_feature_map_count, uint32_t dimension_count,
	const uint32_t* input_sizes, const uint32_t* subsampling_sizes, const uint32_t* strides, const uint32_t* round_ups,
	uint32_t feature_map_subsampling_size, uint32_t entry_subsampling_size);
NNF_HIP_API int nnf_hip_average_subsampling_fusable(uint32_t entry_count, uint32_t feature_map_count, uint32_t input_width, uint32_t input_height,
	uint32_t window_width, uint32_t window_height);

/* The same for a group of two inputs joined by an Add (input_count 2, has_add 1: each input's own layers,
 * the sum times add_alpha as in nnforge/plain/add_layer_tester_plain.cpp:56-59, the tail layers) in front of
 * an average over whole planes - the last block of a residual network in front of its global average
 * (examples/imagenet/imagenet_toolset.cpp:518-522, 815-826): inputs[0] and inputs[1] have the shape of the
 * subsampling input, neither the sum nor the group's result is ever stored, and the output carries the bits
 * of the layers run one after another. NNF_HIP_EUNSUPPORTED for windows smaller than the plane, planes of
 * fewer than 4 or more than 240 floats and groups with more than two layers that carry weights;
 * nnf_hip_average_subsampling_joinable answers that from the shapes alone. */
NNF_HIP_API int nnf_hip_average_subsampling_joined_forward(void* stream, float* output, const float* const* inputs,
	const nnf_hip_chain_desc* prologue, const float* const* chunk_ptrs,
	uint32_t entry_count, uint32_t feature_map_count, uint32_t input_width, uint32_t input_height,
	uint32_t window_width, uint32_t window_height, float mult);
NNF_HIP_API int nnf_hip_average_subsampling_joinable(uint32_t entry_count, uint32_t feature_map_count, uint32_t input_width, uint32_t input_height,
	uint32_t window_width, uint32_t window_height);

/* Per-feature-map running statistics on the device: the state stat_data_bunch_writer keeps per
 * feature map (nnforge/stat_data_bunch_writer.h:45-63) and fills on the host from outputs copied
 * back (nnforge/stat_data_bunch_writer.cpp:45-79). average = (float)mean and
 * std_dev = sqrtf((float)(m2 / n)) as in nnforge/stat_data_bunch_writer.cpp:97-98. The reference
 * updates the state one value at a time; the device reduces runs of entries and merges them in a
 * fixed order, all in double precision: mean and m2 agree with the sequential update to double
 * rounding (at most one fp32 unit in the last place after the conversion), min and max compare
 * equal. Used to refresh batch norm weights (nnforge/toolset.cpp:1562-1630). */
typedef struct nnf_hip_running_stat
{
	double n;
	double mean;
	double m2;       /* sum of squared deviations from the mean */
	float min_val;
	float max_val;
} nnf_hip_running_stat;

/* n = 0, mean = 0, m2 = 0, min = FLT_MAX, max = -FLT_MAX for feature_map_count states (device memory) */
NNF_HIP_API int nnf_hip_feature_map_stat_init(void* stream, nnf_hip_running_stat* device_stats, uint32_t feature_map_count);
/* device workspace (partial states of the runs of entries the reduction is cut into) that lets an accumulate
 * call of entry_count entries use the launch shape it prefers. A workspace of this size also serves every call
 * with fewer entries: accumulate plans its runs inside the workspace it is given. */
NNF_HIP_API int nnf_hip_feature_map_stat_workspace_bytes(uint32_t entry_count, uint32_t feature_map_count,
	uint32_t neuron_count_per_feature_map, size_t* bytes);
/* number of partial states (32 bytes each) an accumulate call of entry_count entries would write into a
 * workspace of workspace_bytes; NNF_HIP_EINVAL when no launch shape fits that workspace. No device needed. */
NNF_HIP_API int nnf_hip_feature_map_stat_partial_count(uint32_t entry_count, uint32_t feature_map_count,
	uint32_t neuron_count_per_feature_map, size_t workspace_bytes, uint32_t* partial_states);
/* folds entry_count entries of input ([entry][feature_map][neurons]) into device_stats; NNF_HIP_EINVAL when the
 * workspace is too small for any launch shape (it never is when sized by nnf_hip_feature_map_stat_workspace_bytes
 * for this or a larger entry count) */
NNF_HIP_API int nnf_hip_feature_map_stat_accumulate(void* stream, nnf_hip_running_stat* device_stats,
	void* device_workspace, size_t workspace_bytes, const float* input,
	uint32_t entry_count, uint32_t feature_map_count, uint32_t neuron_count_per_feature_map);

/* nnf_hip_feature_map_stat_accumulate for callers that cannot allocate device memory and so have no workspace to
 * pass: code that records a HIP graph, tight serving loops, harnesses that forbid hipMalloc. No counterpart in the
 * reference. Same kernels and same results as nnf_hip_feature_map_stat_accumulate; the partial states go into a
 * fixed array of NNF_HIP_STAT_STATIC_SCRATCH_BYTES inside the library's device image (each GPU the library runs on
 * holds its own copy until the process ends), whose address is looked up once per device: by
 * nnf_hip_feature_map_stat_init, else by the first call here, in both cases for the device that is current, which
 * must be the stream's. The call itself allocates nothing and frees nothing. Limit:
 * NNF_HIP_STAT_STATIC_SCRATCH_BYTES / 32 = 8192 partial states, one per feature map and run of entries. The runs
 * are planned inside that limit; a shape is refused (NNF_HIP_ESCRATCH, nothing launched) only when even the longest
 * runs the kernels' index arithmetic allows leave more states than that: more than 8192 feature maps, or planes of
 * u loads (u = neuron_count_per_feature_map / 4, or neuron_count_per_feature_map when that is no multiple of 4) with
 * feature_map_count * ceil(entry_count / max(1, floor((2^32 - 1) / u^2))) > 8192. All calls on one GPU share the
 * array: calls that can overlap (different streams, different threads) race on it and must be ordered by the
 * caller; nothing in it has to be cleared between calls (the first launch writes every state the second reads). */
#define NNF_HIP_STAT_STATIC_SCRATCH_BYTES 262144
NNF_HIP_API int nnf_hip_feature_map_stat_accumulate_static(void* stream, nnf_hip_running_stat* device_stats,
	const float* input, uint32_t entry_count, uint32_t feature_map_count, uint32_t neuron_count_per_feature_map);

/* ---- runtime plumbing, so that host C++ above this ABI needs no HIP headers --------------------
 * Counterparts in the reference: cuda_linear_buffer_device (nnforge/cuda/cuda_linear_buffer_device.cpp:28-45),
 * cuda_stream / cuda_event (nnforge/cuda/cuda_stream.cpp, cuda_event.cpp), cuda_safe_call
 * (nnforge/cuda/neural_network_cuda_exception.h:27-39). */
NNF_HIP_API int nnf_hip_device_count(int* count);
NNF_HIP_API int nnf_hip_set_device(int device_id);
NNF_HIP_API int nnf_hip_device_info(int device_id, char* name, size_t name_capacity, uint64_t* global_memory_bytes,
	uint32_t* compute_unit_count, uint32_t* wavefront_size, uint32_t* clock_khz);
NNF_HIP_API int nnf_hip_malloc(void** device_ptr, size_t bytes); /* size rounded up to 16 bytes, like
	the reference's device buffers (nnforge/cuda/util_cuda.cu:731-735) */
NNF_HIP_API int nnf_hip_free(void* device_ptr);
NNF_HIP_API int nnf_hip_memcpy_h2d(void* device_dst, const void* host_src, size_t bytes, void* stream); /* stream null: synchronous */
NNF_HIP_API int nnf_hip_memcpy_d2h(void* host_dst, const void* device_src, size_t bytes, void* stream);
NNF_HIP_API int nnf_hip_memcpy_d2d(void* device_dst, const void* device_src, size_t bytes, void* stream);
NNF_HIP_API int nnf_hip_host_malloc(void** host_ptr, size_t bytes); /* pinned */
NNF_HIP_API int nnf_hip_host_free(void* host_ptr);
NNF_HIP_API int nnf_hip_stream_create(void** stream);
NNF_HIP_API int nnf_hip_stream_destroy(void* stream);
NNF_HIP_API int nnf_hip_stream_synchronize(void* stream);
NNF_HIP_API int nnf_hip_device_synchronize(void);
NNF_HIP_API int nnf_hip_event_create(void** event);
NNF_HIP_API int nnf_hip_event_destroy(void* event);
NNF_HIP_API int nnf_hip_event_record(void* event, void* stream);
NNF_HIP_API int nnf_hip_event_synchronize(void* event);
NNF_HIP_API int nnf_hip_event_elapsed_ms(float* milliseconds, void* start_event, void* stop_event);
NNF_HIP_API int nnf_hip_stream_wait_event(void* stream, void* event);
/* A recorded sequence of launches (a HIP graph): what is enqueued on `stream` between begin and end is recorded instead
 * of run (kernel launches only: no memory is set or copied by this library's entry points), end hands back an executable
 * graph that nnf_hip_graph_launch replays on a stream. The pointers and sizes of the recorded launches are fixed. */
NNF_HIP_API int nnf_hip_stream_begin_capture(void* stream);
NNF_HIP_API int nnf_hip_stream_end_capture(void* stream, void** graph_exec);
NNF_HIP_API int nnf_hip_graph_launch(void* graph_exec, void* stream);
NNF_HIP_API int nnf_hip_graph_destroy(void* graph_exec);

/* Plain device-to-device streaming copy kernel (float4 loads and stores, same launch shape as the
 * chain kernel). Used as the yardstick for achievable HBM bandwidth and for scaling profiler
 * counters; no counterpart in the reference. bytes must be a multiple of 16. */
NNF_HIP_API int nnf_hip_copy_kernel(void* stream, void* device_dst, const void* device_src, size_t bytes);

/* Self-check of the two short division sequences the Sigmoid and TanH kernels use in place of the
 * general IEEE division (reciprocal estimate + one Newton step for 1/(e + 1); quotient, exact
 * remainder, one correction for (e - 1)/(e + 1)): enqueues a sweep over every non-negative float e with
 * e + 1 <= 2^126 and adds the number of results that differ in bits from IEEE division to
 * device_mismatch_counts[0] (reciprocal) and [1] (quotient), two counters in device memory that the
 * caller has zeroed. Both must stay 0: the bit parity of nnforge/plain/sigmoid_layer_tester_plain.cpp:51
 * and nnforge/plain/hyperbolic_tangent_layer_tester_plain.cpp:55-56 rests on it. */
NNF_HIP_API int nnf_hip_check_division_sequences(void* stream, uint64_t* device_mismatch_counts);

/* Kernels the library has launched from the calling thread since it was loaded. The driver reads it on both sides of a
 * pass of its plan to report how many launches a pass is (a call that takes several groups decides by itself how many
 * kernels they share). No counterpart in the reference. */
NNF_HIP_API int nnf_hip_launch_count(uint64_t* count);

NNF_HIP_API const char* nnf_hip_error_string(int code);
NNF_HIP_API const char* nnf_hip_version(void);

#ifdef __cplusplus
}
#endif

#endif /* NNFORGE_HIP_H */
