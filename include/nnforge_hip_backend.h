/*
 * nnforge_hip_backend.h - C bridge over the C++ hip backend (include/nnforge_hip/hip_backend.h) for
 * callers without a C++ toolchain: run a text-format nnForge schema on host arrays through
 * factory_generator_hip -> forward_propagation_hip, or only plan it. The tests and tools drive the
 * backend through this bridge; a C++ application uses the classes directly, as it would use
 * nnForge's plain or cuda backend (examples/gtsrb/gtsrb.cpp:29-63 shows the reference's pattern).
 *
 * Return value: 0 = success; non-zero = failure, with the exception text in `report`.
 */
#ifndef NNFORGE_HIP_BACKEND_H
#define NNFORGE_HIP_BACKEND_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NNF_BACKEND_API __attribute__((visibility("default")))

typedef struct nnf_backend_weights
{
	const char* layer_name;
	uint32_t chunk_count;
	const uint32_t* chunk_sizes;   /* floats per chunk */
	const float* const* chunks;
} nnf_backend_weights;

typedef struct nnf_backend_input
{
	const char* layer_name;        /* a data layer of the schema */
	uint32_t feature_map_count;
	uint32_t dimension_count;
	const uint32_t* dimension_sizes; /* x first */
	const float* data;             /* entry_count entries back to back; may be null when only planning */
} nnf_backend_input;

typedef struct nnf_backend_output
{
	const char* layer_name;
	float* data;                   /* receives entry_count entries */
	size_t capacity_floats;
	size_t written_floats;         /* set by the call */
} nnf_backend_output;

/* struct_size: sizeof(nnf_backend_options) as the caller's header declares it. The library reads that many bytes and
 * takes the members added since as zero (each member's default), so a caller built against an older header keeps
 * working; a size of zero is refused. Zero the structure, set struct_size, then the members wanted. */
typedef struct nnf_backend_options
{
	uint32_t struct_size;
	int32_t fuse;                  /* hip_fuse */
	int32_t dont_share_buffers;    /* hip_dont_share_buffers */
	int32_t max_entry_count;       /* hip_max_entry_count; <= 0: default */
	int32_t profile;               /* per-launch times in the report */
	int32_t weights_from_folder;   /* 1: `weights_folder` holds <layer>.data files */
	const char* weights_folder;
	const char* profile_folder;    /* with profile: folder for forward_prop_perf_per_layer_action_NNN.csv; null: no file */
	int32_t stat_on_host;          /* nnf_backend_layer_statistics: copy the outputs back and update the statistics
	                                  value by value on the host, as the reference does, instead of reducing on the device */
	int32_t kernel_stream_count;   /* hip_kernel_stream_count; 1 = hip_single_command_stream; <= 0: default */
	int32_t one_launch_per_group;  /* 1: hip_batch_independent_groups off (every fused group gets a launch of its own) */
	int32_t host_thread_count;     /* threads that read input entries (sets hip_reserved_thread_count to the processors beyond
	                                  them; at most 16 are used); <= 0: default, all processors but one */
	int32_t max_io_staging_mb;     /* hip_max_io_staging_mb: pinned staging (input + output entries) per I/O slot that bounds a
	                                  packet of run(); 0: default (64), < 0: no bound */
	int32_t resident_packets;      /* nnf_backend_time_kernels: sets of data / output buffers the timed passes go round; <= 0: 1 */
	int32_t concat_copies_every_input; /* 1: hip_concat_in_place off (every Concat layer copies all its inputs; by default fused groups
	                                  that only a Concat reads write their results into its output) */
	int32_t replay_recorded_plan;  /* nnf_backend_time_kernels: 1: the launches of a pass are recorded once as a HIP graph and the
	                                  timed passes replay it (one kernel stream) */
	int32_t keep_unregistered_layers; /* 1: a layer of a type this backend has no class for (Convolution, LCS, LError ...) does not
	                                  make the schema an error: it is kept as it stands in the file and computes nothing - its
	                                  output comes in as an input under the layer's own name, with the configuration given for
	                                  it, and what only such layers read is neither wanted nor computed. 0: such a type is an
	                                  error ("No layer is registered with type ..."), as in the reference */
} nnf_backend_options;

/* Runs the schema on device 0. The report lists one line per launch ("step: ..."), the buffer plan
 * and, with profile, per-launch seconds. */
NNF_BACKEND_API int nnf_backend_run_schema(
	const char* schema_text,
	const nnf_backend_weights* weights, uint32_t weights_count,
	const nnf_backend_input* inputs, uint32_t input_count,
	uint32_t entry_count,
	nnf_backend_output* outputs, uint32_t output_count,
	const nnf_backend_options* options,
	char* report, size_t report_capacity);

/* Statistics of one layer's output over entry_count entries (forward_propagation::run into a
 * stat_data_bunch_writer): minimum, maximum, average and standard deviation per feature map, each
 * array feature_map_count floats long. */
/* A data set file of nnForge (".dt": nnforge/structured_data_stream_reader.cpp:28-61) and the layer it belongs to. */
typedef struct nnf_backend_dataset_file
{
	const char* layer_name;
	const char* path;
} nnf_backend_dataset_file;

/* Inference from data set files to data set files, one network, the way toolset::run_inference does it in its
 * dump mode (nnforge/toolset.cpp:551-655): a file per data layer goes in through structured_data_bunch_stream_reader
 * (a data layer named dataset_value reads the constant 1), the outputs are collected by
 * neuron_value_set_data_bunch_writer, every compact_samples consecutive entries of an output are replaced by their
 * mean (0 or 1: none; the entries a tiling layer made of one input entry), and each output layer is written to its
 * file. The report lists the outputs, the launch plan and the run's statistics. */
NNF_BACKEND_API int nnf_backend_run_dataset(
	const char* schema_text,
	const nnf_backend_weights* weights, uint32_t weights_count,
	const nnf_backend_dataset_file* inputs, uint32_t input_count,
	const nnf_backend_dataset_file* outputs, uint32_t output_count,
	uint32_t compact_samples,
	const nnf_backend_options* options,
	char* report, size_t report_capacity);

/* Host only: reads part `part` of `part_count` equal parts of a data set file through the same readers (part_count 0 or
 * 1: the whole file), folds every compact_samples consecutive entries into their mean and writes the result as a data
 * set file. The report holds the configuration, the entry counts and the per-neuron average of what was read. */
NNF_BACKEND_API int nnf_backend_rewrite_dataset(const char* in_path, const char* out_path, uint32_t compact_samples,
	uint32_t part_count, uint32_t part, char* report, size_t report_capacity);

NNF_BACKEND_API int nnf_backend_layer_statistics(
	const char* schema_text,
	const nnf_backend_weights* weights, uint32_t weights_count,
	const nnf_backend_input* inputs, uint32_t input_count,
	uint32_t entry_count,
	const char* layer_name, uint32_t feature_map_count,
	float* min_values, float* max_values, float* averages, float* std_devs,
	const nnf_backend_options* options,
	char* report, size_t report_capacity);

/* toolset::update_bn_weights (nnforge/toolset.cpp:1562-1630) on in-memory data: refreshes mean and
 * inverse sigma of every BatchNorm layer from the inputs' statistics and writes all weights to
 * out_folder as <layer>.data files. The report holds the lines the reference prints. */
NNF_BACKEND_API int nnf_backend_update_bn_weights(
	const char* schema_text,
	const nnf_backend_weights* weights, uint32_t weights_count,
	const nnf_backend_input* inputs, uint32_t input_count,
	uint32_t entry_count,
	const nnf_backend_options* options,
	const char* out_folder,
	char* report, size_t report_capacity);

/* Times the launch plan of the schema alone, on one packet of entry_count entries that stays in device memory
 * (forward_propagation_hip::time_kernels): uploaded once, then `warmup` untimed and `passes` timed runs of the plan,
 * nothing copied back. With options->resident_packets = R > 1 the data and output layers have R sets of device buffers and
 * the passes go round them (a small network then reads memory, not the last-level cache). The report lists the plan like
 * nnf_backend_run_schema, then "launches: N" (kernels one pass launches), "plan_steps: N" (steps of the plan that launch
 * something; steps handed to the kernels together share launches), "resident_packets: R", "timed_entries: N",
 * "wall_seconds_per_pass: S" (device synchronisation on both sides of the timed passes),
 * "device_seconds_per_pass: S" (events on the kernel stream) and "host_seconds_per_pass: S" (what the calling thread
 * spends enqueuing a pass while the device runs behind it). Inputs whose data pointers are equal are fine: the
 * values do not matter for the time. */
NNF_BACKEND_API int nnf_backend_time_kernels(
	const char* schema_text,
	const nnf_backend_weights* weights, uint32_t weights_count,
	const nnf_backend_input* inputs, uint32_t input_count,
	uint32_t entry_count,
	const char* const* output_layer_names, uint32_t output_count,
	const nnf_backend_options* options,
	uint32_t warmup, uint32_t passes,
	char* report, size_t report_capacity);

/* Plans launches and buffers without touching a device (works on a machine without a GPU).
 * memory_bytes: the device memory to plan for. */
NNF_BACKEND_API int nnf_backend_plan_schema(
	const char* schema_text,
	const nnf_backend_input* inputs, uint32_t input_count,
	const char* const* output_layer_names, uint32_t output_count,
	const nnf_backend_options* options,
	uint64_t memory_bytes,
	char* report, size_t report_capacity);

/* Parses a schema and writes it back in text format (round trip of the reader/writer). A buffer too
 * small for the whole text is an error (the message says how many bytes are needed). keep_unregistered_layers: as in
 * nnf_backend_options; the layers kept that way are written back with the parameter messages they were read with. */
NNF_BACKEND_API int nnf_backend_rewrite_schema(const char* schema_text, int32_t keep_unregistered_layers, char* out_text, size_t out_capacity);

/* Parses a schema and lists its layers in forward propagation order, a line each:
 * "layer: <type>\t<name>\t<input names, comma separated>\t<the layer's parameter strings, joined by '; '>\t<own|external>". */
NNF_BACKEND_API int nnf_backend_list_layers(const char* schema_text, int32_t keep_unregistered_layers, char* report, size_t report_capacity);

/* Writes / reads <layer>.data files in nnForge's format (weights in, weights out through `weights`
 * arrays owned by the caller; reading fills caller-provided chunks and checks their sizes). */
NNF_BACKEND_API int nnf_backend_write_weights(const char* folder, const nnf_backend_weights* weights, uint32_t weights_count, char* report, size_t report_capacity);
NNF_BACKEND_API int nnf_backend_read_weights(const char* folder, const char* layer_name, uint32_t chunk_count, const uint32_t* chunk_sizes, float* const* chunks, char* report, size_t report_capacity);

#ifdef __cplusplus
}
#endif

#endif /* NNFORGE_HIP_BACKEND_H */
