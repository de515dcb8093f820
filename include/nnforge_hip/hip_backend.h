// The "hip" backend: a sibling of nnForge's plain and cuda backends for MI355X. It provides
// layer_tester objects per layer type, chosen by type name, and a forward_propagation
// implementation that fuses runs of element-wise layers into single kernel launches.
// Everything device-side goes through the C ABI of include/nnforge_hip.h; this header needs no
// HIP headers.
#pragma once

#include "core.h"
#include "layers.h"
#include "propagation.h"
#include "schema.h"
#include "../nnforge_hip.h"

#include <iosfwd>
#include <map>
#include <string>
#include <vector>

namespace nnforge
{
	namespace hip
	{
		// Failure of a C-ABI / HIP runtime call (nnforge/cuda/neural_network_cuda_exception.h:27-39)
		class neural_network_hip_exception : public neural_network_exception
		{
		public:
			neural_network_hip_exception(int error_code, const char * filename, int line_number);
			int error_code;
		};

		void hip_check(int code, const char * filename, int line_number);
		#define hip_safe_call(callstr) ::nnforge::hip::hip_check((callstr), __FILE__, __LINE__)

		// Device allocation owned by the object (nnforge/cuda/cuda_linear_buffer_device.h); sizes are
		// rounded up to 16 bytes by the allocator.
		class hip_linear_buffer_device
		{
		public:
			typedef std::shared_ptr<hip_linear_buffer_device> ptr;
			typedef std::shared_ptr<const hip_linear_buffer_device> const_ptr;

			explicit hip_linear_buffer_device(size_t size);
			~hip_linear_buffer_device();
			operator void *() { return buf; }
			operator const void *() const { return buf; }
			operator float *() { return static_cast<float *>(buf); }
			operator const float *() const { return static_cast<const float *>(buf); }
			size_t get_size() const { return size; }

		private:
			hip_linear_buffer_device(const hip_linear_buffer_device&) = delete;
			hip_linear_buffer_device& operator =(const hip_linear_buffer_device&) = delete;
			void * buf;
			size_t size;
		};

		// Device selection and memory budget (nnforge/cuda/cuda_running_configuration.h)
		class hip_running_configuration
		{
		public:
			typedef std::shared_ptr<const hip_running_configuration> const_ptr;

			// queries the device (throws when there is none)
			hip_running_configuration(int device_id, float max_global_memory_usage_ratio, bool fuse_layers, bool dont_share_buffers, int max_entry_count,
				int kernel_stream_count = default_kernel_stream_count, bool batch_independent_groups = true, unsigned int reserved_thread_count = 1);
			// A configuration that never touches a device: for planning launches and buffers (and testing
			// that logic) on a machine without a GPU. Running a network with it throws.
			static std::shared_ptr<const hip_running_configuration> create_offline(
				unsigned long long global_memory_size, float max_global_memory_usage_ratio, bool fuse_layers, bool dont_share_buffers, int max_entry_count,
				int kernel_stream_count = default_kernel_stream_count, bool batch_independent_groups = true);
			bool is_offline() const { return offline; }
			void set_device() const;
			size_t get_max_bytes() const;
			// The threads that read input entries, one job per entry, while the thread that called run() hands the packet
			// before to the writer (nnforge/cuda/cuda_multi_running_configuration.h:55, .cpp:96-97): as many as the
			// process has processors, less reserved_thread_count, at least 1 and at most max_job_thread_count (reading
			// entries is copying: beyond that the host's memory is the limit, not its cores). None when offline.
			threadpool_job_runner::ptr get_job_runner() const { return job_runner; }
			static constexpr unsigned int max_job_thread_count = 16;

			int device_id;
			float max_global_memory_usage_ratio;
			bool fuse_layers;
			bool dont_share_buffers;
			int max_entry_count;
			// Streams the kernels of a packet are spread over: steps that do not depend on each other overlap the
			// start of one with the end of another. Measured with 51 independent one-read-one-write launches of the
			// sizes of the ResNet-50 post-convolution stack: 64 entries 894 us on one stream, 835 on two, 828 on three;
			// 8 entries 198, 146, 139 us.
			static constexpr int default_kernel_stream_count = 3;
			int kernel_stream_count;
			// Runs of consecutive fused groups that do not depend on each other go to the kernels in one call, eleven
			// groups to a launch, and the steps are ordered so that these runs are few and of about one size; such runs
			// take one kernel stream (kernel_stream_count then plays no part). Measured
			// on the 49 groups of the ResNet-50 post-convolution stack, all in one call: 64 entries 1091 -> 1042 us,
			// 8 entries 243 -> 172 us.
			bool batch_independent_groups;
			// A fused group that only a Concat layer reads writes its result into that layer's output instead of a
			// tensor of its own that the Concat would copy (four branches of 64 + 128 + 32 + 32 maps of 28 x 28 at 128 entries:
			// 37 us against 75 us); switch off to have every Concat copy
			bool concat_in_place = true;
			unsigned int reserved_thread_count;
			// run() makes its packets no larger than this much pinned staging (input + output entries) per I/O slot, so that
			// reading, copying, computing and writing of neighbouring packets overlap; 0: no bound. It never pushes a
			// packet under min_packet_entries_under_staging_bound entries (a network with many or large data layers would
			// otherwise run its plan entry by entry).
			size_t max_io_staging_bytes = static_cast<size_t>(64) << 20;
			static constexpr unsigned int min_packet_entries_under_staging_bound = 8;
			std::string device_name;
			unsigned long long global_memory_size;
			unsigned int compute_unit_count;
			unsigned int wavefront_size;
			unsigned int clock_khz;

		private:
			hip_running_configuration() = default;
			bool offline = false;
			threadpool_job_runner::ptr job_runner;
		};

		std::ostream& operator<<(std::ostream& out, const hip_running_configuration& config);

		// Per layer instance object that enqueues the layer's forward pass on a stream
		// (the contract of nnforge/cuda/layer_tester_cuda.h:34-96).
		class layer_tester_hip
		{
		public:
			typedef std::shared_ptr<layer_tester_hip> ptr;

			virtual ~layer_tester_hip() = default;

			void configure(
				const std::vector<layer_configuration_specific>& input_configuration_specific_list,
				const layer_configuration_specific& output_configuration_specific,
				layer::const_ptr layer_schema,
				hip_running_configuration::const_ptr hip_config);

			// stream_id: a HIP stream handle. entry_count counts the entries of the output; the inputs hold as many,
			// except where the layer itself changes the count (windows over entries, tiling). The output buffer
			// may be the buffer of input get_input_index_layer_can_write().
			virtual void enqueue_forward_propagation(
				void * stream_id,
				hip_linear_buffer_device::ptr output_buffer,
				const std::vector<hip_linear_buffer_device::const_ptr>& schema_data,
				const std::vector<hip_linear_buffer_device::const_ptr>& data,
				const std::vector<hip_linear_buffer_device::const_ptr>& data_custom,
				const std::vector<hip_linear_buffer_device::const_ptr>& input_buffers,
				const std::vector<hip_linear_buffer_device::const_ptr>& persistent_working_data,
				hip_linear_buffer_device::ptr temporary_working_fixed_buffer,
				hip_linear_buffer_device::ptr temporary_working_per_entry_buffer,
				unsigned int entry_count) = 0;

			// uploads the weights: one device buffer per chunk, in chunk order
			virtual std::vector<hip_linear_buffer_device::const_ptr> get_data(layer_data::const_ptr host_data) const;

			// integer side data of the layer: tells the tester (notify_data_custom), then uploads one device buffer per chunk
			virtual std::vector<hip_linear_buffer_device::const_ptr> set_get_data_custom(layer_data_custom::const_ptr host_data_custom);

			// device buffers the tester fills once and keeps across calls; handed back to it with every enqueue
			virtual std::vector<hip_linear_buffer_device::const_ptr> get_persistent_working_data() const;

			virtual int get_input_index_layer_can_write() const { return -1; }
			// minimum size, and whether the tester would make use of a larger buffer
			virtual std::pair<size_t, bool> get_temporary_working_fixed_buffer_size() const { return std::make_pair(static_cast<size_t>(0), false); }
			virtual size_t get_temporary_working_per_entry_buffer_size() const { return 0; }

			// nnforge/cuda/layer_tester_cuda.h:82 asks which inputs the tester wants to read through a texture; this
			// backend has no texture path and no tester overrides it: always empty
			virtual std::vector<unsigned int> get_linear_addressing_through_texture_per_entry() const { return std::vector<unsigned int>(); }

			// Element-wise testers describe themselves as one op of a fused group: fills op (its chunk
			// index is set by the caller) and returns how many weight chunks the op consumes, or -1
			// when the layer cannot be part of a fused group.
			virtual int get_chain_op(nnf_hip_op& op) const { return -1; }

			// Subsampling testers can apply the element-wise layers in front of them to the values they
			// read, so that the result of those layers is never stored. can_apply_prologue: whether this
			// tester's shapes allow it for a group of prologue_input_count inputs (1: a chain of layers; 2: two
			// chains joined by an Add, with layers behind it). enqueue_forward_propagation_with_prologue: the
			// forward pass with the layers of prologue (whose shape is this tester's input; its inputs in
			// input_buffers, its weights in chunk_ptrs) applied first.
			virtual bool can_apply_prologue(unsigned int prologue_input_count) const { return false; }
			virtual void enqueue_forward_propagation_with_prologue(
				void * stream_id,
				hip_linear_buffer_device::ptr output_buffer,
				const std::vector<hip_linear_buffer_device::const_ptr>& input_buffers,
				const nnf_hip_chain_desc& prologue,
				const float * const * chunk_ptrs,
				unsigned int entry_count);

			// A tester that only puts its inputs side by side (Concat) need not copy an input that was written to its
			// place in the output buffer by the step that made it. can_take_inputs_in_place: whether this tester can
			// leave inputs out; enqueue_forward_propagation_with_inputs_in_place: the forward pass for the inputs
			// whose flag is false (the buffers of the others are not looked at).
			virtual bool can_take_inputs_in_place() const { return false; }
			virtual void enqueue_forward_propagation_with_inputs_in_place(
				void * stream_id,
				hip_linear_buffer_device::ptr output_buffer,
				const std::vector<hip_linear_buffer_device::const_ptr>& input_buffers,
				const std::vector<bool>& inputs_in_place,
				unsigned int entry_count);

		protected:
			layer_tester_hip() = default;
			virtual void tester_configured() {}
			virtual void notify_data_custom(layer_data_custom::const_ptr host_data_custom) {}

			layer::const_ptr layer_schema;
			hip_running_configuration::const_ptr hip_config;
			std::vector<layer_configuration_specific> input_configuration_specific_list;
			std::vector<unsigned int> input_elem_count_per_entry_list;
			std::vector<unsigned int> input_elem_count_per_feature_map_list;
			layer_configuration_specific output_configuration_specific;
			unsigned int output_elem_count_per_entry;
			unsigned int output_elem_count_per_feature_map;

		private:
			layer_tester_hip(const layer_tester_hip&) = delete;
			layer_tester_hip& operator =(const layer_tester_hip&) = delete;
		};

		// Prototype that makes testers of one layer type (nnforge/cuda/layer_testing_schema.h:36-71)
		class layer_testing_schema
		{
		public:
			typedef std::shared_ptr<layer_testing_schema> ptr;
			typedef std::shared_ptr<const layer_testing_schema> const_ptr;
			virtual ~layer_testing_schema() = default;

			layer_testing_schema::ptr create(layer::const_ptr layer_schema) const;
			layer_tester_hip::ptr create_tester(
				const std::vector<layer_configuration_specific>& input_configuration_specific_list,
				const layer_configuration_specific& output_configuration_specific,
				hip_running_configuration::const_ptr hip_config) const;
			virtual std::string get_type_name() const = 0;

		protected:
			layer_testing_schema() = default;
			virtual layer_testing_schema::ptr create_specific() const = 0;
			virtual layer_tester_hip::ptr create_tester_specific(
				const std::vector<layer_configuration_specific>& input_configuration_specific_list,
				const layer_configuration_specific& output_configuration_specific,
				const hip_running_configuration& hip_config) const = 0;
			layer::const_ptr layer_schema;
		};

		// String-keyed registry of the prototypes (nnforge/cuda/layer_testing_schema_factory.cpp:26-50;
		// same role as layer_tester_plain_factory, nnforge/plain/layer_tester_plain_factory.cpp:27-51)
		class layer_testing_schema_factory
		{
		public:
			bool register_layer_testing_schema(layer_testing_schema::const_ptr sample_layer_testing_schema);
			bool unregister_layer_testing_schema(const std::string& layer_type_name);
			// throws "No layer tester is registered with type ..." for an unknown type
			layer_testing_schema::ptr create_testing_schema_layer(layer::const_ptr layer) const;
			static layer_testing_schema_factory& get_singleton();

		private:
			layer_testing_schema_factory() = default;
			std::map<std::string, layer_testing_schema::const_ptr> sample_map;
		};

		// One launch of the forward pass: a single layer or a fused group of element-wise layers.
		struct forward_step
		{
			std::vector<std::string> layer_names;  // members in execution order; back() produces the output
			std::vector<std::string> input_names;  // layers whose buffers are read, in kernel input order
			bool fused;                            // several layers in one launch: the fused-group kernel, or a subsampling
			                                       // layer (the last name) that applies the element-wise layers in front of it
			// The kernel stream the launch goes to. Steps that depend on each other (one reads what the other wrote, or
			// writes a buffer the other still uses) share a stream; steps that have nothing to do with each other take
			// the streams in turn and may overlap.
			unsigned int stream_index = 0;
			// Consecutive fused groups that do not depend on each other are handed to the kernels in one call
			// (nnf_hip_chain_forward_batch): steps with the same index >= 0 form such a run; -1: launched on its own.
			int batch_index = -1;
			// A fused group that writes its result straight into the output of the Concat layer behind it (entry by entry,
			// at its feature maps' place): the name of that layer, empty otherwise. For the Concat step itself: the inputs
			// it finds in place and does not copy.
			std::string writes_into;
			std::vector<std::string> inputs_in_place;
			std::string description() const;       // e.g. "bn1+add1+relu1 <- conv_a, conv_b"
		};

		// nnforge/cuda/forward_propagation_cuda.h restated for one MI355X.
		class forward_propagation_hip : public forward_propagation
		{
		public:
			forward_propagation_hip(
				const network_schema& schema,
				const std::vector<std::string>& output_layer_names,
				debug_state::ptr debug,
				profile_state::ptr profile,
				hip_running_configuration::const_ptr hip_config);
			~forward_propagation_hip() override;

			// the launch plan of the current configuration (valid after set_input_configuration_specific / run)
			const std::vector<forward_step>& get_steps() const { return steps; }
			// device bytes per entry of the current buffer plan, and the packet size derived from it
			size_t get_per_entry_buffer_bytes() const { return per_entry_bytes; }
			unsigned int get_max_entry_count() const { return max_entry_count; }
			// entries per packet of the latest run() (0 before the first): max_entry_count, the reader's entry count and the
			// configuration's staging bound decide it
			unsigned int get_packet_entry_count() const { return packet_entry_count; }

			// Times the launch plan alone, on data that stays in device memory: reads one packet of up to entry_count
			// entries from the reader and uploads it, runs the plan once and warmup times more untimed, then `passes`
			// times bracketed by a device synchronisation on both sides (wall clock) and by events on the kernel stream.
			// resident_packets > 1: the data and output layers get that many sets of device buffers (every set holds
			// the same packet) and the passes go round them, so that a small network's tensors come from memory and
			// not from the last-level cache; buffers in between are shared by all sets. Nothing is copied back and
			// the writer's role is empty: this is the figure of merit of the kernels and of the way the driver
			// enqueues them, without the host link. No counterpart in the reference.
			struct kernel_timing
			{
				unsigned int entry_count;      // entries the packet held
				unsigned int resident_packets; // buffer sets the passes went round
				unsigned int plan_step_count;  // steps of the plan that launch something
				unsigned int launch_count;     // kernels one pass launches (steps that go to the kernels in one call share launches)
				float wall_seconds_per_pass;
				float device_seconds_per_pass; // from events on the kernel stream
				float host_seconds_per_pass;   // what the calling thread spends enqueuing a pass (the device runs behind it)
			};
			// replay_recorded_plan: the launches of a pass are recorded once (a HIP graph per set of buffers) and the timed
			// passes replay the recordings - what the calling thread spends per pass is then one call per pass.
			kernel_timing time_kernels(structured_data_bunch_reader& reader, unsigned int entry_count, unsigned int warmup, unsigned int passes,
				unsigned int resident_packets = 1, bool replay_recorded_plan = false);

		protected:
			void actual_set_data(network_data::const_ptr data) override;
			void actual_clear_data() override;
			void actual_run(
				structured_data_bunch_reader& reader,
				structured_data_bunch_writer& writer,
				unsigned int& entries_processed,
				std::map<layer_name_with_action, float>& action_seconds,
				float& idle_seconds) override;
			void layer_config_map_modified() override;
			float get_max_bytes_per_second() const override; // HBM peak of the MI355X

		private:
			struct impl;
			struct run_buffers;
			// streams, device buffers for packets of `packet` entries (data and output layers once per I/O slot), pinned
			// staging, weight pointers; what the run before left is used again when it was made for the same sizes
			// (staging_slot_count <= 0: as many as slot_count)
			run_buffers& prepare_run(unsigned int packet, int slot_count, bool with_output_staging, bool stats_on_device, int staging_slot_count = 0);
			std::unique_ptr<impl> p;
			std::unique_ptr<run_buffers> kept_run; // released when the weights, the shapes or the packet size change
			hip_running_configuration::const_ptr hip_config;
			std::vector<forward_step> steps;
			size_t per_entry_bytes;
			unsigned int max_entry_count;
			unsigned int packet_entry_count = 0;
		};

		// nnforge/cuda/forward_propagation_cuda_factory.h
		class forward_propagation_hip_factory : public forward_propagation_factory
		{
		public:
			explicit forward_propagation_hip_factory(hip_running_configuration::const_ptr hip_config) : hip_config(hip_config) {}
			forward_propagation::ptr create(
				const network_schema& schema,
				const std::vector<std::string>& output_layer_names,
				debug_state::ptr debug,
				profile_state::ptr profile) const override;

		private:
			hip_running_configuration::const_ptr hip_config;
		};

		// nnforge/cuda/factory_generator_cuda.h: options hip_device_id, hip_max_global_memory_usage_ratio,
		// hip_fuse, hip_dont_share_buffers, hip_single_command_stream (as cuda_single_command_stream,
		// nnforge/cuda/factory_generator_cuda.cpp:105-106), hip_batch_independent_groups, hip_kernel_stream_count, hip_max_entry_count,
		// hip_reserved_thread_count (as cuda_reserved_thread_count, nnforge/cuda/factory_generator_cuda.cpp:95), hip_max_io_staging_mb
		class factory_generator_hip : public factory_generator
		{
		public:
			factory_generator_hip();
			void initialize() override;
			forward_propagation_factory::ptr create_forward_propagation_factory() const override;
			backward_propagation_factory::ptr create_backward_propagation_factory() const override; // throws: inference only
			void info() const override;
			std::vector<bool_option> get_bool_options() override;
			std::vector<float_option> get_float_options() override;
			std::vector<int_option> get_int_options() override;

			int hip_device_id;
			float hip_max_global_memory_usage_ratio;
			bool hip_fuse;
			bool hip_dont_share_buffers;
			bool hip_single_command_stream;
			bool hip_batch_independent_groups;
			int hip_kernel_stream_count;
			int hip_max_entry_count;
			int hip_reserved_thread_count;
			int hip_max_io_staging_mb;
			bool hip_concat_in_place;

		private:
			hip_running_configuration::const_ptr hip_config;
		};

		// registers the layer types and the testers of this backend (nnforge/cuda/cuda.cpp:92-160,
		// nnforge/plain/plain.cpp:92-126)
		void init();
	}
}
