// Runtime objects of the hip backend and one layer_tester_hip per layer type. Each tester calls
// the C-ABI entry point that replaces the matching plain tester; element-wise testers also
// describe themselves as an op of a fused group.
#include "nnforge_hip/hip_backend.h"

#include <cstring>
#include <iostream>
#include <sstream>

namespace nnforge
{
	namespace hip
	{
		// ---- errors, buffers, device configuration -----------------------------------------

		neural_network_hip_exception::neural_network_hip_exception(int error_code, const char * filename, int line_number)
			: neural_network_exception(std::string(nnf_hip_error_string(error_code)) + " (code " + std::to_string(error_code) + ")", filename, line_number)
			, error_code(error_code)
		{
		}

		void hip_check(int code, const char * filename, int line_number)
		{
			if (code != NNF_HIP_OK)
				throw neural_network_hip_exception(code, filename, line_number);
		}

		hip_linear_buffer_device::hip_linear_buffer_device(size_t size) : buf(nullptr), size(size)
		{
			hip_safe_call(nnf_hip_malloc(&buf, size));
		}

		hip_linear_buffer_device::~hip_linear_buffer_device()
		{
			if (buf != nullptr)
				nnf_hip_free(buf);
		}

		constexpr int hip_running_configuration::default_kernel_stream_count;

		hip_running_configuration::hip_running_configuration(int device_id, float max_global_memory_usage_ratio, bool fuse_layers, bool dont_share_buffers, int max_entry_count,
			int kernel_stream_count, bool batch_independent_groups, unsigned int reserved_thread_count)
			: device_id(device_id)
			, max_global_memory_usage_ratio(max_global_memory_usage_ratio)
			, fuse_layers(fuse_layers)
			, dont_share_buffers(dont_share_buffers)
			, max_entry_count(max_entry_count)
			, kernel_stream_count(kernel_stream_count)
			, batch_independent_groups(batch_independent_groups)
			, reserved_thread_count(reserved_thread_count)
			, global_memory_size(0)
			, compute_unit_count(0)
			, wavefront_size(0)
			, clock_khz(0)
		{
			int device_count = 0;
			hip_safe_call(nnf_hip_device_count(&device_count));
			if (device_count <= 0)
				throw neural_network_exception("No HIP device found");
			if ((device_id < 0) || (device_id >= device_count))
				throw neural_network_exception("Device ID " + std::to_string(device_id) + " specified while " + std::to_string(device_count) + " devices are available");
			char name[256];
			uint64_t mem = 0;
			hip_safe_call(nnf_hip_device_info(device_id, name, sizeof(name), &mem, &compute_unit_count, &wavefront_size, &clock_khz));
			device_name = name;
			global_memory_size = mem;
			const unsigned int processors = get_available_processor_count();
			job_runner.reset(new threadpool_job_runner(std::min(max_job_thread_count, (processors > reserved_thread_count) ? processors - reserved_thread_count : 1U)));
		}

		hip_running_configuration::const_ptr hip_running_configuration::create_offline(
			unsigned long long global_memory_size, float max_global_memory_usage_ratio, bool fuse_layers, bool dont_share_buffers, int max_entry_count,
			int kernel_stream_count, bool batch_independent_groups)
		{
			std::shared_ptr<hip_running_configuration> res(new hip_running_configuration());
			res->kernel_stream_count = kernel_stream_count;
			res->batch_independent_groups = batch_independent_groups;
			res->reserved_thread_count = 1;
			res->device_id = -1;
			res->max_global_memory_usage_ratio = max_global_memory_usage_ratio;
			res->fuse_layers = fuse_layers;
			res->dont_share_buffers = dont_share_buffers;
			res->max_entry_count = max_entry_count;
			res->device_name = "offline";
			res->global_memory_size = global_memory_size;
			res->compute_unit_count = 0;
			res->wavefront_size = 64;
			res->clock_khz = 0;
			res->offline = true;
			return res;
		}

		void hip_running_configuration::set_device() const
		{
			if (!offline)
				hip_safe_call(nnf_hip_set_device(device_id));
		}

		size_t hip_running_configuration::get_max_bytes() const
		{
			return static_cast<size_t>(static_cast<double>(global_memory_size) * static_cast<double>(max_global_memory_usage_ratio));
		}

		std::ostream& operator<<(std::ostream& out, const hip_running_configuration& config)
		{
			out << "--- HIP device ---" << std::endl;
			out << "Device Id = " << config.device_id << std::endl;
			out << "Device name = " << config.device_name << std::endl;
			out << "Global memory = " << (config.global_memory_size >> 20) << " MB" << std::endl;
			out << "Compute units = " << config.compute_unit_count << ", wavefront " << config.wavefront_size << ", clock " << (config.clock_khz / 1000) << " MHz" << std::endl;
			out << "Memory usage ratio = " << config.max_global_memory_usage_ratio << ", fuse element-wise layers = " << (config.fuse_layers ? "yes" : "no")
				<< ", independent groups launched together = " << (config.batch_independent_groups ? "yes" : "no")
				<< ", kernel streams = " << config.kernel_stream_count << std::endl;
			if (config.get_job_runner())
				out << "Job runner thread count = " << config.get_job_runner()->thread_count << std::endl;
			return out;
		}

		// ---- tester base, testing schema, registry -----------------------------------------

		void layer_tester_hip::configure(
			const std::vector<layer_configuration_specific>& input_configuration_specific_list,
			const layer_configuration_specific& output_configuration_specific,
			layer::const_ptr layer_schema,
			hip_running_configuration::const_ptr hip_config)
		{
			this->layer_schema = layer_schema;
			this->input_configuration_specific_list = input_configuration_specific_list;
			this->output_configuration_specific = output_configuration_specific;
			this->hip_config = hip_config;
			input_elem_count_per_entry_list.clear();
			input_elem_count_per_feature_map_list.clear();
			for(const layer_configuration_specific& c : input_configuration_specific_list)
			{
				input_elem_count_per_entry_list.push_back(c.get_neuron_count());
				input_elem_count_per_feature_map_list.push_back(c.get_neuron_count_per_feature_map());
			}
			output_elem_count_per_entry = output_configuration_specific.get_neuron_count();
			output_elem_count_per_feature_map = output_configuration_specific.get_neuron_count_per_feature_map();
			tester_configured();
		}

		std::vector<hip_linear_buffer_device::const_ptr> layer_tester_hip::get_data(layer_data::const_ptr host_data) const
		{
			std::vector<hip_linear_buffer_device::const_ptr> res;
			if (!host_data)
				return res;
			for(const std::vector<float>& chunk : *host_data)
			{
				const size_t bytes = chunk.size() * sizeof(float);
				hip_linear_buffer_device::ptr buf(new hip_linear_buffer_device(bytes));
				if (bytes > 0)
					hip_safe_call(nnf_hip_memcpy_h2d(*buf, chunk.data(), bytes, nullptr));
				res.push_back(buf);
			}
			return res;
		}

		std::vector<hip_linear_buffer_device::const_ptr> layer_tester_hip::set_get_data_custom(layer_data_custom::const_ptr host_data_custom)
		{
			notify_data_custom(host_data_custom);
			std::vector<hip_linear_buffer_device::const_ptr> res;
			if (!host_data_custom)
				return res;
			for(const std::vector<int>& chunk : *host_data_custom)
			{
				const size_t bytes = chunk.size() * sizeof(int);
				hip_linear_buffer_device::ptr buf(new hip_linear_buffer_device(bytes));
				if (bytes > 0)
					hip_safe_call(nnf_hip_memcpy_h2d(*buf, chunk.data(), bytes, nullptr));
				res.push_back(buf);
			}
			return res;
		}

		std::vector<hip_linear_buffer_device::const_ptr> layer_tester_hip::get_persistent_working_data() const
		{
			return std::vector<hip_linear_buffer_device::const_ptr>();
		}

		void layer_tester_hip::enqueue_forward_propagation_with_prologue(void *, hip_linear_buffer_device::ptr, const std::vector<hip_linear_buffer_device::const_ptr>&,
			const nnf_hip_chain_desc&, const float * const *, unsigned int)
		{
			throw neural_network_exception("Layer " + layer_schema->instance_name + " of type " + layer_schema->get_type_name() + " cannot apply other layers to its input");
		}

		void layer_tester_hip::enqueue_forward_propagation_with_inputs_in_place(void *, hip_linear_buffer_device::ptr, const std::vector<hip_linear_buffer_device::const_ptr>&,
			const std::vector<bool>&, unsigned int)
		{
			throw neural_network_exception("Layer " + layer_schema->instance_name + " of type " + layer_schema->get_type_name() + " reads all its inputs: none of them can be taken as being in place");
		}

		layer_testing_schema::ptr layer_testing_schema::create(layer::const_ptr layer_schema) const
		{
			layer_testing_schema::ptr res = create_specific();
			res->layer_schema = layer_schema;
			return res;
		}

		layer_tester_hip::ptr layer_testing_schema::create_tester(
			const std::vector<layer_configuration_specific>& input_configuration_specific_list,
			const layer_configuration_specific& output_configuration_specific,
			hip_running_configuration::const_ptr hip_config) const
		{
			layer_tester_hip::ptr res = create_tester_specific(input_configuration_specific_list, output_configuration_specific, *hip_config);
			res->configure(input_configuration_specific_list, output_configuration_specific, layer_schema, hip_config);
			return res;
		}

		bool layer_testing_schema_factory::register_layer_testing_schema(layer_testing_schema::const_ptr sample)
		{
			return sample_map.insert(std::make_pair(sample->get_type_name(), sample)).second;
		}

		bool layer_testing_schema_factory::unregister_layer_testing_schema(const std::string& layer_type_name)
		{
			return sample_map.erase(layer_type_name) == 1;
		}

		layer_testing_schema::ptr layer_testing_schema_factory::create_testing_schema_layer(layer::const_ptr layer) const
		{
			std::map<std::string, layer_testing_schema::const_ptr>::const_iterator it = sample_map.find(layer->get_type_name());
			if (it == sample_map.end())
				throw neural_network_exception("No layer tester is registered with type " + layer->get_type_name());
			return it->second->create(layer);
		}

		layer_testing_schema_factory& layer_testing_schema_factory::get_singleton()
		{
			static layer_testing_schema_factory instance;
			return instance;
		}

		// ---- the testers -------------------------------------------------------------------

		namespace
		{
			const float * float_ptr(const hip_linear_buffer_device::const_ptr& b)
			{
				return static_cast<const float *>(*b);
			}

			void require_inputs(const std::vector<hip_linear_buffer_device::const_ptr>& input_buffers, size_t count, const char * what)
			{
				if (input_buffers.size() < count)
					throw neural_network_exception(std::string(what) + ": " + std::to_string(input_buffers.size()) + " input buffers supplied, " + std::to_string(count) + " needed");
			}

			void require_data(const std::vector<hip_linear_buffer_device::const_ptr>& data, size_t count, const char * what)
			{
				if (data.size() != count)
					throw neural_network_exception(std::string(what) + ": " + std::to_string(data.size()) + " weight chunks supplied, " + std::to_string(count) + " needed");
			}

			// Element-wise testers share everything but the entry point they call.
			class elementwise_tester : public layer_tester_hip
			{
			public:
				int get_input_index_layer_can_write() const override { return 0; } // as every plain tester on this path
			};

			class batch_norm_layer_tester_hip : public elementwise_tester
			{
			public:
				void enqueue_forward_propagation(void * stream_id, hip_linear_buffer_device::ptr output_buffer,
					const std::vector<hip_linear_buffer_device::const_ptr>&, const std::vector<hip_linear_buffer_device::const_ptr>& data,
					const std::vector<hip_linear_buffer_device::const_ptr>&, const std::vector<hip_linear_buffer_device::const_ptr>& input_buffers,
					const std::vector<hip_linear_buffer_device::const_ptr>&, hip_linear_buffer_device::ptr, hip_linear_buffer_device::ptr,
					unsigned int entry_count) override
				{
					require_inputs(input_buffers, 1, "BatchNorm");
					require_data(data, 4, "BatchNorm");
					hip_safe_call(nnf_hip_batch_norm_forward(stream_id, *output_buffer, float_ptr(input_buffers[0]),
						float_ptr(data[0]), float_ptr(data[1]), float_ptr(data[2]), float_ptr(data[3]),
						entry_count, output_configuration_specific.feature_map_count, output_elem_count_per_feature_map));
				}

				int get_chain_op(nnf_hip_op& op) const override
				{
					op.kind = NNF_HIP_OP_BATCH_NORM;
					op.f0 = op.f1 = 0.0F;
					return 4;
				}

			protected:
				void tester_configured() override
				{
					std::shared_ptr<const batch_norm_layer> l = std::dynamic_pointer_cast<const batch_norm_layer>(layer_schema);
					if (!l)
						throw neural_network_exception("BatchNorm tester configured with a layer of type " + layer_schema->get_type_name());
					if (l->feature_map_count != output_configuration_specific.feature_map_count)
						throw neural_network_exception("Feature map count in layer (" + std::to_string(l->feature_map_count) + ") and input configuration (" + std::to_string(output_configuration_specific.feature_map_count) + ") don't match");
				}
			};

			class rectified_linear_layer_tester_hip : public elementwise_tester
			{
			public:
				void enqueue_forward_propagation(void * stream_id, hip_linear_buffer_device::ptr output_buffer,
					const std::vector<hip_linear_buffer_device::const_ptr>&, const std::vector<hip_linear_buffer_device::const_ptr>&,
					const std::vector<hip_linear_buffer_device::const_ptr>&, const std::vector<hip_linear_buffer_device::const_ptr>& input_buffers,
					const std::vector<hip_linear_buffer_device::const_ptr>&, hip_linear_buffer_device::ptr, hip_linear_buffer_device::ptr,
					unsigned int entry_count) override
				{
					require_inputs(input_buffers, 1, "ReLU");
					hip_safe_call(nnf_hip_rectified_linear_forward(stream_id, *output_buffer, float_ptr(input_buffers[0]), negative_slope,
						static_cast<uint64_t>(entry_count) * output_elem_count_per_entry));
				}

				int get_chain_op(nnf_hip_op& op) const override
				{
					op.kind = NNF_HIP_OP_RELU;
					op.f0 = negative_slope;
					op.f1 = 0.0F;
					return 0;
				}

			protected:
				void tester_configured() override
				{
					std::shared_ptr<const rectified_linear_layer> l = std::dynamic_pointer_cast<const rectified_linear_layer>(layer_schema);
					if (!l)
						throw neural_network_exception("ReLU tester configured with a layer of type " + layer_schema->get_type_name());
					negative_slope = l->negative_slope;
				}

			private:
				float negative_slope = 0.0F;
			};

			class parametric_rectified_linear_layer_tester_hip : public elementwise_tester
			{
			public:
				void enqueue_forward_propagation(void * stream_id, hip_linear_buffer_device::ptr output_buffer,
					const std::vector<hip_linear_buffer_device::const_ptr>&, const std::vector<hip_linear_buffer_device::const_ptr>& data,
					const std::vector<hip_linear_buffer_device::const_ptr>&, const std::vector<hip_linear_buffer_device::const_ptr>& input_buffers,
					const std::vector<hip_linear_buffer_device::const_ptr>&, hip_linear_buffer_device::ptr, hip_linear_buffer_device::ptr,
					unsigned int entry_count) override
				{
					require_inputs(input_buffers, 1, "PReLU");
					require_data(data, 1, "PReLU");
					hip_safe_call(nnf_hip_parametric_rectified_linear_forward(stream_id, *output_buffer, float_ptr(input_buffers[0]), float_ptr(data[0]),
						entry_count, output_configuration_specific.feature_map_count, output_elem_count_per_feature_map));
				}

				int get_chain_op(nnf_hip_op& op) const override
				{
					op.kind = NNF_HIP_OP_PRELU;
					op.f0 = op.f1 = 0.0F;
					return 1;
				}

			protected:
				void tester_configured() override
				{
					std::shared_ptr<const parametric_rectified_linear_layer> l = std::dynamic_pointer_cast<const parametric_rectified_linear_layer>(layer_schema);
					if (!l)
						throw neural_network_exception("PReLU tester configured with a layer of type " + layer_schema->get_type_name());
					if (l->feature_map_count != output_configuration_specific.feature_map_count)
						throw neural_network_exception("Feature map count in layer (" + std::to_string(l->feature_map_count) + ") and input configuration (" + std::to_string(output_configuration_specific.feature_map_count) + ") don't match");
				}
			};

			class exponential_linear_layer_tester_hip : public elementwise_tester
			{
			public:
				void enqueue_forward_propagation(void * stream_id, hip_linear_buffer_device::ptr output_buffer,
					const std::vector<hip_linear_buffer_device::const_ptr>&, const std::vector<hip_linear_buffer_device::const_ptr>&,
					const std::vector<hip_linear_buffer_device::const_ptr>&, const std::vector<hip_linear_buffer_device::const_ptr>& input_buffers,
					const std::vector<hip_linear_buffer_device::const_ptr>&, hip_linear_buffer_device::ptr, hip_linear_buffer_device::ptr,
					unsigned int entry_count) override
				{
					require_inputs(input_buffers, 1, "ELU");
					hip_safe_call(nnf_hip_exponential_linear_forward(stream_id, *output_buffer, float_ptr(input_buffers[0]),
						static_cast<uint64_t>(entry_count) * output_elem_count_per_entry));
				}

				int get_chain_op(nnf_hip_op& op) const override
				{
					op.kind = NNF_HIP_OP_ELU;
					op.f0 = op.f1 = 0.0F;
					return 0;
				}
			};

			class sigmoid_layer_tester_hip : public elementwise_tester
			{
			public:
				void enqueue_forward_propagation(void * stream_id, hip_linear_buffer_device::ptr output_buffer,
					const std::vector<hip_linear_buffer_device::const_ptr>&, const std::vector<hip_linear_buffer_device::const_ptr>&,
					const std::vector<hip_linear_buffer_device::const_ptr>&, const std::vector<hip_linear_buffer_device::const_ptr>& input_buffers,
					const std::vector<hip_linear_buffer_device::const_ptr>&, hip_linear_buffer_device::ptr, hip_linear_buffer_device::ptr,
					unsigned int entry_count) override
				{
					require_inputs(input_buffers, 1, "Sigmoid");
					hip_safe_call(nnf_hip_sigmoid_forward(stream_id, *output_buffer, float_ptr(input_buffers[0]),
						static_cast<uint64_t>(entry_count) * output_elem_count_per_entry));
				}

				int get_chain_op(nnf_hip_op& op) const override
				{
					op.kind = NNF_HIP_OP_SIGMOID;
					op.f0 = op.f1 = 0.0F;
					return 0;
				}
			};

			class hyperbolic_tangent_layer_tester_hip : public elementwise_tester
			{
			public:
				void enqueue_forward_propagation(void * stream_id, hip_linear_buffer_device::ptr output_buffer,
					const std::vector<hip_linear_buffer_device::const_ptr>&, const std::vector<hip_linear_buffer_device::const_ptr>&,
					const std::vector<hip_linear_buffer_device::const_ptr>&, const std::vector<hip_linear_buffer_device::const_ptr>& input_buffers,
					const std::vector<hip_linear_buffer_device::const_ptr>&, hip_linear_buffer_device::ptr, hip_linear_buffer_device::ptr,
					unsigned int entry_count) override
				{
					require_inputs(input_buffers, 1, "TanH");
					hip_safe_call(nnf_hip_hyperbolic_tangent_forward(stream_id, *output_buffer, float_ptr(input_buffers[0]), scale, steepness,
						static_cast<uint64_t>(entry_count) * output_elem_count_per_entry));
				}

				int get_chain_op(nnf_hip_op& op) const override
				{
					op.kind = NNF_HIP_OP_TANH;
					op.f0 = scale;
					op.f1 = steepness;
					return 0;
				}

			protected:
				void tester_configured() override
				{
					std::shared_ptr<const hyperbolic_tangent_layer> l = std::dynamic_pointer_cast<const hyperbolic_tangent_layer>(layer_schema);
					if (!l)
						throw neural_network_exception("TanH tester configured with a layer of type " + layer_schema->get_type_name());
					scale = l->scale;
					steepness = l->steepness;
				}

			private:
				float scale = 1.0F;
				float steepness = 1.0F;
			};

			class add_layer_tester_hip : public elementwise_tester
			{
			public:
				void enqueue_forward_propagation(void * stream_id, hip_linear_buffer_device::ptr output_buffer,
					const std::vector<hip_linear_buffer_device::const_ptr>&, const std::vector<hip_linear_buffer_device::const_ptr>&,
					const std::vector<hip_linear_buffer_device::const_ptr>&, const std::vector<hip_linear_buffer_device::const_ptr>& input_buffers,
					const std::vector<hip_linear_buffer_device::const_ptr>&, hip_linear_buffer_device::ptr, hip_linear_buffer_device::ptr,
					unsigned int entry_count) override
				{
					require_inputs(input_buffers, 1, "Add");
					std::vector<const float *> inputs;
					for(const hip_linear_buffer_device::const_ptr& b : input_buffers)
						inputs.push_back(float_ptr(b));
					hip_safe_call(nnf_hip_add_forward(stream_id, *output_buffer, inputs.data(), static_cast<uint32_t>(inputs.size()), alpha,
						static_cast<uint64_t>(entry_count) * output_elem_count_per_entry));
				}

				float get_alpha() const { return alpha; }

			protected:
				void tester_configured() override
				{
					std::shared_ptr<const add_layer> l = std::dynamic_pointer_cast<const add_layer>(layer_schema);
					if (!l)
						throw neural_network_exception("Add tester configured with a layer of type " + layer_schema->get_type_name());
					alpha = l->alpha;
				}

			private:
				float alpha = 1.0F;
			};

			class softmax_layer_tester_hip : public layer_tester_hip
			{
			public:
				void enqueue_forward_propagation(void * stream_id, hip_linear_buffer_device::ptr output_buffer,
					const std::vector<hip_linear_buffer_device::const_ptr>&, const std::vector<hip_linear_buffer_device::const_ptr>&,
					const std::vector<hip_linear_buffer_device::const_ptr>&, const std::vector<hip_linear_buffer_device::const_ptr>& input_buffers,
					const std::vector<hip_linear_buffer_device::const_ptr>&, hip_linear_buffer_device::ptr, hip_linear_buffer_device::ptr,
					unsigned int entry_count) override
				{
					require_inputs(input_buffers, 1, "Softmax");
					hip_safe_call(nnf_hip_softmax_forward(stream_id, *output_buffer, float_ptr(input_buffers[0]),
						entry_count, output_configuration_specific.feature_map_count, output_elem_count_per_feature_map));
				}

				int get_input_index_layer_can_write() const override { return 0; } // nnforge/plain/softmax_layer_tester_plain.cpp:93-100
			};

			class average_subsampling_layer_tester_hip : public layer_tester_hip
			{
			public:
				void enqueue_forward_propagation(void * stream_id, hip_linear_buffer_device::ptr output_buffer,
					const std::vector<hip_linear_buffer_device::const_ptr>&, const std::vector<hip_linear_buffer_device::const_ptr>&,
					const std::vector<hip_linear_buffer_device::const_ptr>&, const std::vector<hip_linear_buffer_device::const_ptr>& input_buffers,
					const std::vector<hip_linear_buffer_device::const_ptr>&, hip_linear_buffer_device::ptr, hip_linear_buffer_device::ptr,
					unsigned int entry_count) override
				{
					require_inputs(input_buffers, 1, "AverageSubsampling");
					// entry_count counts the entries of the output; the input holds entry_window times as many
					if (plain_2d)
						hip_safe_call(nnf_hip_average_subsampling_forward(stream_id, *output_buffer, float_ptr(input_buffers[0]),
							entry_count, output_configuration_specific.feature_map_count, input_sizes[0], input_sizes[1], windows[0], windows[1], mult));
					else
						hip_safe_call(nnf_hip_average_subsampling_nd_forward(stream_id, *output_buffer, float_ptr(input_buffers[0]), entry_count,
							input_configuration_specific_list[0].feature_map_count, dimension_count, input_sizes.data(), windows.data(),
							feature_map_window, entry_window, mult));
				}

				bool can_apply_prologue(unsigned int prologue_input_count) const override
				{
					if (!plain_2d)
						return false;
					if (prologue_input_count == 1)
						return nnf_hip_average_subsampling_fusable(1, output_configuration_specific.feature_map_count, input_sizes[0], input_sizes[1],
							windows[0], windows[1]) == NNF_HIP_OK;
					// two inputs joined by an Add: the average over whole planes takes them
					return (prologue_input_count == 2) && (nnf_hip_average_subsampling_joinable(1, output_configuration_specific.feature_map_count, input_sizes[0], input_sizes[1],
						windows[0], windows[1]) == NNF_HIP_OK);
				}

				void enqueue_forward_propagation_with_prologue(void * stream_id, hip_linear_buffer_device::ptr output_buffer,
					const std::vector<hip_linear_buffer_device::const_ptr>& input_buffers, const nnf_hip_chain_desc& prologue, const float * const * chunk_ptrs,
					unsigned int entry_count) override
				{
					require_inputs(input_buffers, prologue.input_count, "AverageSubsampling with layers folded in");
					if (prologue.input_count == 1)
					{
						hip_safe_call(nnf_hip_average_subsampling_fused_forward(stream_id, *output_buffer, float_ptr(input_buffers[0]), &prologue, chunk_ptrs,
							entry_count, output_configuration_specific.feature_map_count, input_sizes[0], input_sizes[1], windows[0], windows[1], mult));
						return;
					}
					const float * const inputs[2] = { float_ptr(input_buffers[0]), float_ptr(input_buffers[1]) };
					hip_safe_call(nnf_hip_average_subsampling_joined_forward(stream_id, *output_buffer, inputs, &prologue, chunk_ptrs,
						entry_count, output_configuration_specific.feature_map_count, input_sizes[0], input_sizes[1], windows[0], windows[1], mult));
				}

			protected:
				void tester_configured() override
				{
					std::shared_ptr<const average_subsampling_layer> l = std::dynamic_pointer_cast<const average_subsampling_layer>(layer_schema);
					if (!l)
						throw neural_network_exception("AverageSubsampling tester configured with a layer of type " + layer_schema->get_type_name());
					const layer_configuration_specific& in = input_configuration_specific_list.at(0);
					if ((in.get_dimension_count() < 1) || (in.get_dimension_count() > NNF_HIP_MAX_SUBSAMPLING_DIMENSIONS) || (l->subsampling_sizes.size() != in.get_dimension_count()))
						throw neural_network_exception("The hip average subsampling tester handles 1 to 4 spatial dimensions, layer " + layer_schema->instance_name + " has " + std::to_string(in.get_dimension_count()));
					entry_window = l->entry_subsampling_size;
					dimension_count = in.get_dimension_count();
					input_sizes.assign(in.dimension_sizes.begin(), in.dimension_sizes.end());
					windows.clear();
					for(unsigned int i = 0; i < dimension_count; ++i)
						windows.push_back(l->get_subsampling_size(i, in.dimension_sizes[i], output_configuration_specific.dimension_sizes[i]));
					feature_map_window = l->get_fm_subsampling_size(in.feature_map_count, output_configuration_specific.feature_map_count);
					plain_2d = (dimension_count <= 2) && (feature_map_window == 1) && (entry_window == 1);
					// the 2-D entry point takes width and height: a 1-D layer is one row high
					while (input_sizes.size() < 2)
					{
						input_sizes.push_back(1);
						windows.push_back(1);
					}
					// The multiplier of the reference's plain tester: window sum (over feature maps: their mean) unless the schema sets alpha.
					mult = l->get_plain_tester_alpha(feature_map_window);
				}

			private:
				std::vector<uint32_t> input_sizes, windows;
				uint32_t dimension_count = 1, feature_map_window = 1, entry_window = 1;
				bool plain_2d = true;
				float mult = 1.0F;
			};

			class absolute_layer_tester_hip : public elementwise_tester
			{
			public:
				void enqueue_forward_propagation(void * stream_id, hip_linear_buffer_device::ptr output_buffer,
					const std::vector<hip_linear_buffer_device::const_ptr>&, const std::vector<hip_linear_buffer_device::const_ptr>&,
					const std::vector<hip_linear_buffer_device::const_ptr>&, const std::vector<hip_linear_buffer_device::const_ptr>& input_buffers,
					const std::vector<hip_linear_buffer_device::const_ptr>&, hip_linear_buffer_device::ptr, hip_linear_buffer_device::ptr,
					unsigned int entry_count) override
				{
					require_inputs(input_buffers, 1, "Absolute");
					hip_safe_call(nnf_hip_absolute_forward(stream_id, *output_buffer, float_ptr(input_buffers[0]),
						static_cast<uint64_t>(entry_count) * output_elem_count_per_entry));
				}

				int get_chain_op(nnf_hip_op& op) const override
				{
					op.kind = NNF_HIP_OP_ABSOLUTE;
					op.f0 = op.f1 = 0.0F;
					return 0;
				}
			};

			// Inference: the input passes through (nnforge/cuda/dropout_layer_tester_cuda.cpp:27-51); in
			// place nothing is launched, inside a fused group the layer costs nothing.
			class dropout_layer_tester_hip : public elementwise_tester
			{
			public:
				void enqueue_forward_propagation(void * stream_id, hip_linear_buffer_device::ptr output_buffer,
					const std::vector<hip_linear_buffer_device::const_ptr>&, const std::vector<hip_linear_buffer_device::const_ptr>&,
					const std::vector<hip_linear_buffer_device::const_ptr>&, const std::vector<hip_linear_buffer_device::const_ptr>& input_buffers,
					const std::vector<hip_linear_buffer_device::const_ptr>&, hip_linear_buffer_device::ptr, hip_linear_buffer_device::ptr,
					unsigned int entry_count) override
				{
					require_inputs(input_buffers, 1, "Dropout");
					hip_safe_call(nnf_hip_dropout_forward(stream_id, *output_buffer, float_ptr(input_buffers[0]),
						static_cast<uint64_t>(entry_count) * output_elem_count_per_entry));
				}

				int get_chain_op(nnf_hip_op& op) const override
				{
					op.kind = NNF_HIP_OP_DROPOUT;
					op.f0 = op.f1 = 0.0F;
					return 0;
				}
			};

			class concat_layer_tester_hip : public layer_tester_hip
			{
			public:
				void enqueue_forward_propagation(void * stream_id, hip_linear_buffer_device::ptr output_buffer,
					const std::vector<hip_linear_buffer_device::const_ptr>&, const std::vector<hip_linear_buffer_device::const_ptr>&,
					const std::vector<hip_linear_buffer_device::const_ptr>&, const std::vector<hip_linear_buffer_device::const_ptr>& input_buffers,
					const std::vector<hip_linear_buffer_device::const_ptr>&, hip_linear_buffer_device::ptr, hip_linear_buffer_device::ptr,
					unsigned int entry_count) override
				{
					require_inputs(input_buffers, input_elem_count_per_entry_list.size(), "Concat");
					std::vector<const float *> inputs;
					std::vector<uint32_t> counts;
					for(size_t i = 0; i < input_elem_count_per_entry_list.size(); ++i)
					{
						inputs.push_back(float_ptr(input_buffers[i]));
						counts.push_back(input_elem_count_per_entry_list[i]);
					}
					hip_safe_call(nnf_hip_concat_forward(stream_id, *output_buffer, inputs.data(), counts.data(), static_cast<uint32_t>(inputs.size()), entry_count));
				}

				bool can_take_inputs_in_place() const override { return true; }

				void enqueue_forward_propagation_with_inputs_in_place(void * stream_id, hip_linear_buffer_device::ptr output_buffer,
					const std::vector<hip_linear_buffer_device::const_ptr>& input_buffers, const std::vector<bool>& inputs_in_place, unsigned int entry_count) override
				{
					require_inputs(input_buffers, input_elem_count_per_entry_list.size(), "Concat");
					if (inputs_in_place.size() != input_buffers.size())
						throw neural_network_exception("Concat: " + std::to_string(inputs_in_place.size()) + " flags for " + std::to_string(input_buffers.size()) + " inputs");
					std::vector<const float *> inputs;
					std::vector<uint32_t> counts;
					std::vector<uint8_t> flags;
					for(size_t i = 0; i < input_elem_count_per_entry_list.size(); ++i)
					{
						inputs.push_back(inputs_in_place[i] ? nullptr : float_ptr(input_buffers[i]));
						counts.push_back(input_elem_count_per_entry_list[i]);
						flags.push_back(inputs_in_place[i] ? 1 : 0);
					}
					hip_safe_call(nnf_hip_concat_forward_partial(stream_id, *output_buffer, inputs.data(), counts.data(), flags.data(), static_cast<uint32_t>(inputs.size()), entry_count));
				}
			};

			class maxout_layer_tester_hip : public layer_tester_hip
			{
			public:
				void enqueue_forward_propagation(void * stream_id, hip_linear_buffer_device::ptr output_buffer,
					const std::vector<hip_linear_buffer_device::const_ptr>&, const std::vector<hip_linear_buffer_device::const_ptr>&,
					const std::vector<hip_linear_buffer_device::const_ptr>&, const std::vector<hip_linear_buffer_device::const_ptr>& input_buffers,
					const std::vector<hip_linear_buffer_device::const_ptr>&, hip_linear_buffer_device::ptr, hip_linear_buffer_device::ptr,
					unsigned int entry_count) override
				{
					require_inputs(input_buffers, 1, "Maxout");
					hip_safe_call(nnf_hip_maxout_forward(stream_id, *output_buffer, float_ptr(input_buffers[0]), entry_count,
						output_configuration_specific.feature_map_count, output_elem_count_per_feature_map, feature_map_subsampling_size));
				}

			protected:
				void tester_configured() override
				{
					std::shared_ptr<const maxout_layer> l = std::dynamic_pointer_cast<const maxout_layer>(layer_schema);
					if (!l)
						throw neural_network_exception("Maxout tester configured with a layer of type " + layer_schema->get_type_name());
					feature_map_subsampling_size = l->feature_map_subsampling_size;
				}

			private:
				unsigned int feature_map_subsampling_size = 2;
			};

			class max_subsampling_layer_tester_hip : public layer_tester_hip
			{
			public:
				void enqueue_forward_propagation(void * stream_id, hip_linear_buffer_device::ptr output_buffer,
					const std::vector<hip_linear_buffer_device::const_ptr>&, const std::vector<hip_linear_buffer_device::const_ptr>&,
					const std::vector<hip_linear_buffer_device::const_ptr>&, const std::vector<hip_linear_buffer_device::const_ptr>& input_buffers,
					const std::vector<hip_linear_buffer_device::const_ptr>&, hip_linear_buffer_device::ptr, hip_linear_buffer_device::ptr,
					unsigned int entry_count) override
				{
					require_inputs(input_buffers, 1, "MaxSubsampling");
					// entry_count counts the entries of the output
					if (tile_count != 0)
					{
						if (entry_count % tile_count != 0)
							throw neural_network_exception("Max subsampling with tiling (layer " + layer_schema->instance_name + "): " + std::to_string(entry_count)
								+ " output entries are not a multiple of " + std::to_string(tile_count));
						hip_safe_call(nnf_hip_max_subsampling_tiling_forward(stream_id, *output_buffer, float_ptr(input_buffers[0]), entry_count / tile_count,
							input_configuration_specific_list[0].feature_map_count, static_cast<uint32_t>(input_sizes.size()),
							input_sizes.data(), windows.data(), is_min ? 1 : 0));
						return;
					}
					hip_safe_call(nnf_hip_max_subsampling_forward(stream_id, *output_buffer, float_ptr(input_buffers[0]), entry_count,
						input_configuration_specific_list[0].feature_map_count, static_cast<uint32_t>(input_sizes.size()),
						input_sizes.data(), windows.data(), strides.data(), round_ups.data(), feature_map_subsampling_size, entry_window, is_min ? 1 : 0));
				}

				bool can_apply_prologue(unsigned int prologue_input_count) const override
				{
					return (prologue_input_count == 1) && (tile_count == 0) && (entry_window == 1) && nnf_hip_max_subsampling_fusable(1, input_configuration_specific_list[0].feature_map_count, static_cast<uint32_t>(input_sizes.size()),
						input_sizes.data(), windows.data(), strides.data(), round_ups.data(), feature_map_subsampling_size, 1) == NNF_HIP_OK;
				}

				void enqueue_forward_propagation_with_prologue(void * stream_id, hip_linear_buffer_device::ptr output_buffer,
					const std::vector<hip_linear_buffer_device::const_ptr>& input_buffers, const nnf_hip_chain_desc& prologue, const float * const * chunk_ptrs,
					unsigned int entry_count) override
				{
					require_inputs(input_buffers, 1, "MaxSubsampling with layers folded in");
					hip_safe_call(nnf_hip_max_subsampling_fused_forward(stream_id, *output_buffer, float_ptr(input_buffers[0]), &prologue, chunk_ptrs, entry_count,
						input_configuration_specific_list[0].feature_map_count, static_cast<uint32_t>(input_sizes.size()),
						input_sizes.data(), windows.data(), strides.data(), round_ups.data(), feature_map_subsampling_size, 1, is_min ? 1 : 0));
				}

			protected:
				void tester_configured() override
				{
					std::shared_ptr<const max_subsampling_layer> l = std::dynamic_pointer_cast<const max_subsampling_layer>(layer_schema);
					if (!l)
						throw neural_network_exception("MaxSubsampling tester configured with a layer of type " + layer_schema->get_type_name());
					const layer_configuration_specific& in = input_configuration_specific_list.at(0);
					if ((in.get_dimension_count() < 1) || (in.get_dimension_count() > NNF_HIP_MAX_SUBSAMPLING_DIMENSIONS))
						throw neural_network_exception("The hip max subsampling tester handles 1 to 4 spatial dimensions, layer " + layer_schema->instance_name + " has " + std::to_string(in.get_dimension_count()));
					input_sizes.assign(in.dimension_sizes.begin(), in.dimension_sizes.end());
					windows.assign(l->subsampling_sizes.begin(), l->subsampling_sizes.end());
					strides.assign(l->strides.begin(), l->strides.end());
					round_ups.clear();
					for(bool r : l->round_ups)
						round_ups.push_back(r ? 1u : 0u);
					feature_map_subsampling_size = l->feature_map_subsampling_size;
					entry_window = l->entry_subsampling_size;
					tile_count = l->tiling ? static_cast<unsigned int>(l->get_tiling_factor()) : 0;
					is_min = l->is_min;
				}

			private:
				std::vector<uint32_t> input_sizes, windows, strides, round_ups;
				unsigned int feature_map_subsampling_size = 1, entry_window = 1;
				unsigned int tile_count = 0; // 0: no tiling
				bool is_min = false;
			};

			template<class LAYER, class TESTER>
			class simple_testing_schema : public layer_testing_schema
			{
			public:
				std::string get_type_name() const override { return LAYER::layer_type_name; }

			protected:
				layer_testing_schema::ptr create_specific() const override
				{
					return layer_testing_schema::ptr(new simple_testing_schema<LAYER, TESTER>());
				}

				layer_tester_hip::ptr create_tester_specific(const std::vector<layer_configuration_specific>&, const layer_configuration_specific&,
					const hip_running_configuration&) const override
				{
					return layer_tester_hip::ptr(new TESTER());
				}
			};

			template<class LAYER, class TESTER> void register_tester()
			{
				layer_testing_schema_factory::get_singleton().register_layer_testing_schema(
					layer_testing_schema::const_ptr(new simple_testing_schema<LAYER, TESTER>()));
			}
		}

		// used by the fusion pass
		bool get_add_alpha(const layer_tester_hip& tester, float& alpha)
		{
			const add_layer_tester_hip * t = dynamic_cast<const add_layer_tester_hip *>(&tester);
			if (t == nullptr)
				return false;
			alpha = t->get_alpha();
			return true;
		}

		void init()
		{
			nnforge::init();
			register_tester<batch_norm_layer, batch_norm_layer_tester_hip>();
			register_tester<rectified_linear_layer, rectified_linear_layer_tester_hip>();
			register_tester<parametric_rectified_linear_layer, parametric_rectified_linear_layer_tester_hip>();
			register_tester<exponential_linear_layer, exponential_linear_layer_tester_hip>();
			register_tester<sigmoid_layer, sigmoid_layer_tester_hip>();
			register_tester<hyperbolic_tangent_layer, hyperbolic_tangent_layer_tester_hip>();
			register_tester<add_layer, add_layer_tester_hip>();
			register_tester<softmax_layer, softmax_layer_tester_hip>();
			register_tester<average_subsampling_layer, average_subsampling_layer_tester_hip>();
			register_tester<absolute_layer, absolute_layer_tester_hip>();
			register_tester<dropout_layer, dropout_layer_tester_hip>();
			register_tester<concat_layer, concat_layer_tester_hip>();
			register_tester<maxout_layer, maxout_layer_tester_hip>();
			register_tester<max_subsampling_layer, max_subsampling_layer_tester_hip>();
		}
	}
}
