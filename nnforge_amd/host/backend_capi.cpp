// C bridge over the C++ hip backend (declared in include/nnforge_hip_backend.h).
#include "nnforge_hip_backend.h"
#include "nnforge_hip/hip_backend.h"
#include "nnforge_hip/data_streams.h"

#include <fstream>

#include <cstdio>
#include <cstring>
#include <exception>
#include <sstream>

using namespace nnforge;

namespace
{
	void copy_text(const std::string& text, char * dst, size_t capacity)
	{
		if ((dst == nullptr) || (capacity == 0))
			return;
		const size_t n = std::min(text.size(), capacity - 1);
		std::memcpy(dst, text.data(), n);
		dst[n] = '\0';
	}

	network_schema parse_schema(const char * schema_text, bool keep_unregistered_layers)
	{
		hip::init(); // idempotent: registration ignores duplicates
		if (schema_text == nullptr)
			throw neural_network_exception("schema text is null");
		std::istringstream in(schema_text);
		network_schema schema;
		schema.read_proto(in, keep_unregistered_layers);
		return schema;
	}

	std::map<std::string, layer_configuration_specific> input_configs(const nnf_backend_input * inputs, uint32_t input_count)
	{
		std::map<std::string, layer_configuration_specific> res;
		for(uint32_t i = 0; i < input_count; ++i)
		{
			std::vector<unsigned int> dims(inputs[i].dimension_sizes, inputs[i].dimension_sizes + inputs[i].dimension_count);
			res[inputs[i].layer_name] = layer_configuration_specific(inputs[i].feature_map_count, dims);
		}
		return res;
	}

	void describe_plan(const hip::forward_propagation_hip& fp, std::ostream& out)
	{
		// "step: fused|single <layers> <- <inputs> @<kernel stream>[ #<run of groups launched together>][ ><Concat layer the
		// group writes into>][ =<inputs the Concat finds in place, comma separated>]"
		for(const hip::forward_step& s : fp.get_steps())
		{
			out << "step: " << (s.fused ? "fused " : "single ") << s.description() << " @" << s.stream_index;
			if (s.batch_index >= 0)
				out << " #" << s.batch_index;
			if (!s.writes_into.empty())
				out << " >" << s.writes_into;
			if (!s.inputs_in_place.empty())
			{
				out << " =";
				for(size_t i = 0; i < s.inputs_in_place.size(); ++i)
					out << (i == 0 ? "" : ",") << s.inputs_in_place[i];
			}
			out << "\n";
		}
		out << "per_entry_bytes: " << fp.get_per_entry_buffer_bytes() << "\n";
		out << "max_entry_count: " << fp.get_max_entry_count() << "\n";
		if (fp.get_packet_entry_count() > 0)
			out << "packet_entries: " << fp.get_packet_entry_count() << "\n"; // of the latest run()
	}

	// The caller's options as this library's structure: struct_size bytes of it are the caller's, the members behind
	// them (added since the caller was built) are zero, which is every member's "default" value.
	const nnf_backend_options * checked_options(const nnf_backend_options * caller_options, nnf_backend_options& storage)
	{
		if (caller_options == nullptr)
			return nullptr;
		if ((caller_options->struct_size < 2 * sizeof(uint32_t)) || (caller_options->struct_size > 4096))
			throw neural_network_exception("nnf_backend_options.struct_size is " + std::to_string(caller_options->struct_size)
				+ ": set it to sizeof(nnf_backend_options) of the header the caller was built with");
		std::memset(&storage, 0, sizeof(storage));
		std::memcpy(&storage, caller_options, std::min<size_t>(caller_options->struct_size, sizeof(storage)));
		return &storage;
	}

	void apply_options(hip::factory_generator_hip& generator, const nnf_backend_options * options)
	{
		generator.apply_default_options();
		if (options != nullptr)
		{
			generator.hip_concat_in_place = options->concat_copies_every_input == 0;
			if (options->max_io_staging_mb != 0)
				generator.hip_max_io_staging_mb = std::max(0, options->max_io_staging_mb);
			generator.hip_fuse = options->fuse != 0;
			generator.hip_dont_share_buffers = options->dont_share_buffers != 0;
			if (options->max_entry_count > 0)
				generator.hip_max_entry_count = options->max_entry_count;
			if (options->kernel_stream_count > 0)
				generator.hip_kernel_stream_count = options->kernel_stream_count;
			generator.hip_batch_independent_groups = options->one_launch_per_group == 0;
			if (options->host_thread_count > 0)
				generator.hip_reserved_thread_count = std::max(0, static_cast<int>(get_available_processor_count()) - options->host_thread_count);
		}
		generator.initialize();
	}

	void fill_data(network_data& data, const nnf_backend_weights * weights, uint32_t weights_count, const nnf_backend_options * options)
	{
		if ((options != nullptr) && options->weights_from_folder)
			data.read(options->weights_folder);
		for(uint32_t i = 0; i < weights_count; ++i)
		{
			layer_data::ptr d(new layer_data());
			for(uint32_t c = 0; c < weights[i].chunk_count; ++c)
				d->push_back(std::vector<float>(weights[i].chunks[c], weights[i].chunks[c] + weights[i].chunk_sizes[c]));
			data.add(weights[i].layer_name, d);
		}
	}

	// hands everything on to a stat_data_bunch_writer without being one: the backend then takes the
	// general path (outputs copied back, write() per entry)
	class forwarding_writer : public structured_data_bunch_writer
	{
	public:
		explicit forwarding_writer(structured_data_bunch_writer& target) : target(target) {}
		void set_config_map(const std::map<std::string, layer_configuration_specific> config_map) override { target.set_config_map(config_map); }
		void write(unsigned int entry_id, const std::map<std::string, const float *>& data_map) override { target.write(entry_id, data_map); }
	private:
		structured_data_bunch_writer& target;
	};

	// every entry goes straight to its place in the caller's arrays
	class caller_arrays_writer : public structured_data_bunch_writer
	{
	public:
		caller_arrays_writer(nnf_backend_output * outputs, uint32_t output_count) : entries_written(output_count, 0)
		{
			for(uint32_t i = 0; i < output_count; ++i)
				by_name[outputs[i].layer_name] = std::make_pair(i, &outputs[i]);
		}
		void set_config_map(const std::map<std::string, layer_configuration_specific> config_map) override { this->config_map = config_map; }
		void write(unsigned int entry_id, const std::map<std::string, const float *>& data_map) override
		{
			for(const std::pair<const std::string, const float *>& src : data_map)
			{
				const std::pair<uint32_t, nnf_backend_output *>& dst = by_name.at(src.first);
				const size_t neuron_count = config_map.at(src.first).get_neuron_count();
				if ((static_cast<size_t>(entry_id) + 1) * neuron_count > dst.second->capacity_floats)
					throw neural_network_exception("Output buffer for layer " + src.first + " is too small: " + std::to_string(dst.second->capacity_floats) + " floats, "
						+ std::to_string((static_cast<size_t>(entry_id) + 1) * neuron_count) + " needed");
				std::memcpy(dst.second->data + static_cast<size_t>(entry_id) * neuron_count, src.second, neuron_count * sizeof(float));
				entries_written[dst.first] = std::max(entries_written[dst.first], entry_id + 1);
			}
		}
		size_t written_floats(uint32_t output_index) const
		{
			for(const std::pair<const std::string, std::pair<uint32_t, nnf_backend_output *> >& o : by_name)
				if (o.second.first == output_index)
					return static_cast<size_t>(entries_written[output_index]) * (config_map.count(o.first) ? config_map.at(o.first).get_neuron_count() : 0);
			return 0;
		}
		std::map<std::string, layer_configuration_specific> config_map;

	private:
		std::map<std::string, std::pair<uint32_t, nnf_backend_output *> > by_name;
		std::vector<unsigned int> entries_written;
	};

	template<class F> int guarded(F f, char * report, size_t report_capacity)
	{
		try
		{
			std::ostringstream out;
			f(out);
			copy_text(out.str(), report, report_capacity);
			return 0;
		}
		catch (const hip::neural_network_hip_exception& e)
		{
			copy_text(e.what(), report, report_capacity);
			return (e.error_code != 0) ? e.error_code : 1;
		}
		catch (const std::exception& e)
		{
			copy_text(e.what(), report, report_capacity);
			return 1;
		}
	}
}

extern "C"
{
	int nnf_backend_run_schema(
		const char* schema_text,
		const nnf_backend_weights* weights, uint32_t weights_count,
		const nnf_backend_input* inputs, uint32_t input_count,
		uint32_t entry_count,
		nnf_backend_output* outputs, uint32_t output_count,
		const nnf_backend_options* caller_options,
		char* report, size_t report_capacity)
	{
		return guarded([&](std::ostream& out)
		{
			nnf_backend_options option_storage;
			const nnf_backend_options * const options = checked_options(caller_options, option_storage);
			const network_schema schema = parse_schema(schema_text, (options != nullptr) && (options->keep_unregistered_layers != 0));
			if ((outputs == nullptr) || (output_count == 0))
				throw neural_network_exception("No output layers specified for forward_propagation");

			hip::factory_generator_hip generator;
			apply_options(generator, options);
			forward_propagation_factory::ptr factory = generator.create_forward_propagation_factory();

			std::vector<std::string> output_names;
			for(uint32_t i = 0; i < output_count; ++i)
				output_names.push_back(outputs[i].layer_name);
			const bool profile = (options != nullptr) && (options->profile != 0);
			forward_propagation::ptr fp = factory->create(schema, output_names, debug_state::ptr(new debug_state(false)), profile_state::ptr(new profile_state(profile, (profile && (options->profile_folder != nullptr)) ? options->profile_folder : "")));

			network_data data;
			if ((options != nullptr) && options->weights_from_folder)
				data.read(options->weights_folder);
			for(uint32_t i = 0; i < weights_count; ++i)
			{
				layer_data::ptr d(new layer_data());
				for(uint32_t c = 0; c < weights[i].chunk_count; ++c)
					d->push_back(std::vector<float>(weights[i].chunks[c], weights[i].chunks[c] + weights[i].chunk_sizes[c]));
				data.add(weights[i].layer_name, d);
			}
			fp->set_data(data);

			memory_data_bunch_reader reader(entry_count);
			const std::map<std::string, layer_configuration_specific> configs = input_configs(inputs, input_count);
			for(uint32_t i = 0; i < input_count; ++i)
				reader.add(inputs[i].layer_name, configs.find(inputs[i].layer_name)->second, inputs[i].data);
			caller_arrays_writer writer(outputs, output_count);
			const forward_propagation::stat st = fp->run(reader, writer);

			for(uint32_t i = 0; i < output_count; ++i)
			{
				outputs[i].written_floats = writer.written_floats(i);
				out << "output: " << outputs[i].layer_name << " " << writer.config_map[outputs[i].layer_name] << "\n";
			}

			const hip::forward_propagation_hip * hfp = dynamic_cast<const hip::forward_propagation_hip *>(fp.get());
			if (hfp != nullptr)
				describe_plan(*hfp, out);
			out << "entries: " << st.entry_processed_count << "\n";
			out << "stat: " << st << "\n";
			for(const std::pair<const layer_name_with_action, float>& a : fp->get_last_action_seconds())
				out << "seconds: " << fp->get_action_layer_names(a.first) << " " << a.second << "\n";
		}, report, report_capacity);
	}

	int nnf_backend_run_dataset(
		const char* schema_text,
		const nnf_backend_weights* weights, uint32_t weights_count,
		const nnf_backend_dataset_file* inputs, uint32_t input_count,
		const nnf_backend_dataset_file* outputs, uint32_t output_count,
		uint32_t compact_samples,
		const nnf_backend_options* caller_options,
		char* report, size_t report_capacity)
	{
		return guarded([&](std::ostream& out)
		{
			nnf_backend_options option_storage;
			const nnf_backend_options * const options = checked_options(caller_options, option_storage);
			const network_schema schema = parse_schema(schema_text, (options != nullptr) && (options->keep_unregistered_layers != 0));
			if ((outputs == nullptr) || (output_count == 0))
				throw neural_network_exception("No output layers specified for forward_propagation");
			std::vector<std::string> output_names;
			for(uint32_t i = 0; i < output_count; ++i)
				output_names.push_back(outputs[i].layer_name);

			hip::factory_generator_hip generator;
			apply_options(generator, options);
			forward_propagation::ptr fp = generator.create_forward_propagation_factory()->create(schema, output_names,
				debug_state::ptr(new debug_state(false)), profile_state::ptr(new profile_state(false)));
			network_data data;
			fill_data(data, weights, weights_count, options);
			fp->set_data(data);

			// the reader toolset::get_structured_data_bunch_reader builds (nnforge/toolset.cpp:659-678): a file per data
			// layer, and the constant 1 for a data layer called dataset_value
			std::map<std::string, structured_data_reader::ptr> readers;
			for(uint32_t i = 0; i < input_count; ++i)
			{
				std::shared_ptr<std::istream> in(new std::ifstream(inputs[i].path, std::ios_base::in | std::ios_base::binary));
				if (!*in)
					throw neural_network_exception(std::string("Cannot open ") + inputs[i].path);
				readers[inputs[i].layer_name] = structured_data_reader::ptr(new structured_data_stream_reader(in));
			}
			readers["dataset_value"] = structured_data_reader::ptr(new structured_data_constant_reader(1.0F, layer_configuration_specific(1)));
			structured_data_bunch_stream_reader reader(readers);

			neuron_value_set_data_bunch_writer writer;
			const forward_propagation::stat st = fp->run(reader, writer);

			// what run_inference does in its dump mode (nnforge/toolset.cpp:592-650): fold the samples of an entry, write a file per layer
			for(uint32_t i = 0; i < output_count; ++i)
			{
				std::pair<layer_configuration_specific, neuron_value_set::ptr>& res = writer.layer_name_to_config_and_value_set_map.at(outputs[i].layer_name);
				res.second->compact((compact_samples == 0) ? 1 : compact_samples);
				std::shared_ptr<std::ostream> file(new std::ofstream(outputs[i].path, std::ios_base::out | std::ios_base::trunc | std::ios_base::binary));
				if (!*file)
					throw neural_network_exception(std::string("Cannot open ") + outputs[i].path + " for writing");
				{
					structured_data_stream_writer dw(file, res.first);
					unsigned int entry_id = 0;
					for(const std::shared_ptr<std::vector<float> >& entry : res.second->neuron_value_list)
						dw.write(entry_id++, entry->data());
				}
				out << "output: " << outputs[i].layer_name << " " << res.first << " entries " << res.second->neuron_value_list.size() << "\n";
			}
			const hip::forward_propagation_hip * hfp = dynamic_cast<const hip::forward_propagation_hip *>(fp.get());
			if (hfp != nullptr)
				describe_plan(*hfp, out);
			out << "entries: " << st.entry_processed_count << "\n";
			out << "stat: " << st << "\n";
		}, report, report_capacity);
	}

	int nnf_backend_rewrite_dataset(const char* in_path, const char* out_path, uint32_t compact_samples, uint32_t part_count, uint32_t part,
		char* report, size_t report_capacity)
	{
		return guarded([&](std::ostream& out)
		{
			if ((in_path == nullptr) || (out_path == nullptr))
				throw neural_network_exception("dataset path is null");
			std::shared_ptr<std::istream> in(new std::ifstream(in_path, std::ios_base::in | std::ios_base::binary));
			if (!*in)
				throw neural_network_exception(std::string("Cannot open ") + in_path);
			std::map<std::string, structured_data_reader::ptr> readers;
			readers["data"] = structured_data_reader::ptr(new structured_data_stream_reader(in));
			structured_data_bunch_stream_reader reader(readers, (part_count == 0) ? 1 : part_count);
			reader.set_epoch(part);
			const layer_configuration_specific config = reader.get_config_map().at("data");

			neuron_value_set values(config.get_neuron_count());
			std::vector<float> entry(config.get_neuron_count());
			std::map<std::string, float *> data_map;
			data_map["data"] = entry.data();
			for(unsigned int entry_id = 0; reader.read(entry_id, data_map); ++entry_id)
				values.add_entry(entry.data());
			out << "config: " << config << "\n";
			out << "entries_read: " << values.neuron_value_list.size() << " of " << reader.get_entry_count() << "\n";
			if (!values.neuron_value_list.empty())
			{
				out << "average:";
				out.precision(17);
				const std::shared_ptr<std::vector<double> > average = values.get_average();
				for(double v : *average)
					out << " " << v;
				out << "\n";
			}
			values.compact((compact_samples == 0) ? 1 : compact_samples);
			std::shared_ptr<std::ostream> file(new std::ofstream(out_path, std::ios_base::out | std::ios_base::trunc | std::ios_base::binary));
			if (!*file)
				throw neural_network_exception(std::string("Cannot open ") + out_path + " for writing");
			structured_data_stream_writer dw(file, config);
			for(const std::shared_ptr<std::vector<float> >& e : values.neuron_value_list)
				dw.write(e->data());
			out << "entries_written: " << values.neuron_value_list.size() << "\n";
		}, report, report_capacity);
	}

	int nnf_backend_layer_statistics(
		const char* schema_text,
		const nnf_backend_weights* weights, uint32_t weights_count,
		const nnf_backend_input* inputs, uint32_t input_count,
		uint32_t entry_count,
		const char* layer_name, uint32_t feature_map_count,
		float* min_values, float* max_values, float* averages, float* std_devs,
		const nnf_backend_options* caller_options,
		char* report, size_t report_capacity)
	{
		return guarded([&](std::ostream& out)
		{
			nnf_backend_options option_storage;
			const nnf_backend_options * const options = checked_options(caller_options, option_storage);
			const network_schema schema = parse_schema(schema_text, (options != nullptr) && (options->keep_unregistered_layers != 0));
			if (layer_name == nullptr)
				throw neural_network_exception("No output layers specified for forward_propagation");
			hip::factory_generator_hip generator;
			apply_options(generator, options);
			forward_propagation::ptr fp = generator.create_forward_propagation_factory()->create(schema, std::vector<std::string>(1, layer_name),
				debug_state::ptr(new debug_state(false)), profile_state::ptr(new profile_state(false)));
			network_data data;
			fill_data(data, weights, weights_count, options);
			fp->set_data(data);

			memory_data_bunch_reader reader(entry_count);
			const std::map<std::string, layer_configuration_specific> configs = input_configs(inputs, input_count);
			for(uint32_t i = 0; i < input_count; ++i)
				reader.add(inputs[i].layer_name, configs.find(inputs[i].layer_name)->second, inputs[i].data);

			stat_data_bunch_writer writer;
			forward_propagation::stat st;
			if ((options != nullptr) && (options->stat_on_host != 0))
			{
				forwarding_writer through(writer);
				st = fp->run(reader, through);
			}
			else
				st = fp->run(reader, writer);

			const std::vector<feature_map_data_stat> stat = writer.get_stat().at(layer_name);
			if (stat.size() != feature_map_count)
				throw neural_network_exception("Layer " + std::string(layer_name) + " has " + std::to_string(stat.size()) + " feature maps, room for " + std::to_string(feature_map_count) + " supplied");
			for(size_t f = 0; f < stat.size(); ++f)
			{
				min_values[f] = stat[f].min;
				max_values[f] = stat[f].max;
				averages[f] = stat[f].average;
				std_devs[f] = stat[f].std_dev;
			}
			out << "entries: " << st.entry_processed_count << "\n";
			out << "writer_entries: " << writer.get_entry_count() << "\n";
		}, report, report_capacity);
	}

	int nnf_backend_update_bn_weights(
		const char* schema_text,
		const nnf_backend_weights* weights, uint32_t weights_count,
		const nnf_backend_input* inputs, uint32_t input_count,
		uint32_t entry_count,
		const nnf_backend_options* caller_options,
		const char* out_folder,
		char* report, size_t report_capacity)
	{
		return guarded([&](std::ostream& out)
		{
			nnf_backend_options option_storage;
			const nnf_backend_options * const options = checked_options(caller_options, option_storage);
			const network_schema schema = parse_schema(schema_text, (options != nullptr) && (options->keep_unregistered_layers != 0));
			if (out_folder == nullptr)
				throw neural_network_exception("No folder given for the refreshed weights");
			hip::factory_generator_hip generator;
			apply_options(generator, options);
			forward_propagation_factory::ptr factory = generator.create_forward_propagation_factory();
			network_data data;
			fill_data(data, weights, weights_count, options);

			memory_data_bunch_reader reader(entry_count);
			const std::map<std::string, layer_configuration_specific> configs = input_configs(inputs, input_count);
			for(uint32_t i = 0; i < input_count; ++i)
				reader.add(inputs[i].layer_name, configs.find(inputs[i].layer_name)->second, inputs[i].data);

			update_bn_weights(schema, data, reader, *factory, debug_state::ptr(), profile_state::ptr(), &out);
			data.write(out_folder);
		}, report, report_capacity);
	}

	int nnf_backend_plan_schema(
		const char* schema_text,
		const nnf_backend_input* inputs, uint32_t input_count,
		const char* const* output_layer_names, uint32_t output_count,
		const nnf_backend_options* caller_options,
		uint64_t memory_bytes,
		char* report, size_t report_capacity)
	{
		return guarded([&](std::ostream& out)
		{
			nnf_backend_options option_storage;
			const nnf_backend_options * const options = checked_options(caller_options, option_storage);
			const network_schema schema = parse_schema(schema_text, (options != nullptr) && (options->keep_unregistered_layers != 0));
			std::vector<std::string> output_names;
			for(uint32_t i = 0; i < output_count; ++i)
				output_names.push_back(output_layer_names[i]);
			const bool fuse = (options == nullptr) || (options->fuse != 0);
			const bool dont_share = (options != nullptr) && (options->dont_share_buffers != 0);
			const int max_entries = ((options != nullptr) && (options->max_entry_count > 0)) ? options->max_entry_count : 4096;
			const int kernel_streams = ((options != nullptr) && (options->kernel_stream_count > 0)) ? options->kernel_stream_count : hip::hip_running_configuration::default_kernel_stream_count;
			const bool batch = (options == nullptr) || (options->one_launch_per_group == 0);
			std::shared_ptr<hip::hip_running_configuration> offline = std::const_pointer_cast<hip::hip_running_configuration>(
				hip::hip_running_configuration::create_offline(memory_bytes, 0.9F, fuse, dont_share, max_entries, kernel_streams, batch));
			offline->concat_in_place = (options == nullptr) || (options->concat_copies_every_input == 0);
			hip::hip_running_configuration::const_ptr config = offline;
			hip::forward_propagation_hip fp(schema, output_names, debug_state::ptr(new debug_state(false)), profile_state::ptr(new profile_state(false)), config);
			fp.set_input_configuration_specific(input_configs(inputs, input_count));
			describe_plan(fp, out);
		}, report, report_capacity);
	}

	int nnf_backend_time_kernels(
		const char* schema_text,
		const nnf_backend_weights* weights, uint32_t weights_count,
		const nnf_backend_input* inputs, uint32_t input_count,
		uint32_t entry_count,
		const char* const* output_layer_names, uint32_t output_count,
		const nnf_backend_options* caller_options,
		uint32_t warmup, uint32_t passes,
		char* report, size_t report_capacity)
	{
		return guarded([&](std::ostream& out)
		{
			nnf_backend_options option_storage;
			const nnf_backend_options * const options = checked_options(caller_options, option_storage);
			const network_schema schema = parse_schema(schema_text, (options != nullptr) && (options->keep_unregistered_layers != 0));
			std::vector<std::string> output_names;
			for(uint32_t i = 0; i < output_count; ++i)
				output_names.push_back(output_layer_names[i]);
			hip::factory_generator_hip generator;
			apply_options(generator, options);
			forward_propagation::ptr fp = generator.create_forward_propagation_factory()->create(schema, output_names,
				debug_state::ptr(new debug_state(false)), profile_state::ptr(new profile_state(false)));
			network_data data;
			fill_data(data, weights, weights_count, options);
			fp->set_data(data);

			memory_data_bunch_reader reader(entry_count);
			const std::map<std::string, layer_configuration_specific> configs = input_configs(inputs, input_count);
			for(uint32_t i = 0; i < input_count; ++i)
				reader.add(inputs[i].layer_name, configs.find(inputs[i].layer_name)->second, inputs[i].data);
			hip::forward_propagation_hip * hfp = dynamic_cast<hip::forward_propagation_hip *>(fp.get());
			if (hfp == nullptr)
				throw neural_network_exception("The factory did not make a forward_propagation_hip");
			const unsigned int resident_packets = ((options != nullptr) && (options->resident_packets > 0)) ? static_cast<unsigned int>(options->resident_packets) : 1U;
			const hip::forward_propagation_hip::kernel_timing t = hfp->time_kernels(reader, entry_count, warmup, passes, resident_packets,
				(options != nullptr) && (options->replay_recorded_plan != 0));
			describe_plan(*hfp, out);
			out << "launches: " << t.launch_count << "\n";
			out << "plan_steps: " << t.plan_step_count << "\n";
			out << "resident_packets: " << t.resident_packets << "\n";
			out << "timed_entries: " << t.entry_count << "\n";
			out.precision(9);
			out << "wall_seconds_per_pass: " << t.wall_seconds_per_pass << "\n";
			out << "device_seconds_per_pass: " << t.device_seconds_per_pass << "\n";
			out << "host_seconds_per_pass: " << t.host_seconds_per_pass << "\n";
		}, report, report_capacity);
	}

	int nnf_backend_list_layers(const char* schema_text, int32_t keep_unregistered_layers, char* report, size_t report_capacity)
	{
		return guarded([&](std::ostream& out)
		{
			const network_schema schema = parse_schema(schema_text, keep_unregistered_layers != 0);
			for(const layer::const_ptr& l : schema.get_layers_in_forward_propagation_order())
			{
				out << "layer: " << l->get_type_name() << "\t" << l->instance_name << "\t";
				for(size_t i = 0; i < l->input_layer_instance_names.size(); ++i)
					out << (i == 0 ? "" : ",") << l->input_layer_instance_names[i];
				out << "\t";
				const std::vector<std::string> params = l->get_parameter_strings();
				for(size_t i = 0; i < params.size(); ++i)
					out << (i == 0 ? "" : "; ") << params[i];
				out << "\t" << ((dynamic_cast<const external_layer *>(l.get()) != nullptr) ? "external" : "own") << "\n";
			}
		}, report, report_capacity);
	}

	int nnf_backend_rewrite_schema(const char* schema_text, int32_t keep_unregistered_layers, char* out_text, size_t out_capacity)
	{
		return guarded([&](std::ostream& out)
		{
			const network_schema schema = parse_schema(schema_text, keep_unregistered_layers != 0);
			std::ostringstream text;
			schema.write_proto(text);
			// the text is the result: cut short it would be a different schema
			if (text.str().size() + 1 > out_capacity)
				throw neural_network_exception("The schema text takes " + std::to_string(text.str().size() + 1) + " bytes, the buffer holds " + std::to_string(out_capacity));
			out << text.str();
		}, out_text, out_capacity);
	}

	int nnf_backend_write_weights(const char* folder, const nnf_backend_weights* weights, uint32_t weights_count, char* report, size_t report_capacity)
	{
		return guarded([&](std::ostream&)
		{
			network_data data;
			for(uint32_t i = 0; i < weights_count; ++i)
			{
				layer_data::ptr d(new layer_data());
				for(uint32_t c = 0; c < weights[i].chunk_count; ++c)
					d->push_back(std::vector<float>(weights[i].chunks[c], weights[i].chunks[c] + weights[i].chunk_sizes[c]));
				data.add(weights[i].layer_name, d);
			}
			data.write(folder);
		}, report, report_capacity);
	}

	int nnf_backend_read_weights(const char* folder, const char* layer_name, uint32_t chunk_count, const uint32_t* chunk_sizes, float* const* chunks, char* report, size_t report_capacity)
	{
		return guarded([&](std::ostream&)
		{
			network_data data;
			data.read(folder);
			layer_data::ptr d = data.get(layer_name);
			if (d->size() != chunk_count)
				throw neural_network_exception("data weight vector count " + std::to_string(d->size()) + " doesn't satisfy layer configuration " + std::to_string(chunk_count));
			for(uint32_t c = 0; c < chunk_count; ++c)
			{
				if ((*d)[c].size() != chunk_sizes[c])
					throw neural_network_exception("data weight count " + std::to_string((*d)[c].size()) + " for vector " + std::to_string(c) + " doesn't satisfy layer configuration " + std::to_string(chunk_sizes[c]));
				std::memcpy(chunks[c], (*d)[c].data(), chunk_sizes[c] * sizeof(float));
			}
		}, report, report_capacity);
	}
}
