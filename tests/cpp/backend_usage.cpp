// The hip backend used from C++ the way an nnForge application uses a backend
// (examples/gtsrb/gtsrb.cpp:29-63 + toolset::run_inference, nnforge/toolset.cpp:551-575):
// factory_generator -> forward_propagation_factory -> forward_propagation, a schema in text
// format, weights as network_data, a reader and a writer. Prints "ok" when the network's output
// equals a straightforward host evaluation of the same layers bit for bit.
#include <nnforge_hip/hip_backend.h>
#include <nnforge_hip/data_streams.h>

#include <fstream>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <iostream>
#include <random>
#include <sstream>

using namespace nnforge;

namespace
{
	const char * schema_text = R"(
name: "usage"
layer { type: "Data" name: "conv_main" }
layer { type: "Data" name: "conv_shortcut" }
layer { type: "BatchNorm" name: "main_bn" input_layer_name: "conv_main" batch_norm_param { feature_map_count: 6 } }
layer { type: "Add" name: "res" input_layer_name: "conv_shortcut" input_layer_name: "main_bn" }
layer { type: "PReLU" name: "res_prelu" input_layer_name: "res" prelu_param { feature_map_count: 6 } }
layer { type: "AverageSubsampling" name: "pool" input_layer_name: "res_prelu"
	average_subsampling_param { dimension_param { subsampling_size: 7 } dimension_param { subsampling_size: 7 } alpha: 0.0204081628 } }
layer { type: "Softmax" name: "prob" input_layer_name: "pool" }
)";

	// a reader that produces entries on the fly and ends after entry_count entries
	class generated_reader : public structured_data_bunch_reader
	{
	public:
		generated_reader(unsigned int entry_count, const layer_configuration_specific& config) : entry_count(entry_count), config(config) {}
		std::map<std::string, layer_configuration_specific> get_config_map() const override
		{
			std::map<std::string, layer_configuration_specific> res;
			res["conv_main"] = config;
			res["conv_shortcut"] = config;
			return res;
		}
		static float value(unsigned int entry_id, unsigned int layer, unsigned int i)
		{
			return std::sin(0.37f * static_cast<float>(i + 31 * entry_id) + 1.3f * static_cast<float>(layer)) * 2.0f;
		}
		bool read(unsigned int entry_id, const std::map<std::string, float *>& data_map) override
		{
			if (entry_id >= entry_count)
				return false;
			for(const std::pair<const std::string, float *>& item : data_map)
				for(unsigned int i = 0; i < config.get_neuron_count(); ++i)
					item.second[i] = value(entry_id, item.first == "conv_main" ? 0 : 1, i);
			return true;
		}
		int get_entry_count() const override { return -1; } // unknown: the driver has to find the end

	private:
		unsigned int entry_count;
		layer_configuration_specific config;
	};
}

int main(int argc, char ** argv)
{
	try
	{
		hip::factory_generator_hip generator;
		generator.apply_default_options();
		generator.hip_max_entry_count = 5; // several packets
		generator.initialize();
		generator.info();

		network_schema schema;
		std::istringstream in(schema_text);
		schema.read_proto(in);

		const unsigned int c = 6, entries = 13;
		network_data data(schema.get_layers());
		data.initialize(schema.get_layers());
		std::mt19937 gen(7);
		std::uniform_real_distribution<float> dist(0.5F, 1.5F);
		for(std::vector<float>& chunk : *data.get("main_bn"))
			for(float& v : chunk)
				v = dist(gen);
		for(float& v : (*data.get("res_prelu"))[0])
			v = dist(gen) * 0.2F;

		std::vector<std::string> outputs;
		outputs.push_back("prob");
		outputs.push_back("res_prelu");
		forward_propagation::ptr fp = generator.create_forward_propagation_factory()->create(
			schema, outputs, debug_state::ptr(new debug_state(true)), profile_state::ptr(new profile_state(true)));
		fp->set_data(data);

		const layer_configuration_specific config(c, std::vector<unsigned int>(2, 7));
		generated_reader reader(entries, config);
		memory_data_bunch_writer writer;
		const forward_propagation::stat st = fp->run(reader, writer);
		std::cout << st << std::endl;
		if (st.entry_processed_count != entries)
		{
			std::cout << "processed " << st.entry_processed_count << " entries, expected " << entries << std::endl;
			return 1;
		}

		// host evaluation, same operation order (compiled without contraction)
		const layer_data& bn = *data.get("main_bn");
		const std::vector<float>& slopes = (*data.get("res_prelu"))[0];
		unsigned int mismatches = 0;
		for(unsigned int e = 0; e < entries; ++e)
		{
			float pooled[6];
			for(unsigned int f = 0; f < c; ++f)
			{
				const float mult = bn[0][f] * bn[3][f];
				const float add = bn[1][f] - mult * bn[2][f];
				float sum = 0.0F;
				for(unsigned int p = 0; p < 49; ++p)
				{
					const unsigned int i = f * 49 + p;
					const float main_v = generated_reader::value(e, 0, i) * mult + add;
					float r = 0.0F;
					r += generated_reader::value(e, 1, i);
					r += main_v;
					r = r * 1.0F;
					const float y = r * (r >= 0.0F ? 1.0F : slopes[f]);
					const float got = writer.values["res_prelu"][static_cast<size_t>(e) * c * 49 + i];
					if (std::memcmp(&got, &y, 4) != 0)
						++mismatches;
					sum += y;
				}
				pooled[f] = sum * 0.0204081628F;
			}
			float max_val = -1.0e+37F;
			for(unsigned int f = 0; f < c; ++f)
				max_val = std::max(max_val, pooled[f]);
			float ex[6], sum = 0.0F;
			for(unsigned int f = 0; f < c; ++f)
			{
				ex[f] = expf(pooled[f] - max_val);
				sum += ex[f];
			}
			const float mult = 1.0F / sum;
			for(unsigned int f = 0; f < c; ++f)
			{
				const float want = ex[f] * mult;
				const float got = writer.values["prob"][static_cast<size_t>(e) * c + f];
				if (std::fabs(got - want) > 1.0e-5F * want)
					++mismatches;
			}
		}
		for(const std::pair<const layer_name_with_action, float>& a : fp->get_last_action_seconds())
			std::cout << "action " << a.first.get_name() << " " << a.first.get_action().str() << " (" << fp->get_action_layer_names(a.first) << "): " << a.second << " s" << std::endl;
		if (mismatches != 0)
		{
			std::cout << mismatches << " mismatches" << std::endl;
			return 1;
		}

		// what the reference's classes throw, the backend throws too
		try
		{
			generator.create_backward_propagation_factory();
			std::cout << "backward propagation did not throw" << std::endl;
			return 1;
		}
		catch (const neural_network_exception&)
		{
		}

		// a reader that fails in the middle of a run: the exception reaches the caller, nothing is freed
		// under a copy or kernel still in flight, and the same object runs again afterwards
		class failing_reader : public generated_reader
		{
		public:
			using generated_reader::generated_reader;
			bool read(unsigned int entry_id, const std::map<std::string, float *>& data_map) override
			{
				if (entry_id == 8)
					throw neural_network_exception("reader failed at entry 8");
				return generated_reader::read(entry_id, data_map);
			}
		};
		try
		{
			failing_reader bad(entries, config);
			memory_data_bunch_writer sink;
			fp->run(bad, sink);
			std::cout << "failing reader did not throw" << std::endl;
			return 1;
		}
		catch (const neural_network_exception& e)
		{
			if (std::string(e.what()).find("entry 8") == std::string::npos)
			{
				std::cout << "unexpected exception: " << e.what() << std::endl;
				return 1;
			}
		}
		{
			memory_data_bunch_writer again;
			fp->run(reader, again);
			if (again.values["res_prelu"] != writer.values["res_prelu"])
			{
				std::cout << "run after a failed run differs" << std::endl;
				return 1;
			}
		}

		// the same data from data set files, the way toolset::run_inference reads and collects it: bits as before
		{
			const std::string folder = (argc > 1) ? argv[1] : ".";
			std::map<std::string, structured_data_reader::ptr> file_readers;
			for(const char * layer_name : { "conv_main", "conv_shortcut" })
			{
				const std::string path = folder + "/" + layer_name + ".dt";
				{
					std::shared_ptr<std::ostream> file(new std::ofstream(path, std::ios_base::out | std::ios_base::trunc | std::ios_base::binary));
					structured_data_stream_writer dw(file, config);
					std::vector<float> entry(config.get_neuron_count());
					std::map<std::string, float *> one;
					one[layer_name] = entry.data();
					for(unsigned int entry_id = 0; reader.read(entry_id, one); ++entry_id)
						dw.write(entry_id, entry.data());
				}
				file_readers[layer_name] = structured_data_reader::ptr(new structured_data_stream_reader(
					std::shared_ptr<std::istream>(new std::ifstream(path, std::ios_base::in | std::ios_base::binary))));
			}
			structured_data_bunch_stream_reader from_files(file_readers);
			if (from_files.get_entry_count() != static_cast<int>(entries))
			{
				std::cout << "data set files hold " << from_files.get_entry_count() << " entries, expected " << entries << std::endl;
				return 1;
			}
			neuron_value_set_data_bunch_writer collected;
			fp->run(from_files, collected);
			for(const char * layer_name : { "prob", "res_prelu" })
			{
				const neuron_value_set& got = *collected.layer_name_to_config_and_value_set_map.at(layer_name).second;
				const std::vector<float>& want = writer.values[layer_name];
				bool same = got.neuron_value_list.size() == entries;
				for(unsigned int e = 0; same && (e < entries); ++e)
					same = std::memcmp(got.neuron_value_list[e]->data(), want.data() + static_cast<size_t>(e) * got.neuron_count, got.neuron_count * sizeof(float)) == 0;
				if (!same)
				{
					std::cout << "run from data set files differs for " << layer_name << std::endl;
					return 1;
				}
			}
		}

		// One object, run after run: what a run allocated is used again by the next one and must follow new
		// weights and another kind of writer. Reference: a fresh object with the new weights.
		{
			network_data other(schema.get_layers(), data);
			layer_data::ptr steeper(new layer_data(*data.get("res_prelu")));
			for(float& v : (*steeper)[0])
				v *= 3.0F;
			other.add("res_prelu", steeper);
			forward_propagation::ptr fresh = generator.create_forward_propagation_factory()->create(
				schema, outputs, debug_state::ptr(), profile_state::ptr());
			fresh->set_data(other);
			memory_data_bunch_writer want;
			fresh->run(reader, want);
			if (want.values["res_prelu"] == writer.values["res_prelu"])
			{
				std::cout << "other slopes, same output: the check checks nothing" << std::endl;
				return 1;
			}
			fp->set_data(other);
			memory_data_bunch_writer got;
			fp->run(reader, got);
			stat_data_bunch_writer statistics_between;
			fp->run(reader, statistics_between);
			memory_data_bunch_writer got_again;
			fp->run(reader, got_again);
			if ((got.values != want.values) || (got_again.values != want.values) || (statistics_between.get_entry_count() != entries))
			{
				std::cout << "runs of one object after new weights / another writer differ from a fresh object" << std::endl;
				return 1;
			}
			fp->set_data(data);
		}

		// toolset::update_bn_weights as a library call: afterwards the batch norm output, taken with
		// gamma 1 and beta 0, has mean 0 and deviation 1 over the reader's data
		update_bn_weights(schema, data, reader, *generator.create_forward_propagation_factory(), debug_state::ptr(), profile_state::ptr(), nullptr);
		{
			network_data probe_data(schema.get_layers(), data); // shares the layers' weights with data ...
			layer_data::ptr plain_bn(new layer_data(*data.get("main_bn"))); // ... so the modified layer gets its own copy
			std::fill((*plain_bn)[0].begin(), (*plain_bn)[0].end(), 1.0F);
			std::fill((*plain_bn)[1].begin(), (*plain_bn)[1].end(), 0.0F);
			probe_data.add("main_bn", plain_bn);
			forward_propagation::ptr probe = generator.create_forward_propagation_factory()->create(
				schema, std::vector<std::string>(1, "main_bn"), debug_state::ptr(), profile_state::ptr());
			probe->set_data(probe_data);
			stat_data_bunch_writer stat_writer;
			probe->run(reader, stat_writer);
			const std::vector<feature_map_data_stat> after = stat_writer.get_stat().at("main_bn");
			for(const feature_map_data_stat& st2 : after)
			{
				std::cout << st2 << std::endl;
				if ((std::fabs(st2.average) > 1.0e-5F) || (std::fabs(st2.std_dev - 1.0F) > 1.0e-5F))
				{
					std::cout << "batch norm output is not normalised after update_bn_weights" << std::endl;
					return 1;
				}
			}
			if (stat_writer.get_entry_count() != entries)
			{
				std::cout << "statistics over " << stat_writer.get_entry_count() << " entries, expected " << entries << std::endl;
				return 1;
			}
		}
		std::cout << "ok" << std::endl;
		return 0;
	}
	catch (const std::exception& e)
	{
		std::cout << "exception: " << e.what() << std::endl;
		return 1;
	}
}
