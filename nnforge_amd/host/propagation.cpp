#include "nnforge_hip/propagation.h"

#include <algorithm>
#include <cmath>
#include <limits>
#include <chrono>
#include <cstdio>
#include <cstring>
#include <condition_variable>
#include <deque>
#include <fstream>
#include <mutex>
#include <thread>

#include <sched.h>

namespace nnforge
{
	struct threadpool_job_runner::impl
	{
		std::mutex m;
		std::condition_variable wake;
		std::deque<std::function<void()> > jobs;
		bool stopping = false;
		std::vector<std::thread> threads;

		void work()
		{
			for(;;)
			{
				std::function<void()> job;
				{
					std::unique_lock<std::mutex> lock(m);
					wake.wait(lock, [this]() { return stopping || !jobs.empty(); });
					if (jobs.empty())
						return; // stopping and nothing left
					job = std::move(jobs.front());
					jobs.pop_front();
				}
				job();
			}
		}
	};

	threadpool_job_runner::threadpool_job_runner(unsigned int thread_count)
		: thread_count(std::max(1U, thread_count))
		, p(new impl())
	{
		for(unsigned int i = 0; i < this->thread_count; ++i)
			p->threads.emplace_back(&impl::work, p.get());
	}

	threadpool_job_runner::~threadpool_job_runner()
	{
		{
			std::lock_guard<std::mutex> lock(p->m);
			p->stopping = true;
		}
		p->wake.notify_all();
		for(std::thread& t : p->threads)
			t.join();
	}

	void threadpool_job_runner::post(std::function<void()> job)
	{
		{
			std::lock_guard<std::mutex> lock(p->m);
			p->jobs.push_back(std::move(job));
		}
		p->wake.notify_one();
	}

	unsigned int get_available_processor_count()
	{
		cpu_set_t set;
		CPU_ZERO(&set);
		if (sched_getaffinity(0, sizeof(set), &set) == 0)
		{
			const int allowed = CPU_COUNT(&set);
			if (allowed > 0)
				return static_cast<unsigned int>(allowed);
		}
		return std::max(1U, std::thread::hardware_concurrency());
	}

	// ---- in-memory reader / writer ---------------------------------------------------------

	void memory_data_bunch_reader::add(const std::string& layer_name, const layer_configuration_specific& config, const float * data_ptr)
	{
		config_map[layer_name] = config;
		data[layer_name] = data_ptr;
	}

	bool memory_data_bunch_reader::read(unsigned int entry_id, const std::map<std::string, float *>& data_map)
	{
		if (entry_id >= entry_count)
			return false;
		for(const std::pair<const std::string, float *>& dst : data_map)
		{
			std::map<std::string, const float *>::const_iterator src = data.find(dst.first);
			if (src == data.end())
				throw neural_network_exception("No data supplied for layer " + dst.first);
			const size_t neuron_count = config_map.find(dst.first)->second.get_neuron_count();
			std::memcpy(dst.second, src->second + static_cast<size_t>(entry_id) * neuron_count, neuron_count * sizeof(float));
		}
		return true;
	}

	void memory_data_bunch_writer::set_config_map(const std::map<std::string, layer_configuration_specific> new_config_map)
	{
		config_map = new_config_map;
		values.clear();
		entry_count = 0;
	}

	void memory_data_bunch_writer::write(unsigned int entry_id, const std::map<std::string, const float *>& data_map)
	{
		for(const std::pair<const std::string, const float *>& src : data_map)
		{
			const size_t neuron_count = config_map[src.first].get_neuron_count();
			std::vector<float>& dst = values[src.first];
			if (dst.size() < (static_cast<size_t>(entry_id) + 1) * neuron_count)
				dst.resize((static_cast<size_t>(entry_id) + 1) * neuron_count);
			std::memcpy(dst.data() + static_cast<size_t>(entry_id) * neuron_count, src.second, neuron_count * sizeof(float));
		}
		if (entry_id + 1 > entry_count)
			entry_count = entry_id + 1;
	}

	// ---- statistics writer ------------------------------------------------------------------

	std::ostream& operator<< (std::ostream& out, const feature_map_data_stat& val)
	{
		out << "Average " << val.average << ", StdDev " << val.std_dev << ", Min " << val.min << ", Max " << val.max;
		return out;
	}

	stat_data_bunch_writer::running_stat::running_stat()
		: n(0.0), mean(0.0), m2(0.0)
		, min_val(std::numeric_limits<float>::max())
		, max_val(-std::numeric_limits<float>::max())
	{
	}

	stat_data_bunch_writer::stat_data_bunch_writer() : entry_count(0)
	{
	}

	void stat_data_bunch_writer::set_config_map(const std::map<std::string, layer_configuration_specific> new_config_map)
	{
		config_map = new_config_map;
		layer_name_to_running_stat_list_map.clear();
		for(const std::pair<const std::string, layer_configuration_specific>& item : config_map)
			layer_name_to_running_stat_list_map[item.first] = std::vector<running_stat>(item.second.feature_map_count);
	}

	void stat_data_bunch_writer::write(unsigned int, const std::map<std::string, const float *>& data_map)
	{
		for(const std::pair<const std::string, const float *>& item : data_map)
		{
			std::vector<running_stat>& stats = layer_name_to_running_stat_list_map.at(item.first);
			const unsigned int neuron_count_per_feature_map = config_map.at(item.first).get_neuron_count_per_feature_map();
			const float * data = item.second;
			for(running_stat& s : stats)
			{
				for(unsigned int i = 0; i < neuron_count_per_feature_map; ++i, ++data)
				{
					const float val = *data;
					s.min_val = std::min(s.min_val, val);
					s.max_val = std::max(s.max_val, val);
					s.n += 1.0;
					const double val_d = static_cast<double>(val);
					const double delta = val_d - s.mean;
					s.mean += delta / s.n;
					const double delta2 = val_d - s.mean;
					s.m2 += delta * delta2;
				}
			}
		}
		++entry_count;
	}

	void stat_data_bunch_writer::merge(const std::string& layer_name, const std::vector<running_stat>& partial)
	{
		std::vector<running_stat>& stats = layer_name_to_running_stat_list_map.at(layer_name);
		if (partial.size() != stats.size())
			throw neural_network_exception("Statistics of " + std::to_string(partial.size()) + " feature maps supplied for layer " + layer_name + " with " + std::to_string(stats.size()));
		for(size_t f = 0; f < stats.size(); ++f)
		{
			running_stat& s = stats[f];
			const running_stat& b = partial[f];
			if (b.n == 0.0)
				continue;
			const double n = s.n + b.n;
			const double delta = b.mean - s.mean;
			s.mean = (s.n == 0.0) ? b.mean : s.mean + delta * (b.n / n);
			s.m2 = s.m2 + b.m2 + delta * delta * (s.n * b.n / n);
			s.n = n;
			s.min_val = std::min(s.min_val, b.min_val);
			s.max_val = std::max(s.max_val, b.max_val);
		}
	}

	std::map<std::string, std::vector<feature_map_data_stat> > stat_data_bunch_writer::get_stat() const
	{
		std::map<std::string, std::vector<feature_map_data_stat> > res;
		for(const std::pair<const std::string, std::vector<running_stat> >& item : layer_name_to_running_stat_list_map)
		{
			std::vector<feature_map_data_stat> list;
			for(const running_stat& s : item.second)
			{
				feature_map_data_stat st;
				st.average = static_cast<float>(s.mean);
				st.std_dev = sqrtf(static_cast<float>(s.m2 / s.n));
				st.min = s.min_val;
				st.max = s.max_val;
				list.push_back(st);
			}
			res[item.first] = list;
		}
		return res;
	}

	void update_bn_weights(
		const network_schema& schema,
		network_data& data,
		structured_data_bunch_reader& reader,
		const forward_propagation_factory& factory,
		debug_state::ptr debug,
		profile_state::ptr profile,
		std::ostream * log)
	{
		std::vector<std::string> bn_layers;
		for(const layer::const_ptr& l : schema.get_layers_in_forward_propagation_order())
			if (l->get_type_name() == "BatchNorm")
				bn_layers.push_back(l->instance_name);
		if (log != nullptr)
		{
			*log << "Updating Batch Normalization weights for these layers: ";
			for(size_t i = 0; i < bn_layers.size(); ++i)
				*log << (i == 0 ? "" : ", ") << bn_layers[i];
			*log << std::endl;
		}

		for(const std::string& layer_name : bn_layers)
		{
			if (log != nullptr)
				*log << layer_name << std::endl;
			forward_propagation::ptr forward_prop = factory.create(schema, std::vector<std::string>(1, layer_name), debug, profile);

			layer_data::ptr dt = data.get(layer_name);
			if (dt->size() != 4)
				throw neural_network_exception("data weight vector count " + std::to_string(dt->size()) + " doesn't satisfy layer configuration 4 for layer " + layer_name);
			const std::vector<float> gamma_saved = dt->at(0);
			const std::vector<float> beta_saved = dt->at(1);
			std::fill(dt->at(0).begin(), dt->at(0).end(), 1.0F);
			std::fill(dt->at(1).begin(), dt->at(1).end(), 0.0F);

			forward_prop->set_data(data);

			stat_data_bunch_writer writer;
			forward_prop->run(reader, writer);

			const std::vector<feature_map_data_stat> stat = writer.get_stat().at(layer_name);
			for(size_t feature_map_id = 0; feature_map_id < stat.size(); ++feature_map_id)
			{
				if (log != nullptr)
					*log << feature_map_id << ": " << stat[feature_map_id] << std::endl;
				const float old_mean = dt->at(2)[feature_map_id];
				const float old_invsigma = dt->at(3)[feature_map_id];
				const float new_invsigma = old_invsigma / stat[feature_map_id].std_dev;
				const float new_mean = old_mean + stat[feature_map_id].average / old_invsigma;
				dt->at(2)[feature_map_id] = new_mean;
				dt->at(3)[feature_map_id] = new_invsigma;
			}

			dt->at(0) = gamma_saved;
			dt->at(1) = beta_saved;
		}
	}

	std::string profile_state::get_path_to_unique_file(const char * file_prefix, const char * file_extension)
	{
		char buf[32];
		std::snprintf(buf, sizeof(buf), "_%03u.", index++);
		return profile_folder + "/" + file_prefix + buf + file_extension;
	}

	namespace
	{
		std::string percent(float v)
		{
			char buf[32];
			std::snprintf(buf, sizeof(buf), "%.2f%%", static_cast<double>(v * 100.0F));
			return buf;
		}

		// The per-action report of nnforge/profile_util.cpp:25-105 (tab separated, slowest first),
		// with the bandwidth columns a memory-bound backend needs next to the GFLOPS ones.
		void dump_action_performance(
			const std::string& path,
			unsigned int entry_count,
			float total_seconds,
			float max_flops,
			float max_bytes_per_second,
			const std::map<layer_name_with_action, float>& seconds,
			const std::map<layer_name_with_action, float>& flops_per_entry,
			const std::map<layer_name_with_action, float>& bytes_per_entry,
			const std::map<layer_name_with_action, std::string>& names,
			const std::map<layer_name_with_action, std::string>& types)
		{
			typedef std::pair<layer_name_with_action, float> entry;
			std::vector<entry> entries(seconds.begin(), seconds.end());
			std::sort(entries.begin(), entries.end(), [] (const entry& a, const entry& b) { return a.second > b.second; });
			std::ofstream out(path.c_str(), std::ios_base::out | std::ios_base::trunc);
			if (!out)
				throw neural_network_exception("Cannot open " + path + " for writing");
			out << "Layer\tLayer type\tAction\tTime of total\tRelative to peak perf\tAbsolute time, seconds\tAbsolute perf, GFLOPS\tGB/s\tRelative to peak bandwidth" << std::endl;
			for(const entry& e : entries)
			{
				const auto lookup = [&e] (const std::map<layer_name_with_action, float>& m) { std::map<layer_name_with_action, float>::const_iterator it = m.find(e.first); return (it == m.end()) ? 0.0F : it->second; };
				const auto text = [&e] (const std::map<layer_name_with_action, std::string>& m, const std::string& otherwise) { std::map<layer_name_with_action, std::string>::const_iterator it = m.find(e.first); return (it == m.end()) ? otherwise : it->second; };
				const float gflops = lookup(flops_per_entry) * static_cast<float>(entry_count) / e.second * 1.0e-9F;
				const float gbps = lookup(bytes_per_entry) * static_cast<float>(entry_count) / e.second * 1.0e-9F;
				// an action that covers several layers lists all of them (and their types) in the first two columns
				out << text(names, e.first.get_name()) << "\t" << text(types, std::string()) << "\t" << e.first.get_action().str();
				out << "\t" << percent(e.second / total_seconds);
				out << "\t" << ((max_flops > 0.0F) ? percent(gflops / (max_flops * 1.0e-9F)) : std::string("NA"));
				out << "\t" << e.second << "\t" << gflops << "\t" << gbps;
				out << "\t" << ((max_bytes_per_second > 0.0F) ? percent(gbps / (max_bytes_per_second * 1.0e-9F)) : std::string("NA"));
				out << std::endl;
			}
		}
	}

	// ---- forward_propagation ---------------------------------------------------------------

	forward_propagation::forward_propagation(
		const network_schema& full_schema,
		const std::vector<std::string>& output_layer_names,
		debug_state::ptr debug,
		profile_state::ptr profile)
		: output_layer_names(output_layer_names)
		, debug(debug ? debug : debug_state::ptr(new debug_state()))
		, profile(profile ? profile : profile_state::ptr(new profile_state()))
		, output_layers_tiling_factor(1)
		, flops(0.0F)
	{
		if (output_layer_names.empty())
			throw neural_network_exception("No output layers specified for forward_propagation");
		network_schema::ptr reduced(new network_schema(full_schema.get_required_layers(output_layer_names)));
		reduced->name = full_schema.name;
		schema = reduced;
		// a forward action per layer with inputs, waiting for the forward actions of the layers it reads (layers
		// without inputs - data layers, layers computed elsewhere - have no action: their values are there)
		action_schema.reset(new network_action_schema());
		for(const layer::const_ptr& l : schema->get_layers_in_forward_propagation_order())
		{
			if (l->input_layer_instance_names.empty())
				continue;
			std::vector<layer_name_with_action> dependencies;
			for(const std::string& input : l->input_layer_instance_names)
			{
				const layer_name_with_action source(input, layer_action(layer_action::forward));
				if (!schema->get_layer(input)->input_layer_instance_names.empty()
					&& (std::find(dependencies.begin(), dependencies.end(), source) == dependencies.end()))
					dependencies.push_back(source);
			}
			action_schema->add_action(l, layer_action(layer_action::forward), dependencies);
		}
		for(const layer::const_ptr& l : schema->get_data_layers())
			data_layer_names.insert(l->instance_name);

		cumulative_tiling_factor_map = schema->get_cumulative_tiling_factor_map();
		output_layers_tiling_factor = cumulative_tiling_factor_map.at(output_layer_names[0]);
		for(const std::string& n : output_layer_names)
			if (cumulative_tiling_factor_map.at(n) != output_layers_tiling_factor)
				throw neural_network_exception("Inconsistent tiling factors across output layers: "
					+ std::to_string(output_layers_tiling_factor) + " and " + std::to_string(cumulative_tiling_factor_map.at(n)));
	}

	// ---- network_action_schema ---------------------------------------------------------------

	const network_action_schema::node& network_action_schema::find(const layer_name_with_action& action) const
	{
		for(const node& n : nodes)
			if (n.key == action)
				return n;
		throw neural_network_exception("Action not found in action schema: " + action.get_name() + " " + action.get_action().str());
	}

	bool network_action_schema::action_exists(const layer_name_with_action& layer_and_action) const
	{
		for(const node& n : nodes)
			if (n.key == layer_and_action)
				return true;
		return false;
	}

	void network_action_schema::add_action(layer::const_ptr l, layer_action action, const std::vector<layer_name_with_action>& dependencies)
	{
		const layer_name_with_action key(l->instance_name, action);
		if (action_exists(key))
			throw neural_network_exception("Action already exists in action schema: " + key.get_name() + " " + action.str());
		for(const layer_name_with_action& d : dependencies)
			find(d);
		node n;
		n.l = l;
		n.key = key;
		nodes.push_back(n);
		add_dependencies(key, dependencies);
	}

	void network_action_schema::add_dependencies(const layer_name_with_action& source_layer_and_action, const std::vector<layer_name_with_action>& dependencies)
	{
		for(const layer_name_with_action& d : dependencies)
			add_dependency(source_layer_and_action, d);
	}

	void network_action_schema::add_dependency(const layer_name_with_action& source_layer_and_action, const layer_name_with_action& destination_layer_and_action)
	{
		find(destination_layer_and_action);
		node& n = const_cast<node&>(find(source_layer_and_action));
		if (std::find(n.dependencies.begin(), n.dependencies.end(), destination_layer_and_action) == n.dependencies.end())
			n.dependencies.push_back(destination_layer_and_action);
	}

	bool network_action_schema::dependency_exists(const layer_name_with_action& source_layer_and_action, const layer_name_with_action& destination_layer_and_action) const
	{
		if (!action_exists(source_layer_and_action))
			return false;
		const node& n = find(source_layer_and_action);
		return std::find(n.dependencies.begin(), n.dependencies.end(), destination_layer_and_action) != n.dependencies.end();
	}

	std::vector<layer_name_with_action> network_action_schema::get_dependencies(const layer_name_with_action& action) const
	{
		return find(action).dependencies;
	}

	std::vector<layer_name_with_action> network_action_schema::get_actions() const
	{
		std::vector<layer_name_with_action> res;
		for(const node& n : nodes)
			res.push_back(n.key);
		return res;
	}

	layer::const_ptr network_action_schema::get_layer(const layer_name_with_action& action) const
	{
		return find(action).l;
	}

	std::vector<layer_name_with_action> network_action_schema::get_actions_in_execution_order() const
	{
		std::vector<layer_name_with_action> res;
		std::vector<bool> done(nodes.size(), false);
		while (res.size() < nodes.size())
		{
			bool progressed = false;
			for(size_t i = 0; i < nodes.size(); ++i)
			{
				if (done[i])
					continue;
				bool ready = true;
				for(const layer_name_with_action& d : nodes[i].dependencies)
					ready = ready && (std::find(res.begin(), res.end(), d) != res.end());
				if (ready)
				{
					res.push_back(nodes[i].key);
					done[i] = true;
					progressed = true;
				}
			}
			if (!progressed)
				throw neural_network_exception("The action schema has a cycle");
		}
		return res;
	}

	void network_action_schema::drop_actions_not_required_to_do(const std::set<layer_name_with_action>& target_action_set)
	{
		std::set<layer_name_with_action> needed;
		std::vector<layer_name_with_action> todo(target_action_set.begin(), target_action_set.end());
		while (!todo.empty())
		{
			const layer_name_with_action cur = todo.back();
			todo.pop_back();
			if (!needed.insert(cur).second)
				continue;
			for(const layer_name_with_action& d : find(cur).dependencies)
				todo.push_back(d);
		}
		std::vector<node> kept;
		for(const node& n : nodes)
			if (needed.find(n.key) != needed.end())
				kept.push_back(n);
		nodes = kept;
	}

	bool forward_propagation::is_schema_with_weights() const
	{
		for(const layer::const_ptr& l : schema->get_layers())
			if (!l->is_empty_data() || !l->is_empty_data_custom())
				return true;
		return false;
	}

	void forward_propagation::clear_data()
	{
		actual_clear_data();
	}

	void forward_propagation::set_data(const network_data& data)
	{
		const std::vector<layer::const_ptr> layer_list = schema->get_layers();
		network_data::const_ptr new_data(new network_data(layer_list, data));
		new_data->check_network_data_consistency(layer_list);
		actual_set_data(new_data);
	}

	void forward_propagation::set_input_configuration_specific(const std::map<std::string, layer_configuration_specific>& input_configuration_specific_map)
	{
		bool same_input_config = true;
		std::map<std::string, layer_configuration_specific> filtered;
		for(const std::pair<const std::string, layer_configuration_specific>& item : input_configuration_specific_map)
		{
			if (data_layer_names.find(item.first) == data_layer_names.end())
				continue;
			filtered.insert(item);
			std::map<std::string, layer_configuration_specific>::const_iterator known = layer_config_map.find(item.first);
			if ((known == layer_config_map.end()) || (known->second != item.second))
				same_input_config = false;
		}
		if (same_input_config && !layer_config_map.empty())
			return;

		layer_config_map = schema->get_layer_configuration_specific_map(filtered);

		flops = 0.0F;
		for(const layer::const_ptr& l : schema->get_layers())
		{
			if (l->input_layer_instance_names.empty())
				continue;
			std::vector<layer_configuration_specific> inputs;
			for(const std::string& input : l->input_layer_instance_names)
				inputs.push_back(layer_config_map[input]);
			// nnforge/network_action_schema.cpp:166-170
			flops += l->get_forward_flops_per_entry(inputs) * static_cast<float>(cumulative_tiling_factor_map.at(l->instance_name));
		}

		layer_config_map_modified();
	}

	forward_propagation::stat forward_propagation::run(structured_data_bunch_reader& reader, structured_data_bunch_writer& writer)
	{
		stat res;
		const std::chrono::high_resolution_clock::time_point start = std::chrono::high_resolution_clock::now();
		set_input_configuration_specific(reader.get_config_map());
		res.flops_per_entry = flops;
		std::map<std::string, layer_configuration_specific> output_config_map;
		for(const std::string& n : output_layer_names)
			output_config_map[n] = layer_config_map[n];
		writer.set_config_map(output_config_map);
		last_action_seconds.clear();
		float idle_seconds = 0.0F;
		res.entry_processed_count = 0;
		actual_run(reader, writer, res.entry_processed_count, last_action_seconds, idle_seconds);
		const std::chrono::duration<float> sec = std::chrono::high_resolution_clock::now() - start;
		res.total_seconds = sec.count();
		res.idle_seconds = idle_seconds;

		if (profile->is_profile() && !last_action_seconds.empty() && !profile->profile_folder.empty())
			dump_action_performance(
				profile->get_path_to_unique_file("forward_prop_perf_per_layer_action", "csv"),
				res.entry_processed_count, res.total_seconds, get_max_flops(), get_max_bytes_per_second(),
				last_action_seconds, action_flops_per_entry, action_bytes_per_entry, action_layer_names, action_layer_types);
		return res;
	}

	std::string forward_propagation::get_action_layer_names(const layer_name_with_action& action) const
	{
		std::map<layer_name_with_action, std::string>::const_iterator it = action_layer_names.find(action);
		return (it == action_layer_names.end()) ? action.get_name() : it->second;
	}

	float forward_propagation::get_max_flops() const
	{
		return 0.0F; // unknown: the report then says NA (the reference throws "get_max_flops not implemented")
	}

	std::ostream& operator<< (std::ostream& out, const forward_propagation::stat& val)
	{
		const float idle_overhead = (val.total_seconds > 0.0F) ? val.idle_seconds / val.total_seconds : 0.0F;
		const float gflops = (val.total_seconds > 0.0F) ? val.flops_per_entry * static_cast<float>(val.entry_processed_count) / val.total_seconds * 1.0e-9F : 0.0F;
		char buf[256];
		std::snprintf(buf, sizeof(buf), "%.2f seconds, idle %.1f%%, %u entries, %.2e flops per entry, %.1f GFLOPS",
			static_cast<double>(val.total_seconds), static_cast<double>(idle_overhead * 100.0F), val.entry_processed_count,
			static_cast<double>(val.flops_per_entry), static_cast<double>(gflops));
		out << buf;
		return out;
	}

	void factory_generator::apply_default_options()
	{
		for(string_option& o : get_string_options()) *o.var = o.default_value;
		for(multi_string_option& o : get_multi_string_options()) o.var->clear();
		for(path_option& o : get_path_options()) *o.var = o.default_value;
		for(bool_option& o : get_bool_options()) *o.var = o.default_value;
		for(float_option& o : get_float_options()) *o.var = o.default_value;
		for(int_option& o : get_int_options()) *o.var = o.default_value;
	}
}
