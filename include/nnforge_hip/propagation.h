// The plug-in boundary a backend implements: data readers/writers, forward_propagation and its
// factory, factory_generator with its command-line options.
#pragma once

#include "core.h"
#include "schema.h"

#include <functional>
#include <map>
#include <set>
#include <string>
#include <vector>

namespace nnforge
{
	// A fixed set of threads that run the jobs posted to them, first posted first started
	// (nnforge/threadpool_job_runner.h:28-52; where the reference says service.post(job), say post(job)).
	// Backends hand the reading of input entries to it, one job per entry.
	class threadpool_job_runner
	{
	public:
		typedef std::shared_ptr<threadpool_job_runner> ptr;

		explicit threadpool_job_runner(unsigned int thread_count);
		// finishes the jobs already posted, then joins the threads
		~threadpool_job_runner();

		// a job must not let an exception escape
		void post(std::function<void()> job);

		unsigned int thread_count;

	private:
		struct impl;
		std::unique_ptr<impl> p;
		threadpool_job_runner() = delete;
		threadpool_job_runner(const threadpool_job_runner&) = delete;
		threadpool_job_runner& operator =(const threadpool_job_runner&) = delete;
	};

	// processors this process may run on (its affinity mask; never less than 1)
	unsigned int get_available_processor_count();

	// Source of input entries (nnforge/structured_data_bunch_reader.h:27-58).
	class structured_data_bunch_reader
	{
	public:
		typedef std::shared_ptr<structured_data_bunch_reader> ptr;
		virtual ~structured_data_bunch_reader() = default;
		virtual std::map<std::string, layer_configuration_specific> get_config_map() const = 0;
		// fills one entry of every layer in data_map; false when the entry cannot be read
		virtual bool read(unsigned int entry_id, const std::map<std::string, float *>& data_map) = 0;
		virtual void set_epoch(unsigned int epoch_id) {}
		virtual int get_entry_count() const { return -1; } // -1: unknown

	protected:
		structured_data_bunch_reader() = default;
	};

	// Sink of output entries (nnforge/structured_data_bunch_writer.h:27-50).
	class structured_data_bunch_writer
	{
	public:
		typedef std::shared_ptr<structured_data_bunch_writer> ptr;
		virtual ~structured_data_bunch_writer() = default;
		virtual void set_config_map(const std::map<std::string, layer_configuration_specific> config_map) = 0;
		virtual void write(unsigned int entry_id, const std::map<std::string, const float *>& data_map) = 0;

	protected:
		structured_data_bunch_writer() = default;
	};

	// Reader over caller-owned arrays: layer name -> entry_count consecutive entries.
	class memory_data_bunch_reader : public structured_data_bunch_reader
	{
	public:
		memory_data_bunch_reader(unsigned int entry_count) : entry_count(entry_count) {}
		void add(const std::string& layer_name, const layer_configuration_specific& config, const float * data);
		std::map<std::string, layer_configuration_specific> get_config_map() const override { return config_map; }
		bool read(unsigned int entry_id, const std::map<std::string, float *>& data_map) override;
		int get_entry_count() const override { return static_cast<int>(entry_count); }

	private:
		unsigned int entry_count;
		std::map<std::string, layer_configuration_specific> config_map;
		std::map<std::string, const float *> data;
	};

	// Writer that keeps every entry in memory (the role of neuron_value_set_data_bunch_writer,
	// nnforge/neuron_value_set_data_bunch_writer.cpp:21-39).
	class memory_data_bunch_writer : public structured_data_bunch_writer
	{
	public:
		void set_config_map(const std::map<std::string, layer_configuration_specific> config_map) override;
		void write(unsigned int entry_id, const std::map<std::string, const float *>& data_map) override;

		std::map<std::string, layer_configuration_specific> config_map;
		std::map<std::string, std::vector<float> > values; // layer name -> entries back to back
		unsigned int entry_count = 0;
	};

	// nnforge/feature_map_data_stat.h:23-35
	class feature_map_data_stat
	{
	public:
		float min;
		float max;
		float average;
		float std_dev;
	};
	std::ostream& operator<< (std::ostream& out, const feature_map_data_stat& val);

	// Writer that keeps per-feature-map statistics of everything written to it instead of the
	// values (nnforge/stat_data_bunch_writer.h:27-69): minimum, maximum and the single-pass mean /
	// sum of squared deviations in double precision. A backend that reduces its outputs on the
	// device hands the partial states over with merge() instead of calling write() per entry.
	class stat_data_bunch_writer : public structured_data_bunch_writer
	{
	public:
		typedef std::shared_ptr<stat_data_bunch_writer> ptr;

		// same layout as nnf_hip_running_stat of the C ABI
		struct running_stat
		{
			running_stat();
			double n;
			double mean;
			double m2;
			float min_val;
			float max_val;
		};

		stat_data_bunch_writer();
		void set_config_map(const std::map<std::string, layer_configuration_specific> config_map) override;
		void write(unsigned int entry_id, const std::map<std::string, const float *>& data_map) override;
		std::map<std::string, std::vector<feature_map_data_stat> > get_stat() const;

		// folds states accumulated elsewhere over `entries` further entries into this writer
		// (pairwise update of mean and sum of squared deviations)
		void merge(const std::string& layer_name, const std::vector<running_stat>& partial);
		void add_entries(unsigned int entries) { entry_count += entries; }
		unsigned int get_entry_count() const { return entry_count; }
		const std::map<std::string, layer_configuration_specific>& get_config_map() const { return config_map; }

	private:
		std::map<std::string, layer_configuration_specific> config_map;
		std::map<std::string, std::vector<running_stat> > layer_name_to_running_stat_list_map;
		unsigned int entry_count;
	};

	// nnforge/debug_state.h, profile_state.h reduced to their switches
	struct debug_state
	{
		typedef std::shared_ptr<debug_state> ptr;
		explicit debug_state(bool debug_mode = false) : debug_mode(debug_mode) {}
		bool is_debug() const { return debug_mode; }
		bool debug_mode;
	};

	// nnforge/profile_state.h: the switch and the folder the per-action reports go to (empty folder:
	// times are collected but no file is written)
	struct profile_state
	{
		typedef std::shared_ptr<profile_state> ptr;
		explicit profile_state(bool profile_mode = false, const std::string& profile_folder = std::string())
			: profile_mode(profile_mode), profile_folder(profile_folder), index(0) {}
		bool is_profile() const { return profile_mode; }
		// <folder>/<prefix>_NNN.<extension>, NNN counting up per call
		std::string get_path_to_unique_file(const char * file_prefix, const char * file_extension);
		bool profile_mode;
		std::string profile_folder;
		unsigned int index;
	};

	// The actions of a propagation and what each one waits for (nnforge/network_action_schema.h:35-126), as far as
	// forward propagation uses it: one forward action per layer that computes something, depending on the forward
	// actions of the layers it reads. The reference's scheduling helpers on top of the graph (streams, buffer sets,
	// flops-driven ordering, Graphviz output) belong to its own backends and are not restated: this backend plans
	// launches and buffers on its fused steps (forward_propagation_hip).
	class network_action_schema
	{
	public:
		typedef std::shared_ptr<network_action_schema> ptr;
		typedef std::shared_ptr<const network_action_schema> const_ptr;

		network_action_schema() = default;

		// throws when the action exists already or a dependency does not
		void add_action(layer::const_ptr l, layer_action action, const std::vector<layer_name_with_action>& dependencies = std::vector<layer_name_with_action>());
		bool action_exists(const layer_name_with_action& layer_and_action) const;
		void add_dependencies(const layer_name_with_action& source_layer_and_action, const std::vector<layer_name_with_action>& dependencies);
		void add_dependency(const layer_name_with_action& source_layer_and_action, const layer_name_with_action& destination_layer_and_action);
		bool dependency_exists(const layer_name_with_action& source_layer_and_action, const layer_name_with_action& destination_layer_and_action) const;
		// what the action waits for directly
		std::vector<layer_name_with_action> get_dependencies(const layer_name_with_action& action) const;
		// every action behind the actions it waits for; among those free to go, the one added first comes first
		std::vector<layer_name_with_action> get_actions_in_execution_order() const;
		std::vector<layer_name_with_action> get_actions() const; // in the order they were added
		layer::const_ptr get_layer(const layer_name_with_action& action) const;
		// keeps the target actions and everything they wait for, directly or not
		void drop_actions_not_required_to_do(const std::set<layer_name_with_action>& target_action_set);

	private:
		struct node
		{
			layer::const_ptr l;
			layer_name_with_action key;
			std::vector<layer_name_with_action> dependencies;
		};
		const node& find(const layer_name_with_action& action) const;
		std::vector<node> nodes; // in the order of add_action
	};

	// nnforge/forward_propagation.h:39-115
	class forward_propagation
	{
	public:
		class stat
		{
		public:
			unsigned int entry_processed_count;
			float flops_per_entry;
			float total_seconds;
			float idle_seconds;
		};

		typedef std::shared_ptr<forward_propagation> ptr;

		virtual ~forward_propagation() = default;

		// narrows the data to the layers of the schema and checks it against them
		void set_data(const network_data& data);
		void clear_data();

		// not needed before run(): run() takes the configurations from the reader
		void set_input_configuration_specific(const std::map<std::string, layer_configuration_specific>& input_configuration_specific_map);

		stat run(structured_data_bunch_reader& reader, structured_data_bunch_writer& writer);

		bool is_schema_with_weights() const;

		// seconds per action of the last run (filled when profiling is on). A backend that runs several layers
		// in one launch reports the launch under its last layer (the one whose output is stored);
		// get_action_layer_names tells which layers such an action covers.
		const std::map<layer_name_with_action, float>& get_last_action_seconds() const { return last_action_seconds; }
		// the layers an action covers in execution order, joined with '+' (the action's own name when it covers one)
		std::string get_action_layer_names(const layer_name_with_action& action) const;

	protected:
		forward_propagation(
			const network_schema& schema,
			const std::vector<std::string>& output_layer_names,
			debug_state::ptr debug,
			profile_state::ptr profile);

		virtual void actual_set_data(network_data::const_ptr data) = 0;
		virtual void actual_clear_data() = 0;
		virtual void actual_run(
			structured_data_bunch_reader& reader,
			structured_data_bunch_writer& writer,
			unsigned int& entries_processed,
			std::map<layer_name_with_action, float>& action_seconds,
			float& idle_seconds) = 0;
		// called when set_input_configuration_specific changed layer_config_map
		virtual void layer_config_map_modified() = 0;

		// what the backend can do at best, for the "relative to peak" columns of the profile report
		// (nnforge/forward_propagation.h:94 get_max_flops; bytes per second is the figure that matters
		// for the bandwidth-bound layers of this backend)
		virtual float get_max_flops() const;
		virtual float get_max_bytes_per_second() const { return 0.0F; }

	protected:
		network_schema::const_ptr schema; // reduced to what the outputs need
		// one forward action per layer of `schema` that computes something (nnforge/forward_propagation.h:97,
		// network_schema::get_actions_for_forward_propagation, nnforge/network_schema.cpp:242-300)
		network_action_schema::ptr action_schema;
		std::vector<std::string> output_layer_names;
		debug_state::ptr debug;
		profile_state::ptr profile;
		std::map<std::string, layer_configuration_specific> layer_config_map;
		// entries a layer holds per entry read, and that figure for the output layers, which must agree on it
		// (nnforge/forward_propagation.h:103-104, forward_propagation.cpp:54-61)
		std::map<std::string, unsigned int> cumulative_tiling_factor_map;
		unsigned int output_layers_tiling_factor;
		float flops;
		std::set<std::string> data_layer_names;
		std::map<layer_name_with_action, float> last_action_seconds;
		// per action (same keys as the action seconds): the reference's flops model
		// (nnforge/forward_propagation.h:103) and, beside it, the memory traffic the action needs per entry
		std::map<layer_name_with_action, float> action_flops_per_entry;
		std::map<layer_name_with_action, float> action_bytes_per_entry;
		// for actions that cover several layers: the layers' names and their types, each joined with '+'
		std::map<layer_name_with_action, std::string> action_layer_names;
		std::map<layer_name_with_action, std::string> action_layer_types;

	private:
		forward_propagation() = delete;
		forward_propagation(const forward_propagation&) = delete;
		forward_propagation& operator =(const forward_propagation&) = delete;
	};

	std::ostream& operator<< (std::ostream& out, const forward_propagation::stat& val);

	// nnforge/forward_propagation_factory.h:30-46
	class forward_propagation_factory
	{
	public:
		typedef std::shared_ptr<forward_propagation_factory> ptr;
		typedef std::shared_ptr<const forward_propagation_factory> const_ptr;
		virtual ~forward_propagation_factory() = default;
		virtual forward_propagation::ptr create(
			const network_schema& schema,
			const std::vector<std::string>& output_layer_names,
			debug_state::ptr debug,
			profile_state::ptr profile) const = 0;

	protected:
		forward_propagation_factory() = default;
	};

	// Refreshes mean and inverse sigma of every BatchNorm layer from the statistics of the data the
	// reader supplies (toolset::update_bn_weights, nnforge/toolset.cpp:1562-1630): per layer, a forward
	// pass up to that layer with gamma 1 and beta 0 into a stat_data_bunch_writer, then
	// inv_sigma' = inv_sigma / std_dev, mean' = mean + average / inv_sigma. Layers are handled in
	// forward order, each one seeing the refreshed weights of those before it. data is modified in place.
	// log (optional) receives the lines the reference prints.
	void update_bn_weights(
		const network_schema& schema,
		network_data& data,
		structured_data_bunch_reader& reader,
		const forward_propagation_factory& factory,
		debug_state::ptr debug = debug_state::ptr(),
		profile_state::ptr profile = profile_state::ptr(),
		std::ostream * log = nullptr);

	// nnforge/backward_propagation_factory.h: the training side is outside this backend; the type
	// exists so that factory_generator keeps its shape.
	class backward_propagation_factory
	{
	public:
		typedef std::shared_ptr<backward_propagation_factory> ptr;
		virtual ~backward_propagation_factory() = default;
	};

	// option descriptors (nnforge/config_options.h): a name (optionally "long,S" with a short form),
	// the variable to fill, its default and a description
	template<class T> struct config_option
	{
		config_option(const char * name, T * var, const T& default_value, const char * description)
			: name(name), var(var), default_value(default_value), description(description) {}
		std::string name;
		T * var;
		T default_value;
		std::string description;
	};
	typedef config_option<std::string> string_option;
	typedef config_option<bool> bool_option;
	typedef config_option<float> float_option;
	typedef config_option<int> int_option;
	// a path as text where the reference has boost::filesystem::path (nnforge/config_options.h:62-80)
	typedef config_option<std::string> path_option;
	// an option that may be given several times (nnforge/config_options.h:45-60): no default
	struct multi_string_option
	{
		multi_string_option(const char * name, std::vector<std::string> * var, const char * description) : name(name), var(var), description(description) {}
		std::string name;
		std::vector<std::string> * var;
		std::string description;
	};

	// nnforge/factory_generator.h:27-56
	class factory_generator
	{
	public:
		typedef std::shared_ptr<factory_generator> ptr;
		virtual ~factory_generator() = default;
		virtual void initialize() = 0;
		virtual forward_propagation_factory::ptr create_forward_propagation_factory() const = 0;
		virtual backward_propagation_factory::ptr create_backward_propagation_factory() const = 0;
		virtual void info() const = 0;
		virtual std::vector<string_option> get_string_options() { return std::vector<string_option>(); }
		virtual std::vector<multi_string_option> get_multi_string_options() { return std::vector<multi_string_option>(); }
		virtual std::vector<path_option> get_path_options() { return std::vector<path_option>(); }
		virtual std::vector<bool_option> get_bool_options() { return std::vector<bool_option>(); }
		virtual std::vector<float_option> get_float_options() { return std::vector<float_option>(); }
		virtual std::vector<int_option> get_int_options() { return std::vector<int_option>(); }

		// sets every option variable to its default (what the toolset does before parsing the command line)
		void apply_default_options();

	protected:
		factory_generator() = default;
	};
}
