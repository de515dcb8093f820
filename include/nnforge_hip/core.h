// Backend-neutral containers of the inference path, restated by name and meaning from nnForge so
// that code written against nnForge's plug-in surface compiles against this backend without
// Boost or protobuf: exceptions, tensor shape, weight containers, the layer base class and its
// type-name registry.
#pragma once

#include <cstddef>
#include <istream>
#include <map>
#include <memory>
#include <ostream>
#include <set>
#include <stdexcept>
#include <string>
#include <vector>

namespace nnforge
{
	// nnforge/neural_network_exception.h:23-34. Unlike the reference it does not assert(0) in debug
	// builds: error paths are exercised by the tests.
	class neural_network_exception : public std::runtime_error
	{
	public:
		explicit neural_network_exception(const char * message) : std::runtime_error(message) {}
		explicit neural_network_exception(const std::string& message) : std::runtime_error(message) {}
		neural_network_exception(const std::string& message, const char * filename, int line_number);
	};

	// Shape of one entry of a layer's output: feature_map_count planes of
	// dimension_sizes[0] x dimension_sizes[1] x ... neurons, dimension 0 (x) fastest in memory
	// (nnforge/layer_configuration_specific.h:27-64, .cpp:62-117).
	class layer_configuration_specific
	{
	public:
		layer_configuration_specific() : feature_map_count(0) {}
		layer_configuration_specific(unsigned int feature_map_count) : feature_map_count(feature_map_count) {}
		layer_configuration_specific(unsigned int feature_map_count, const std::vector<unsigned int>& dimension_sizes)
			: feature_map_count(feature_map_count), dimension_sizes(dimension_sizes) {}

		// binary form: u32 feature_map_count, u32 dimension_count, u32 sizes[dimension_count]
		void write(std::ostream& output_stream) const;
		void read(std::istream& input_stream);

		unsigned int get_neuron_count() const;
		unsigned int get_neuron_count_per_feature_map() const;
		unsigned int get_dimension_count() const { return static_cast<unsigned int>(dimension_sizes.size()); }

		// offsets: one coordinate per dimension, x first
		unsigned int get_pos(const std::vector<unsigned int>& offsets) const;
		std::vector<unsigned int> get_offsets(unsigned int pos) const;

		// throw neural_network_exception when the two objects differ
		void check_equality(const layer_configuration_specific& other) const;
		void check_equality(unsigned int neuron_count) const;

		bool operator==(const layer_configuration_specific& other) const;
		bool operator!=(const layer_configuration_specific& other) const { return !(*this == other); }

	public:
		unsigned int feature_map_count;
		std::vector<unsigned int> dimension_sizes;
	};

	std::ostream& operator<<(std::ostream& out, const layer_configuration_specific& config);

	// Weights of one layer: a list of chunks of floats (nnforge/layer_data.h:28-48).
	// Binary form (layer_data.cpp:23-52): u32 chunk_count, then per chunk u32 length + floats.
	class layer_data : public std::vector<std::vector<float> >
	{
	public:
		typedef std::shared_ptr<layer_data> ptr;
		typedef std::shared_ptr<const layer_data> const_ptr;

		void write(std::ostream& binary_stream_to_write_to) const;
		void read(std::istream& binary_stream_to_read_from);
		void fill(float val);
	};

	// Integer side data of a layer (nnforge/layer_data_custom.h); none of the layers here has any.
	class layer_data_custom : public std::vector<std::vector<int> >
	{
	public:
		typedef std::shared_ptr<layer_data_custom> ptr;
		typedef std::shared_ptr<const layer_data_custom> const_ptr;
	};

	// What is done to a layer (nnforge/layer_action.h:26-88). This backend only ever runs "forward"; the other
	// kinds exist so that keys built elsewhere compare and print as the reference's do.
	class layer_action
	{
	public:
		enum action_type
		{
			forward = 0,
			backward_data = 1,
			backward_weights = 2,
			backward_data_and_weights = 3,
			update_weights = 4
		};

		layer_action() = default;
		layer_action(action_type at, int backprop_index = -1) : at(at), backprop_index(backprop_index) {}

		action_type get_action_type() const { return at; }
		int get_backprop_index() const { return backprop_index; }
		std::string str() const;

	private:
		action_type at = forward;
		int backprop_index = -1;

		friend bool operator <(const layer_action& x, const layer_action& y);
	};

	inline bool operator <(const layer_action& x, const layer_action& y)
	{
		return ((static_cast<unsigned long long>(x.at) << 32) | static_cast<unsigned int>(x.backprop_index))
			< ((static_cast<unsigned long long>(y.at) << 32) | static_cast<unsigned int>(y.backprop_index));
	}

	// Key of the per-action tables of a propagation (nnforge/layer_name_with_action.h:25-69).
	class layer_name_with_action
	{
	public:
		layer_name_with_action() = default;
		layer_name_with_action(const std::string& name, layer_action action) : name(name), action(action) {}

		const std::string& get_name() const { return name; }
		const layer_action& get_action() const { return action; }

	private:
		std::string name;
		layer_action action;

		friend bool operator <(const layer_name_with_action& x, const layer_name_with_action& y);
	};

	inline bool operator <(const layer_name_with_action& x, const layer_name_with_action& y)
	{
		if (x.name < y.name)
			return true;
		if (y.name < x.name)
			return false;
		return x.action < y.action;
	}

	inline bool operator ==(const layer_name_with_action& x, const layer_name_with_action& y)
	{
		return !(x < y) && !(y < x);
	}

	typedef std::vector<unsigned int> data_config;
	typedef std::vector<unsigned int> data_custom_config;

	// A message of the text-format schema ("layer { ... }", "<type>_param { ... }", "dimension_param { ... }"): its
	// scalar fields as text and its nested messages, which keep their order (e.g. one dimension_param per spatial
	// dimension). It stands where the reference has the classes protoc generates from nnforge/proto/nnforge.proto:
	// layer::read_proto / write_proto receive the layer's message as one of these.
	struct schema_param_block
	{
		std::map<std::string, std::string> scalars;
		std::vector<std::string> scalar_order; // the keys in the order set() received them: the order a writer emits
		std::set<std::string> quoted;          // scalars that stood in quotes in the text a reader parsed (the values are kept without them)
		std::vector<std::pair<std::string, schema_param_block> > blocks;

		// the first nested message of that name, null when there is none
		const schema_param_block * child(const std::string& name) const;
		// for writers: a scalar field (value as it appears in the text format), a nested message
		void set(const std::string& key, const std::string& value_text);
		schema_param_block& add_block(const std::string& name);

		bool has(const std::string& key) const { return scalars.find(key) != scalars.end(); }
		float get_float(const std::string& key, float default_value) const;
		unsigned int get_uint(const std::string& key, unsigned int default_value) const;
		unsigned int require_uint(const std::string& key, const std::string& context) const;
		bool get_bool(const std::string& key, bool default_value) const; // text format: true / false
		std::string get_string(const std::string& key, const std::string& default_value) const; // enum values, unquoted
		std::vector<const schema_param_block *> children(const std::string& name) const;
	};

	// Base of the schema layers (nnforge/layer.h:37-121), forward/inference side only.
	// By how much a layer changes the number of entries that flow through it: max subsampling with tiling makes
	// several entries of one (a factor), windows over entries make one of several (one over a factor)
	// (nnforge/tiling_factor.h:24-56).
	class tiling_factor
	{
	public:
		tiling_factor(unsigned int f = 1, bool b_multiply = true);

		// the factor as a count; throws for "one over ..."
		operator unsigned int() const;
		std::string str() const;
		tiling_factor get_inverse() const;
		tiling_factor& operator *=(const tiling_factor& other);

	private:
		unsigned int f;
		bool b_multiply;

		friend bool operator ==(const tiling_factor& t1, const tiling_factor& t2);
	};

	tiling_factor operator *(const tiling_factor& t1, const tiling_factor& t2);
	bool operator ==(const tiling_factor& t1, const tiling_factor& t2);
	bool operator !=(const tiling_factor& t1, const tiling_factor& t2);

	class layer
	{
	public:
		typedef std::shared_ptr<layer> ptr;
		typedef std::shared_ptr<const layer> const_ptr;

		virtual ~layer() = default;

		virtual layer::ptr clone() const = 0;

		// default: same configuration as the first input
		virtual layer_configuration_specific get_output_layer_configuration_specific(
			const std::vector<layer_configuration_specific>& input_configuration_specific_list) const;

		virtual std::string get_type_name() const = 0;

		// floating point operations per entry of a forward pass (the reference's flops model)
		virtual float get_forward_flops_per_entry(const std::vector<layer_configuration_specific>& input_configuration_specific_list) const = 0;

		// nnforge/layer.h:64-66. layer_proto points at the layer's message of the schema - here a schema_param_block
		// (the "layer { ... }" block) where the reference has a protobuf::Layer. read_proto takes the layer's parameters
		// from its "<type>_param" message (defaults, or an exception, when that is missing, as in the reference);
		// write_proto adds that message when the reference's writer would.
		virtual void read_proto(const void * layer_proto);
		virtual void write_proto(void * layer_proto) const;

		virtual std::vector<std::string> get_parameter_strings() const { return std::vector<std::string>(); }

		// how the layer changes the number of entries (nnforge/layer.cpp:150-153: it does not)
		virtual tiling_factor get_tiling_factor() const { return tiling_factor(1); }

		// all values 0.0F
		layer_data::ptr create_layer_data() const;
		layer_data_custom::ptr create_layer_data_custom() const;

		// throw neural_network_exception when the data does not fit the layer
		void check_layer_data_consistency(const layer_data& data) const;
		void check_layer_data_custom_consistency(const layer_data_custom& data_custom) const;

		// the deterministic part of the reference's randomize_data (identity batch norm, 0.25 PReLU slopes)
		virtual void initialize_data(layer_data& data) const;

		bool is_empty_data() const { return get_data_config().empty(); }
		bool is_empty_data_custom() const { return get_data_custom_config().empty(); }

		virtual data_config get_data_config() const { return data_config(); }
		virtual data_custom_config get_data_custom_config() const { return data_custom_config(); }

	public:
		std::string instance_name;
		std::vector<std::string> input_layer_instance_names;

	protected:
		layer() = default;
	};

	// Registry of layer prototypes by type name (nnforge/layer_factory.h).
	class layer_factory
	{
	public:
		bool register_layer(layer::const_ptr sample_layer);
		bool unregister_layer(const std::string& layer_type_name);
		// throws neural_network_exception for an unknown type
		layer::ptr create_layer(const std::string& layer_type_name) const;
		bool is_registered(const std::string& layer_type_name) const;
		static layer_factory& get_singleton();

	private:
		layer_factory() = default;
		std::map<std::string, layer::const_ptr> sample_name_layer_map;
	};

	// registers the layer types of this backend in layer_factory (nnforge/nnforge.cpp:25-62)
	void init();
}
