// Network description: the layer graph (network_schema), its text-format file, and the weights
// of a network (network_data) with nnForge's "<layer>.data" files.
#pragma once

#include "core.h"

#include <string>
#include <vector>

namespace nnforge
{
	// Directed acyclic graph of layers addressed by instance name (nnforge/network_schema.h:37-104),
	// restricted to what forward propagation needs.
	class network_schema
	{
	public:
		typedef std::shared_ptr<network_schema> ptr;
		typedef std::shared_ptr<const network_schema> const_ptr;

		network_schema() = default;
		// throws on duplicate names, unknown inputs and cycles
		explicit network_schema(const std::vector<layer::const_ptr>& layer_list);

		// protobuf text format of nnforge/proto/nnforge.proto:5-42 (NetworkSchema { name, layer { type,
		// name, input_layer_name*, <type>_param { ... } } }); the sample file of the reference is
		// examples/gtsrb/working_data/schema.txt. Layer types not registered in layer_factory throw ("No layer is
		// registered with type ...", nnforge/layer_factory.cpp) unless keep_unregistered_layers is set: then such a
		// layer becomes an external_layer, which keeps its block of the file and computes nothing.
		void read_proto(std::istream& stream_to_read_from, bool keep_unregistered_layers = false);
		void write_proto(std::ostream& stream_to_write_to) const;

		// Layers needed to compute the given outputs, in forward propagation order. The search stops at external layers:
		// their output comes from outside, so what they read is not needed on their account, and they appear in the
		// result without inputs - as sources of data beside the data layers.
		std::vector<layer::const_ptr> get_required_layers(const std::vector<std::string>& output_layer_names) const;
		bool has_external_layers() const;

		std::vector<layer::const_ptr> get_layers() const { return layers; }
		// layers without inputs: their values come from the reader
		std::vector<layer::const_ptr> get_data_layers() const;
		// inputs always precede their consumers; data layers included
		std::vector<layer::const_ptr> get_layers_in_forward_propagation_order() const;

		// configurations of every layer given those of the data layers (the result includes the inputs)
		std::map<std::string, layer_configuration_specific> get_layer_configuration_specific_map(
			const std::map<std::string, layer_configuration_specific>& input_configuration_specific_map) const;

		// per layer: how many entries it holds for each entry the data layers supply. Data layers hold 1; a layer
		// multiplies the factor of its inputs, which must agree, by its own (nnforge/network_schema.cpp:651-680).
		// Throws when the inputs of a layer disagree or the product is not a whole number.
		std::map<std::string, unsigned int> get_cumulative_tiling_factor_map() const;

		// number of layers that read the output of the given layer
		unsigned int get_consumer_count(const std::string& instance_name) const;

		layer::const_ptr find_layer(const std::string& instance_name) const; // empty when absent
		layer::const_ptr get_layer(const std::string& instance_name) const;  // throws when absent

	public:
		std::string name;

	private:
		void rebuild(const std::vector<layer::const_ptr>& layer_list);

		std::vector<layer::const_ptr> layers; // forward propagation order
		std::map<std::string, size_t> name_to_index;
	};

	// Weights per layer instance name (nnforge/network_data.h, layer_data_list.h).
	class network_data
	{
	public:
		typedef std::shared_ptr<network_data> ptr;
		typedef std::shared_ptr<const network_data> const_ptr;

		network_data() = default;
		// zero-filled (val) data for every layer that has weights
		explicit network_data(const std::vector<layer::const_ptr>& layer_list, float val = 0.0F);
		// the subset of other that layer_list needs; throws when a layer's weights are missing
		network_data(const std::vector<layer::const_ptr>& layer_list, const network_data& other);

		void check_network_data_consistency(const std::vector<layer::const_ptr>& layer_list) const;

		// deterministic initial weights (identity batch norm, PReLU 0.25)
		void initialize(const std::vector<layer::const_ptr>& layer_list);

		// One file per layer with weights: 16-byte GUID d11935b5-3059-49e2-9c33-1c4322f8130d, then
		// layer_data::write (nnforge/layer_data_list.cpp:30-36,154-166).
		void write(const std::string& folder_path) const;
		void read(const std::string& folder_path);

		layer_data::ptr find(const std::string& instance_name) const; // empty when absent
		layer_data_custom::ptr find_custom(const std::string& instance_name) const; // empty when absent
		layer_data::ptr get(const std::string& instance_name) const;  // throws when absent
		void add(const std::string& instance_name, layer_data::ptr data);

		std::map<std::string, layer_data::ptr> data_list;
		std::map<std::string, layer_data_custom::ptr> data_custom_list;
	};
}
