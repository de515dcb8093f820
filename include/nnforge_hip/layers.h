// Schema classes of the layers on the inference path: type names, parameters and weight-chunk
// layouts as nnForge defines them.
#pragma once

#include "core.h"

#include <limits>

namespace nnforge
{
	// Placeholder for externally supplied data (nnforge/data_layer.h); type name "Data".
	class data_layer : public layer
	{
	public:
		data_layer() = default;
		layer::ptr clone() const override;
		std::string get_type_name() const override;
		float get_forward_flops_per_entry(const std::vector<layer_configuration_specific>&) const override { return 0.0F; }
		static const std::string layer_type_name;
	};

	// A layer of a type this backend has no class for (convolution, local contrast subtraction, error functions ...).
	// It keeps the type name, the inputs and the parameter messages as the schema file states them, so that such a
	// schema can be read, planned around and written back. It computes nothing: in a forward_propagation its output
	// arrives as data under the layer's own name, like a data layer's (the reference's own example does this by hand:
	// examples/gtsrb/working_data/schema_tail.txt:10-13 declares "tanh_3_layer" as a Data layer), with the configuration
	// the reader states for it; what only such layers read is not computed. network_schema::read_proto makes these
	// for unregistered types when asked to; by default an unregistered type is an error, as in the reference.
	class external_layer : public layer
	{
	public:
		explicit external_layer(const std::string& type_name);
		layer::ptr clone() const override;
		std::string get_type_name() const override;
		// throws: the configuration of an external layer's output is the caller's to state
		layer_configuration_specific get_output_layer_configuration_specific(
			const std::vector<layer_configuration_specific>& input_configuration_specific_list) const override;
		float get_forward_flops_per_entry(const std::vector<layer_configuration_specific>&) const override { return 0.0F; }
		void read_proto(const void * layer_proto) override;  // keeps every nested message of the layer's block
		void write_proto(void * layer_proto) const override; // and writes them back
		std::vector<std::string> get_parameter_strings() const override;

		std::string type_name;
		schema_param_block params; // the "<type>_param { ... }" messages, verbatim
	};

	// Four weight chunks of feature_map_count floats: gamma, beta, mean, inverse standard
	// deviation (nnforge/batch_norm_layer.h:26, batch_norm_layer.cpp:96-106). epsilon is carried
	// for schema round trips only; inference never reads it.
	class batch_norm_layer : public layer
	{
	public:
		explicit batch_norm_layer(unsigned int feature_map_count = 1, float epsilon = default_batch_normalization_epsilon);
		layer::ptr clone() const override;
		std::string get_type_name() const override;
		float get_forward_flops_per_entry(const std::vector<layer_configuration_specific>& input_configuration_specific_list) const override;
		void read_proto(const void * layer_proto) override;
		void write_proto(void * layer_proto) const override;
		data_config get_data_config() const override;
		void initialize_data(layer_data& data) const override; // gamma 1, beta 0, mean 0, inverse sigma 1
		std::vector<std::string> get_parameter_strings() const override;

		static const std::string layer_type_name;
		static const float default_batch_normalization_epsilon;

		unsigned int feature_map_count;
		float epsilon;

	private:
		void check();
	};

	// nnforge/rectified_linear_layer.h:24-47; type name "ReLU"
	class rectified_linear_layer : public layer
	{
	public:
		explicit rectified_linear_layer(float negative_slope = 0.0F);
		layer::ptr clone() const override;
		std::string get_type_name() const override;
		float get_forward_flops_per_entry(const std::vector<layer_configuration_specific>& input_configuration_specific_list) const override;
		void read_proto(const void * layer_proto) override;
		void write_proto(void * layer_proto) const override;
		std::vector<std::string> get_parameter_strings() const override;

		static const std::string layer_type_name;
		float negative_slope;
	};

	// One slope per feature map in chunk 0 (nnforge/parametric_rectified_linear_layer.h:26-63); "PReLU"
	class parametric_rectified_linear_layer : public layer
	{
	public:
		explicit parametric_rectified_linear_layer(unsigned int feature_map_count = 1);
		layer::ptr clone() const override;
		std::string get_type_name() const override;
		float get_forward_flops_per_entry(const std::vector<layer_configuration_specific>& input_configuration_specific_list) const override;
		void read_proto(const void * layer_proto) override;
		void write_proto(void * layer_proto) const override;
		data_config get_data_config() const override;
		void initialize_data(layer_data& data) const override; // 0.25
		std::vector<std::string> get_parameter_strings() const override;

		static const std::string layer_type_name;
		unsigned int feature_map_count;

	private:
		void check();
	};

	// nnforge/exponential_linear_layer.h:26-40; "ELU" (no alpha parameter exists)
	class exponential_linear_layer : public layer
	{
	public:
		exponential_linear_layer() = default;
		layer::ptr clone() const override;
		std::string get_type_name() const override;
		float get_forward_flops_per_entry(const std::vector<layer_configuration_specific>& input_configuration_specific_list) const override;
		static const std::string layer_type_name;
	};

	// nnforge/sigmoid_layer.h:26-40; "Sigmoid"
	class sigmoid_layer : public layer
	{
	public:
		sigmoid_layer() = default;
		layer::ptr clone() const override;
		std::string get_type_name() const override;
		float get_forward_flops_per_entry(const std::vector<layer_configuration_specific>& input_configuration_specific_list) const override;
		static const std::string layer_type_name;
	};

	// f(x) = scale * tanh(steepness * x) (nnforge/hyperbolic_tangent_layer.h:30-56); "TanH"
	class hyperbolic_tangent_layer : public layer
	{
	public:
		explicit hyperbolic_tangent_layer(float scale = 1.0F, float steepness = 1.0F);
		layer::ptr clone() const override;
		std::string get_type_name() const override;
		float get_forward_flops_per_entry(const std::vector<layer_configuration_specific>& input_configuration_specific_list) const override;
		void read_proto(const void * layer_proto) override;
		void write_proto(void * layer_proto) const override;
		std::vector<std::string> get_parameter_strings() const override;

		static const std::string layer_type_name;
		float scale;
		float steepness;
	};

	// Sum of all inputs times alpha (nnforge/add_layer.h:24-51); "Add"
	class add_layer : public layer
	{
	public:
		explicit add_layer(float alpha = 1.0F);
		layer::ptr clone() const override;
		// all inputs must have the same neuron count (nnforge/add_layer.cpp:44-55)
		layer_configuration_specific get_output_layer_configuration_specific(
			const std::vector<layer_configuration_specific>& input_configuration_specific_list) const override;
		std::string get_type_name() const override;
		float get_forward_flops_per_entry(const std::vector<layer_configuration_specific>& input_configuration_specific_list) const override;
		void read_proto(const void * layer_proto) override;
		void write_proto(void * layer_proto) const override;
		std::vector<std::string> get_parameter_strings() const override;

		static const std::string layer_type_name;
		float alpha;
	};

	// nnforge/softmax_layer.h:23-37; "Softmax"
	class softmax_layer : public layer
	{
	public:
		softmax_layer() = default;
		layer::ptr clone() const override;
		std::string get_type_name() const override;
		float get_forward_flops_per_entry(const std::vector<layer_configuration_specific>& input_configuration_specific_list) const override;
		static const std::string layer_type_name;
	};

	// Spatial average subsampling with relative factors (the window sizes), the subset of
	// nnforge/average_subsampling_layer.h this backend runs: two spatial dimensions, no
	// feature-map or entry subsampling. "AverageSubsampling"
	class average_subsampling_layer : public layer
	{
	public:
		explicit average_subsampling_layer(
			const std::vector<unsigned int>& subsampling_sizes = std::vector<unsigned int>(),
			float alpha = -std::numeric_limits<float>::max());
		layer::ptr clone() const override;
		layer_configuration_specific get_output_layer_configuration_specific(
			const std::vector<layer_configuration_specific>& input_configuration_specific_list) const override;
		std::string get_type_name() const override;
		float get_forward_flops_per_entry(const std::vector<layer_configuration_specific>& input_configuration_specific_list) const override;
		void read_proto(const void * layer_proto) override;
		void write_proto(void * layer_proto) const override;
		std::vector<std::string> get_parameter_strings() const override;

		bool has_alpha() const { return alpha != -std::numeric_limits<float>::max(); }

		// 1 / (number of window elements) unless alpha is set, for relative spatial windows only
		// (average_subsampling_layer::get_effective_alpha given the full configurations,
		// nnforge/average_subsampling_layer.cpp:287-303)
		float get_effective_alpha() const;

		// What the reference's PLAIN tester multiplies by: it passes bare feature-map counts where
		// configurations are expected (nnforge/plain/average_subsampling_layer_tester_plain.cpp:82),
		// so without an explicit alpha the spatial window does not divide and only the feature-map and
		// entry windows do: 1 / (feature_map_window * entry_subsampling_size).
		float get_plain_tester_alpha(unsigned int feature_map_window = 1) const;

		// the window of dimension i / over feature maps for these input and output sizes
		// (nnforge/average_subsampling_layer.cpp:104-132: a relative size is the window itself, an absolute
		// one is the wanted output size and the window is input / output, which must reproduce it)
		unsigned int get_subsampling_size(unsigned int dimension_id, unsigned int input, unsigned int output) const;
		unsigned int get_fm_subsampling_size(unsigned int input, unsigned int output) const;

		// one output entry per entry_subsampling_size input entries (nnforge/average_subsampling_layer.cpp:240-243)
		tiling_factor get_tiling_factor() const override { return tiling_factor(entry_subsampling_size).get_inverse(); }

		// 1 / (number of window elements, feature maps and entries included) unless alpha is set, for these
		// windows (average_subsampling_layer::get_effective_alpha given the full configurations)
		float get_effective_alpha(const std::vector<unsigned int>& windows, unsigned int feature_map_window) const;

		static const std::string layer_type_name;
		std::vector<unsigned int> subsampling_sizes;    // x first: window size (relative) or output size (absolute)
		std::vector<bool> subsampling_relative;         // per dimension; empty = all relative
		unsigned int feature_map_subsampling_size = 1;  // window (relative) or output feature map count (absolute)
		bool feature_map_relative = true;
		unsigned int entry_subsampling_size = 1;
		float alpha;

		bool is_relative(size_t dimension_id) const { return (dimension_id >= subsampling_relative.size()) || subsampling_relative[dimension_id]; }
	};

	// nnforge/absolute_layer.h; "Absolute"
	class absolute_layer : public layer
	{
	public:
		absolute_layer() = default;
		layer::ptr clone() const override;
		std::string get_type_name() const override;
		float get_forward_flops_per_entry(const std::vector<layer_configuration_specific>& input_configuration_specific_list) const override;
		static const std::string layer_type_name;
	};

	// nnforge/dropout_layer.h:26-52; "Dropout". At inference the layer passes its input on; the
	// parameters are kept for schema round trips.
	class dropout_layer : public layer
	{
	public:
		explicit dropout_layer(float dropout_rate = 0.5F, bool per_feature_map = false);
		layer::ptr clone() const override;
		std::string get_type_name() const override;
		float get_forward_flops_per_entry(const std::vector<layer_configuration_specific>&) const override { return 0.0F; }
		void read_proto(const void * layer_proto) override;
		void write_proto(void * layer_proto) const override;
		std::vector<std::string> get_parameter_strings() const override;

		static const std::string layer_type_name;
		float dropout_rate;
		bool per_feature_map;

	private:
		void check();
	};

	// Joins its inputs along feature maps (nnforge/concat_layer.h:23-45); "Concat"
	class concat_layer : public layer
	{
	public:
		concat_layer() = default;
		layer::ptr clone() const override;
		// feature maps add up; neurons per feature map must agree (nnforge/concat_layer.cpp:44-58)
		layer_configuration_specific get_output_layer_configuration_specific(
			const std::vector<layer_configuration_specific>& input_configuration_specific_list) const override;
		std::string get_type_name() const override;
		float get_forward_flops_per_entry(const std::vector<layer_configuration_specific>&) const override { return 0.0F; }
		static const std::string layer_type_name;
	};

	// Maximum over feature_map_subsampling_size feature maps that lie output-feature-map-count apart
	// (nnforge/maxout_layer.h:25-57); "Maxout"
	class maxout_layer : public layer
	{
	public:
		explicit maxout_layer(unsigned int feature_map_subsampling_size = 2);
		layer::ptr clone() const override;
		layer_configuration_specific get_output_layer_configuration_specific(
			const std::vector<layer_configuration_specific>& input_configuration_specific_list) const override;
		std::string get_type_name() const override;
		float get_forward_flops_per_entry(const std::vector<layer_configuration_specific>& input_configuration_specific_list) const override;
		void read_proto(const void * layer_proto) override;
		void write_proto(void * layer_proto) const override;
		std::vector<std::string> get_parameter_strings() const override;

		static const std::string layer_type_name;
		unsigned int feature_map_subsampling_size;

	private:
		void check();
	};

	// Maximum (or minimum) over windows (nnforge/max_subsampling_layer.h:27-82); "MaxSubsampling".
	// Spatial windows with strides and round up, windows over feature maps and over entries, and tiling:
	// with tiling every input entry gives one output entry per shift of the window grid.
	class max_subsampling_layer : public layer
	{
	public:
		explicit max_subsampling_layer(
			const std::vector<unsigned int>& subsampling_sizes = std::vector<unsigned int>(),
			unsigned int feature_map_subsampling_size = 1,
			unsigned int entry_subsampling_size = 1,
			bool is_min = false,
			bool tiling = false,
			const std::vector<bool>& round_ups = std::vector<bool>(),
			const std::vector<unsigned int>& strides = std::vector<unsigned int>());
		layer::ptr clone() const override;
		// (input + stride - window + (round_up ? window - 1 : 0)) / stride per dimension; with tiling
		// (input - (window - 1)) / window (nnforge/max_subsampling_layer.cpp:106-144)
		layer_configuration_specific get_output_layer_configuration_specific(
			const std::vector<layer_configuration_specific>& input_configuration_specific_list) const override;
		std::string get_type_name() const override;
		float get_forward_flops_per_entry(const std::vector<layer_configuration_specific>& input_configuration_specific_list) const override;
		void read_proto(const void * layer_proto) override;
		void write_proto(void * layer_proto) const override;
		std::vector<std::string> get_parameter_strings() const override;
		// tiling: the product of the window sizes; otherwise one over entry_subsampling_size
		// (nnforge/max_subsampling_layer.cpp:239-268)
		tiling_factor get_tiling_factor() const override;
		std::vector<tiling_factor> get_tiling_factor_list() const;

		static const std::string layer_type_name;
		std::vector<unsigned int> subsampling_sizes; // x first
		unsigned int feature_map_subsampling_size;
		unsigned int entry_subsampling_size;
		bool is_min;
		bool tiling;
		std::vector<bool> round_ups;
		std::vector<unsigned int> strides;

	private:
		void check();
	};
}
