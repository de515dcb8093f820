#include "nnforge_hip/layers.h"

#include <cstdio>
#include <sstream>

namespace nnforge
{
	namespace
	{
		float neuron_count_of(const std::vector<layer_configuration_specific>& configs)
		{
			if (configs.empty())
				throw neural_network_exception("flops requested for a layer without input configuration");
			return static_cast<float>(configs[0].get_neuron_count());
		}

		std::string fixed3(float v)
		{
			char buf[64];
			std::snprintf(buf, sizeof(buf), "%.3f", static_cast<double>(v));
			return buf;
		}

		std::string float_text(float v)
		{
			char buf[64];
			std::snprintf(buf, sizeof(buf), "%.9g", static_cast<double>(v));
			return buf;
		}
	}

	// ---- data ------------------------------------------------------------------------------

	const std::string data_layer::layer_type_name = "Data";
	layer::ptr data_layer::clone() const { return layer::ptr(new data_layer(*this)); }
	std::string data_layer::get_type_name() const { return layer_type_name; }

	// ---- batch norm ------------------------------------------------------------------------

	const std::string batch_norm_layer::layer_type_name = "BatchNorm";
	const float batch_norm_layer::default_batch_normalization_epsilon = 2.0e-5F;

	batch_norm_layer::batch_norm_layer(unsigned int feature_map_count, float epsilon)
		: feature_map_count(feature_map_count), epsilon(epsilon)
	{
		check();
	}

	void batch_norm_layer::check()
	{
		if (feature_map_count == 0)
			throw neural_network_exception("Feature map count should be > 0 for batch norm layer");
	}

	layer::ptr batch_norm_layer::clone() const { return layer::ptr(new batch_norm_layer(*this)); }
	std::string batch_norm_layer::get_type_name() const { return layer_type_name; }

	float batch_norm_layer::get_forward_flops_per_entry(const std::vector<layer_configuration_specific>& configs) const
	{
		return neuron_count_of(configs) * 5.0F; // the reference's count (nnforge/batch_norm_layer.cpp:66)
	}

	void batch_norm_layer::read_proto(const void * layer_proto)
	{
		const schema_param_block * block = static_cast<const schema_param_block *>(layer_proto)->child("batch_norm_param");
		if (block == nullptr)
			throw neural_network_exception("No batch_norm_param specified for layer " + instance_name + " of type " + layer_type_name);
		feature_map_count = block->require_uint("feature_map_count", "batch_norm_param of layer " + instance_name);
		epsilon = block->get_float("epsilon", default_batch_normalization_epsilon);
		check();
	}

	void batch_norm_layer::write_proto(void * layer_proto) const
	{
		schema_param_block& param = static_cast<schema_param_block *>(layer_proto)->add_block("batch_norm_param");
		param.set("feature_map_count", std::to_string(feature_map_count));
		if (epsilon != default_batch_normalization_epsilon)
			param.set("epsilon", float_text(epsilon));
	}

	data_config batch_norm_layer::get_data_config() const
	{
		return data_config(4, feature_map_count);
	}

	void batch_norm_layer::initialize_data(layer_data& data) const
	{
		check_layer_data_consistency(data);
		std::fill(data[0].begin(), data[0].end(), 1.0F);
		std::fill(data[1].begin(), data[1].end(), 0.0F);
		std::fill(data[2].begin(), data[2].end(), 0.0F);
		std::fill(data[3].begin(), data[3].end(), 1.0F);
	}

	std::vector<std::string> batch_norm_layer::get_parameter_strings() const
	{
		std::stringstream ss;
		ss << "fm " << feature_map_count;
		if (epsilon != default_batch_normalization_epsilon)
			ss << ", epsilon = " << epsilon;
		return std::vector<std::string>(1, ss.str());
	}

	// ---- ReLU ------------------------------------------------------------------------------

	const std::string rectified_linear_layer::layer_type_name = "ReLU";

	rectified_linear_layer::rectified_linear_layer(float negative_slope) : negative_slope(negative_slope) {}
	layer::ptr rectified_linear_layer::clone() const { return layer::ptr(new rectified_linear_layer(*this)); }
	std::string rectified_linear_layer::get_type_name() const { return layer_type_name; }

	float rectified_linear_layer::get_forward_flops_per_entry(const std::vector<layer_configuration_specific>& configs) const
	{
		return neuron_count_of(configs);
	}

	void rectified_linear_layer::read_proto(const void * layer_proto)
	{
		const schema_param_block * block = static_cast<const schema_param_block *>(layer_proto)->child("relu_param");
		negative_slope = (block != nullptr) ? block->get_float("negative_slope", 0.0F) : 0.0F;
	}

	void rectified_linear_layer::write_proto(void * layer_proto) const
	{
		if (negative_slope != 0.0F)
			static_cast<schema_param_block *>(layer_proto)->add_block("relu_param").set("negative_slope", float_text(negative_slope));
	}

	std::vector<std::string> rectified_linear_layer::get_parameter_strings() const
	{
		std::vector<std::string> res;
		if (negative_slope != 0.0F)
			res.push_back("negative slope " + float_text(negative_slope));
		return res;
	}

	// ---- PReLU -----------------------------------------------------------------------------

	const std::string parametric_rectified_linear_layer::layer_type_name = "PReLU";

	parametric_rectified_linear_layer::parametric_rectified_linear_layer(unsigned int feature_map_count)
		: feature_map_count(feature_map_count)
	{
		check();
	}

	void parametric_rectified_linear_layer::check()
	{
		if (feature_map_count == 0)
			throw neural_network_exception("Feature map count should be > 0 for parametric rectified linear layer");
	}

	layer::ptr parametric_rectified_linear_layer::clone() const { return layer::ptr(new parametric_rectified_linear_layer(*this)); }
	std::string parametric_rectified_linear_layer::get_type_name() const { return layer_type_name; }

	float parametric_rectified_linear_layer::get_forward_flops_per_entry(const std::vector<layer_configuration_specific>& configs) const
	{
		return neuron_count_of(configs) * 2.0F;
	}

	void parametric_rectified_linear_layer::read_proto(const void * layer_proto)
	{
		const schema_param_block * block = static_cast<const schema_param_block *>(layer_proto)->child("prelu_param");
		if (block == nullptr)
			throw neural_network_exception("No prelu_param specified for layer " + instance_name + " of type " + layer_type_name);
		feature_map_count = block->require_uint("feature_map_count", "prelu_param of layer " + instance_name);
		check();
	}

	void parametric_rectified_linear_layer::write_proto(void * layer_proto) const
	{
		static_cast<schema_param_block *>(layer_proto)->add_block("prelu_param").set("feature_map_count", std::to_string(feature_map_count));
	}

	data_config parametric_rectified_linear_layer::get_data_config() const
	{
		return data_config(1, feature_map_count);
	}

	void parametric_rectified_linear_layer::initialize_data(layer_data& data) const
	{
		check_layer_data_consistency(data);
		std::fill(data[0].begin(), data[0].end(), 0.25F);
	}

	std::vector<std::string> parametric_rectified_linear_layer::get_parameter_strings() const
	{
		return std::vector<std::string>(1, "fm " + std::to_string(feature_map_count));
	}

	// ---- ELU, Sigmoid ----------------------------------------------------------------------

	const std::string exponential_linear_layer::layer_type_name = "ELU";
	layer::ptr exponential_linear_layer::clone() const { return layer::ptr(new exponential_linear_layer(*this)); }
	std::string exponential_linear_layer::get_type_name() const { return layer_type_name; }
	float exponential_linear_layer::get_forward_flops_per_entry(const std::vector<layer_configuration_specific>& configs) const
	{
		return neuron_count_of(configs) * 2.0F;
	}

	const std::string sigmoid_layer::layer_type_name = "Sigmoid";
	layer::ptr sigmoid_layer::clone() const { return layer::ptr(new sigmoid_layer(*this)); }
	std::string sigmoid_layer::get_type_name() const { return layer_type_name; }
	float sigmoid_layer::get_forward_flops_per_entry(const std::vector<layer_configuration_specific>& configs) const
	{
		return neuron_count_of(configs) * 4.0F;
	}

	// ---- TanH ------------------------------------------------------------------------------

	const std::string hyperbolic_tangent_layer::layer_type_name = "TanH";

	hyperbolic_tangent_layer::hyperbolic_tangent_layer(float scale, float steepness) : scale(scale), steepness(steepness) {}
	layer::ptr hyperbolic_tangent_layer::clone() const { return layer::ptr(new hyperbolic_tangent_layer(*this)); }
	std::string hyperbolic_tangent_layer::get_type_name() const { return layer_type_name; }

	float hyperbolic_tangent_layer::get_forward_flops_per_entry(const std::vector<layer_configuration_specific>& configs) const
	{
		return neuron_count_of(configs) * 6.0F;
	}

	void hyperbolic_tangent_layer::read_proto(const void * layer_proto)
	{
		const schema_param_block * block = static_cast<const schema_param_block *>(layer_proto)->child("tanh_param");
		scale = (block != nullptr) ? block->get_float("scale", 1.0F) : 1.0F;
		steepness = (block != nullptr) ? block->get_float("steepness", 1.0F) : 1.0F;
	}

	void hyperbolic_tangent_layer::write_proto(void * layer_proto) const
	{
		if ((scale == 1.0F) && (steepness == 1.0F))
			return;
		schema_param_block& param = static_cast<schema_param_block *>(layer_proto)->add_block("tanh_param");
		if (scale != 1.0F)
			param.set("scale", float_text(scale));
		if (steepness != 1.0F)
			param.set("steepness", float_text(steepness));
	}

	std::vector<std::string> hyperbolic_tangent_layer::get_parameter_strings() const
	{
		std::string s;
		if (scale != 1.0F)
			s += "scale " + fixed3(scale);
		if (steepness != 1.0F)
			s += std::string(s.empty() ? "" : ", ") + "steepness " + fixed3(steepness);
		return s.empty() ? std::vector<std::string>() : std::vector<std::string>(1, s);
	}

	// ---- Add -------------------------------------------------------------------------------

	const std::string add_layer::layer_type_name = "Add";

	add_layer::add_layer(float alpha) : alpha(alpha) {}
	layer::ptr add_layer::clone() const { return layer::ptr(new add_layer(*this)); }
	std::string add_layer::get_type_name() const { return layer_type_name; }

	layer_configuration_specific add_layer::get_output_layer_configuration_specific(
		const std::vector<layer_configuration_specific>& configs) const
	{
		if (configs.empty())
			throw neural_network_exception("Layer " + instance_name + " has no input configuration");
		const unsigned int neuron_count_per_entry = configs[0].get_neuron_count();
		for(size_t i = 1; i < configs.size(); ++i)
		{
			if (configs[i].get_neuron_count() != neuron_count_per_entry)
				throw neural_network_exception("Neuron count per entry mismatch in 2 input layers for add_layer");
		}
		return configs[0];
	}

	float add_layer::get_forward_flops_per_entry(const std::vector<layer_configuration_specific>& configs) const
	{
		return neuron_count_of(configs) * static_cast<float>(configs.size());
	}

	void add_layer::read_proto(const void * layer_proto)
	{
		const schema_param_block * block = static_cast<const schema_param_block *>(layer_proto)->child("add_param");
		alpha = (block != nullptr) ? block->get_float("alpha", 1.0F) : 1.0F;
	}

	void add_layer::write_proto(void * layer_proto) const
	{
		if (alpha != 1.0F)
			static_cast<schema_param_block *>(layer_proto)->add_block("add_param").set("alpha", float_text(alpha));
	}

	std::vector<std::string> add_layer::get_parameter_strings() const
	{
		std::vector<std::string> res;
		if (alpha != 1.0F)
			res.push_back("alpha " + float_text(alpha));
		return res;
	}

	// ---- Softmax ---------------------------------------------------------------------------

	const std::string softmax_layer::layer_type_name = "Softmax";
	layer::ptr softmax_layer::clone() const { return layer::ptr(new softmax_layer(*this)); }
	std::string softmax_layer::get_type_name() const { return layer_type_name; }

	float softmax_layer::get_forward_flops_per_entry(const std::vector<layer_configuration_specific>& configs) const
	{
		if (configs.empty())
			throw neural_network_exception("flops requested for a layer without input configuration");
		return static_cast<float>(configs[0].get_neuron_count_per_feature_map() * (configs[0].feature_map_count * 3 - 1));
	}

	// ---- AverageSubsampling ----------------------------------------------------------------

	const std::string average_subsampling_layer::layer_type_name = "AverageSubsampling";

	average_subsampling_layer::average_subsampling_layer(const std::vector<unsigned int>& subsampling_sizes, float alpha)
		: subsampling_sizes(subsampling_sizes), alpha(alpha)
	{
		for(unsigned int s : subsampling_sizes)
			if (s == 0)
				throw neural_network_exception("window dimension for average subsampling layer may not be zero");
	}

	layer::ptr average_subsampling_layer::clone() const { return layer::ptr(new average_subsampling_layer(*this)); }
	std::string average_subsampling_layer::get_type_name() const { return layer_type_name; }

	layer_configuration_specific average_subsampling_layer::get_output_layer_configuration_specific(
		const std::vector<layer_configuration_specific>& configs) const
	{
		if (configs.empty())
			throw neural_network_exception("Layer " + instance_name + " has no input configuration");
		const layer_configuration_specific& in = configs[0];
		if (in.get_dimension_count() != subsampling_sizes.size())
			throw neural_network_exception("Dimension count in layer (" + std::to_string(subsampling_sizes.size()) + ") and input configuration (" + std::to_string(in.get_dimension_count()) + ") don't match");
		layer_configuration_specific res;
		// nnforge/average_subsampling_layer.cpp:74-81
		if (feature_map_relative)
			res.feature_map_count = in.feature_map_count / feature_map_subsampling_size;
		else
		{
			res.feature_map_count = feature_map_subsampling_size;
			get_fm_subsampling_size(in.feature_map_count, res.feature_map_count);
		}
		if (res.feature_map_count == 0)
			throw neural_network_exception("Input feature map count (" + std::to_string(in.feature_map_count) + ") is smaller than feature map subsampling size (" + std::to_string(feature_map_subsampling_size) + ")");
		for(size_t i = 0; i < subsampling_sizes.size(); ++i)
		{
			if (is_relative(i))
			{
				if (in.dimension_sizes[i] < subsampling_sizes[i])
					throw neural_network_exception("Input configuration size (" + std::to_string(in.dimension_sizes[i]) + ") of dimension (" + std::to_string(i) + ") is smaller than subsampling size (" + std::to_string(subsampling_sizes[i]) + ")");
				res.dimension_sizes.push_back(in.dimension_sizes[i] / subsampling_sizes[i]);
			}
			else
			{
				if (in.dimension_sizes[i] < subsampling_sizes[i])
					throw neural_network_exception("Input configuration size (" + std::to_string(in.dimension_sizes[i]) + ") of dimension (" + std::to_string(i) + ") is smaller than subsampled size (" + std::to_string(subsampling_sizes[i]) + ")");
				get_subsampling_size(static_cast<unsigned int>(i), in.dimension_sizes[i], subsampling_sizes[i]);
				res.dimension_sizes.push_back(subsampling_sizes[i]);
			}
		}
		return res;
	}

	unsigned int average_subsampling_layer::get_subsampling_size(unsigned int dimension_id, unsigned int input, unsigned int output) const
	{
		if (is_relative(dimension_id))
			return subsampling_sizes[dimension_id];
		const unsigned int factor = (output == 0) ? 0 : input / output;
		if ((factor == 0) || (input / factor != output))
			throw neural_network_exception("Cannot calculate subsampling factor for input " + std::to_string(input) + " and output " + std::to_string(output));
		return factor;
	}

	unsigned int average_subsampling_layer::get_fm_subsampling_size(unsigned int input, unsigned int output) const
	{
		if (feature_map_relative)
			return feature_map_subsampling_size;
		const unsigned int factor = (output == 0) ? 0 : input / output;
		if ((factor == 0) || (input / factor != output))
			throw neural_network_exception("Cannot calculate fm subsampling factor for input " + std::to_string(input) + " and output " + std::to_string(output));
		return factor;
	}

	float average_subsampling_layer::get_forward_flops_per_entry(const std::vector<layer_configuration_specific>& configs) const
	{
		// nnforge/average_subsampling_layer.cpp:267-285: output neurons * window elements
		const layer_configuration_specific out = get_output_layer_configuration_specific(configs);
		float per_item = static_cast<float>(get_fm_subsampling_size(configs[0].feature_map_count, out.feature_map_count));
		for(size_t i = 0; i < subsampling_sizes.size(); ++i)
			per_item *= static_cast<float>(get_subsampling_size(static_cast<unsigned int>(i), configs[0].dimension_sizes[i], out.dimension_sizes[i]));
		return static_cast<float>(out.get_neuron_count()) * per_item;
	}

	void average_subsampling_layer::read_proto(const void * layer_proto)
	{
		const schema_param_block * block = static_cast<const schema_param_block *>(layer_proto)->child("average_subsampling_param");
		if (block == nullptr)
			throw neural_network_exception("No average_subsampling_param specified for layer " + instance_name + " of type " + layer_type_name);
		subsampling_sizes.clear();
		subsampling_relative.clear();
		for(const schema_param_block * dim : block->children("dimension_param"))
		{
			// nnforge/average_subsampling_layer.cpp:186-194
			if (dim->has("subsampling_size"))
			{
				subsampling_sizes.push_back(dim->get_uint("subsampling_size", 1));
				subsampling_relative.push_back(true);
			}
			else if (dim->has("subsampled_size"))
			{
				subsampling_sizes.push_back(dim->get_uint("subsampled_size", 1));
				subsampling_relative.push_back(false);
			}
			else
				throw neural_network_exception("Neither subsampling_size nor subsampled_size specified for dimension_param of average_subsampling_layer");
		}
		feature_map_subsampling_size = 1;
		feature_map_relative = true;
		const std::vector<const schema_param_block *> fm = block->children("feature_map_param");
		if (!fm.empty())
		{
			if (fm[0]->has("subsampling_size"))
				feature_map_subsampling_size = fm[0]->get_uint("subsampling_size", 1);
			else if (fm[0]->has("subsampled_size"))
			{
				feature_map_subsampling_size = fm[0]->get_uint("subsampled_size", 1);
				feature_map_relative = false;
			}
			else
				throw neural_network_exception("Neither subsampling_size nor subsampled_size specified for feature_map_param of average_subsampling_layer");
		}
		const std::vector<const schema_param_block *> en = block->children("entry_param");
		entry_subsampling_size = en.empty() ? 1 : en[0]->require_uint("subsampling_size", "entry_param of layer " + instance_name);
		alpha = block->has("alpha") ? block->get_float("alpha", 0.0F) : -std::numeric_limits<float>::max();
		for(unsigned int s : subsampling_sizes)
			if (s == 0)
				throw neural_network_exception("window dimension for average subsampling layer may not be zero");
		if ((feature_map_subsampling_size == 0) || (entry_subsampling_size == 0))
			throw neural_network_exception("feature map and entry subsampling sizes for average subsampling layer may not be zero");
	}

	void average_subsampling_layer::write_proto(void * layer_proto) const
	{
		schema_param_block& param = static_cast<schema_param_block *>(layer_proto)->add_block("average_subsampling_param");
		for(size_t i = 0; i < subsampling_sizes.size(); ++i)
			param.add_block("dimension_param").set(is_relative(i) ? "subsampling_size" : "subsampled_size", std::to_string(subsampling_sizes[i]));
		if (!feature_map_relative || (feature_map_subsampling_size != 1))
			param.add_block("feature_map_param").set(feature_map_relative ? "subsampling_size" : "subsampled_size", std::to_string(feature_map_subsampling_size));
		if (entry_subsampling_size != 1)
			param.add_block("entry_param").set("subsampling_size", std::to_string(entry_subsampling_size));
		if (has_alpha())
			param.set("alpha", float_text(alpha));
	}

	std::vector<std::string> average_subsampling_layer::get_parameter_strings() const
	{
		std::stringstream ss;
		for(size_t i = 0; i < subsampling_sizes.size(); ++i)
			ss << (i == 0 ? "" : "x") << (is_relative(i) ? "" : "->") << subsampling_sizes[i];
		if (!feature_map_relative || (feature_map_subsampling_size != 1))
			ss << ", fm " << (feature_map_relative ? "" : "->") << feature_map_subsampling_size;
		if (entry_subsampling_size != 1)
			ss << ", samples " << entry_subsampling_size;
		if (has_alpha())
			ss << ", alpha " << alpha;
		return std::vector<std::string>(1, ss.str());
	}

	float average_subsampling_layer::get_effective_alpha() const
	{
		return get_effective_alpha(subsampling_sizes, feature_map_relative ? feature_map_subsampling_size : 1);
	}

	float average_subsampling_layer::get_effective_alpha(const std::vector<unsigned int>& windows, unsigned int feature_map_window) const
	{
		if (has_alpha())
			return alpha;
		unsigned int elems = feature_map_window * entry_subsampling_size;
		for(unsigned int s : windows)
			elems *= s;
		return 1.0F / static_cast<float>(elems);
	}

	float average_subsampling_layer::get_plain_tester_alpha(unsigned int feature_map_window) const
	{
		return has_alpha() ? alpha : 1.0F / static_cast<float>(feature_map_window * entry_subsampling_size);
	}

	// ---- Absolute ----------------------------------------------------------------------------

	const std::string absolute_layer::layer_type_name = "Absolute";
	layer::ptr absolute_layer::clone() const { return layer::ptr(new absolute_layer(*this)); }
	std::string absolute_layer::get_type_name() const { return layer_type_name; }
	float absolute_layer::get_forward_flops_per_entry(const std::vector<layer_configuration_specific>& configs) const
	{
		return neuron_count_of(configs);
	}

	// ---- Dropout -----------------------------------------------------------------------------

	const std::string dropout_layer::layer_type_name = "Dropout";

	dropout_layer::dropout_layer(float dropout_rate, bool per_feature_map)
		: dropout_rate(dropout_rate), per_feature_map(per_feature_map)
	{
		check();
	}

	void dropout_layer::check()
	{
		if ((dropout_rate < 0.0F) || (dropout_rate >= 1.0F))
			throw neural_network_exception("Error constructing dropout_layer: dropout_rate equals " + float_text(dropout_rate) + ", it should be in [0.0F,1.0F)");
	}

	layer::ptr dropout_layer::clone() const { return layer::ptr(new dropout_layer(*this)); }
	std::string dropout_layer::get_type_name() const { return layer_type_name; }

	void dropout_layer::read_proto(const void * layer_proto)
	{
		const schema_param_block * block = static_cast<const schema_param_block *>(layer_proto)->child("dropout_param");
		// nnforge/dropout_layer.cpp:82-88: a missing block gives the defaults of the message
		dropout_rate = (block != nullptr) ? block->get_float("dropout_rate", 0.5F) : 0.5F;
		per_feature_map = (block != nullptr) ? block->get_bool("per_feature_map", false) : false;
		check();
	}

	void dropout_layer::write_proto(void * layer_proto) const
	{
		// nnforge/dropout_layer.cpp:70-80 writes the block only for a rate other than 0.5
		if (dropout_rate != 0.5F)
		{
			schema_param_block& param = static_cast<schema_param_block *>(layer_proto)->add_block("dropout_param");
			param.set("dropout_rate", float_text(dropout_rate));
			if (per_feature_map)
				param.set("per_feature_map", "true");
		}
	}

	std::vector<std::string> dropout_layer::get_parameter_strings() const
	{
		char buf[64];
		std::snprintf(buf, sizeof(buf), "dropout rate %.3f", static_cast<double>(dropout_rate));
		std::string res(buf);
		if (per_feature_map)
			res += ", per fm";
		return std::vector<std::string>(1, res);
	}

	// ---- layers computed elsewhere -------------------------------------------------------------

	external_layer::external_layer(const std::string& type_name) : type_name(type_name) {}
	layer::ptr external_layer::clone() const { return layer::ptr(new external_layer(*this)); }
	std::string external_layer::get_type_name() const { return type_name; }

	layer_configuration_specific external_layer::get_output_layer_configuration_specific(const std::vector<layer_configuration_specific>&) const
	{
		throw neural_network_exception("Layer " + instance_name + " of type " + type_name
			+ " is computed outside this backend: its output configuration has to be supplied like a data layer's");
	}

	void external_layer::read_proto(const void * layer_proto)
	{
		params = schema_param_block();
		for(const std::pair<std::string, schema_param_block>& b : static_cast<const schema_param_block *>(layer_proto)->blocks)
			if (b.first != "input_layer_name")
				params.blocks.push_back(b);
	}

	void external_layer::write_proto(void * layer_proto) const
	{
		for(const std::pair<std::string, schema_param_block>& b : params.blocks)
			static_cast<schema_param_block *>(layer_proto)->blocks.push_back(b);
	}

	std::vector<std::string> external_layer::get_parameter_strings() const
	{
		return std::vector<std::string>(1, "computed elsewhere");
	}

	// ---- Concat ------------------------------------------------------------------------------

	const std::string concat_layer::layer_type_name = "Concat";
	layer::ptr concat_layer::clone() const { return layer::ptr(new concat_layer(*this)); }
	std::string concat_layer::get_type_name() const { return layer_type_name; }

	layer_configuration_specific concat_layer::get_output_layer_configuration_specific(
		const std::vector<layer_configuration_specific>& configs) const
	{
		if (configs.empty())
			throw neural_network_exception("Layer " + instance_name + " has no input configuration");
		unsigned int feature_map_count = configs[0].feature_map_count;
		const unsigned int neuron_count_per_feature_map = configs[0].get_neuron_count_per_feature_map();
		for(size_t i = 1; i < configs.size(); ++i)
		{
			feature_map_count += configs[i].feature_map_count;
			if (configs[i].get_neuron_count_per_feature_map() != neuron_count_per_feature_map)
				throw neural_network_exception("Neuron count per feature maps mismatch in 2 input layers for concat_layer");
		}
		return layer_configuration_specific(feature_map_count, configs[0].dimension_sizes);
	}

	// ---- Maxout ------------------------------------------------------------------------------

	const std::string maxout_layer::layer_type_name = "Maxout";

	maxout_layer::maxout_layer(unsigned int feature_map_subsampling_size)
		: feature_map_subsampling_size(feature_map_subsampling_size)
	{
		check();
	}

	void maxout_layer::check()
	{
		if (feature_map_subsampling_size < 2)
			throw neural_network_exception("Feature map subsampling size should be >= 2 for maxout layer");
	}

	layer::ptr maxout_layer::clone() const { return layer::ptr(new maxout_layer(*this)); }
	std::string maxout_layer::get_type_name() const { return layer_type_name; }

	layer_configuration_specific maxout_layer::get_output_layer_configuration_specific(
		const std::vector<layer_configuration_specific>& configs) const
	{
		if (configs.empty())
			throw neural_network_exception("Layer " + instance_name + " has no input configuration");
		if ((configs[0].feature_map_count % feature_map_subsampling_size) != 0)
			throw neural_network_exception("Feature map count in layer (" + std::to_string(configs[0].feature_map_count) + ") is not evenly divisible by feature map subsampling count (" + std::to_string(feature_map_subsampling_size) + ")");
		return layer_configuration_specific(configs[0].feature_map_count / feature_map_subsampling_size, configs[0].dimension_sizes);
	}

	float maxout_layer::get_forward_flops_per_entry(const std::vector<layer_configuration_specific>& configs) const
	{
		return static_cast<float>(get_output_layer_configuration_specific(configs).get_neuron_count()) * static_cast<float>(feature_map_subsampling_size - 1);
	}

	void maxout_layer::read_proto(const void * layer_proto)
	{
		const schema_param_block * block = static_cast<const schema_param_block *>(layer_proto)->child("maxout_param");
		if (block == nullptr)
			throw neural_network_exception("No maxout_param specified for layer " + instance_name + " of type " + layer_type_name);
		feature_map_subsampling_size = block->require_uint("feature_map_subsampling_size", "maxout_param of layer " + instance_name);
		check();
	}

	void maxout_layer::write_proto(void * layer_proto) const
	{
		static_cast<schema_param_block *>(layer_proto)->add_block("maxout_param").set("feature_map_subsampling_size", std::to_string(feature_map_subsampling_size));
	}

	std::vector<std::string> maxout_layer::get_parameter_strings() const
	{
		return std::vector<std::string>(1, "fm subsampling " + std::to_string(feature_map_subsampling_size));
	}

	// ---- MaxSubsampling ----------------------------------------------------------------------

	const std::string max_subsampling_layer::layer_type_name = "MaxSubsampling";

	max_subsampling_layer::max_subsampling_layer(
		const std::vector<unsigned int>& subsampling_sizes,
		unsigned int feature_map_subsampling_size,
		unsigned int entry_subsampling_size,
		bool is_min,
		bool tiling,
		const std::vector<bool>& round_ups,
		const std::vector<unsigned int>& strides)
		: subsampling_sizes(subsampling_sizes)
		, feature_map_subsampling_size(feature_map_subsampling_size)
		, entry_subsampling_size(entry_subsampling_size)
		, is_min(is_min)
		, tiling(tiling)
	{
		if (!round_ups.empty() && (round_ups.size() != subsampling_sizes.size()))
			throw neural_network_exception("Invalid dimension count " + std::to_string(round_ups.size()) + " for round ups");
		if (!strides.empty() && (strides.size() != subsampling_sizes.size()))
			throw neural_network_exception("Invalid dimension count " + std::to_string(strides.size()) + " for strides");
		this->round_ups = round_ups.empty() ? std::vector<bool>(subsampling_sizes.size(), false) : round_ups;
		this->strides = strides.empty() ? subsampling_sizes : strides;
		check();
	}

	void max_subsampling_layer::check()
	{
		for(unsigned int s : subsampling_sizes)
			if (s == 0)
				throw neural_network_exception("window dimension for max subsampling layer may not be zero");
		if (feature_map_subsampling_size == 0)
			throw neural_network_exception("feature map subsampling size for max subsampling layer may not be zero");
		if (entry_subsampling_size == 0)
			throw neural_network_exception("feature map subsampling size for max subsampling layer may not be zero"); // the reference's wording
		if (tiling && (entry_subsampling_size > 1))
			throw neural_network_exception("entry_subsampling_size cannot be set with tiling at the same time for max subsampling layer");
		if (tiling && (feature_map_subsampling_size > 1))
			throw neural_network_exception("feature_map_subsampling_size cannot be set with tiling at the same time for max subsampling layer");
		for(size_t i = 0; i < strides.size(); ++i)
			if (strides[i] == 0)
				throw neural_network_exception("stride dimension (" + std::to_string(i) + ") is 0");
		if (tiling)
			for(bool r : round_ups)
				if (r)
					throw neural_network_exception("round up cannot be set with tiling at the same time for max subsampling layer");
	}

	layer::ptr max_subsampling_layer::clone() const { return layer::ptr(new max_subsampling_layer(*this)); }
	std::string max_subsampling_layer::get_type_name() const { return layer_type_name; }

	layer_configuration_specific max_subsampling_layer::get_output_layer_configuration_specific(
		const std::vector<layer_configuration_specific>& configs) const
	{
		if (configs.empty())
			throw neural_network_exception("Layer " + instance_name + " has no input configuration");
		const layer_configuration_specific& in = configs[0];
		if (in.get_dimension_count() != subsampling_sizes.size())
			throw neural_network_exception("Dimension count in layer (" + std::to_string(subsampling_sizes.size()) + ") and input configuration (" + std::to_string(in.get_dimension_count()) + ") don't match");
		layer_configuration_specific res(in.feature_map_count / feature_map_subsampling_size);
		for(size_t i = 0; i < subsampling_sizes.size(); ++i)
		{
			if (tiling)
			{
				if (in.dimension_sizes[i] < (subsampling_sizes[i] * 2 - 1))
					throw neural_network_exception("Input configuration size (" + std::to_string(in.dimension_sizes[i]) + ") of dimension (" + std::to_string(i)
						+ ") is smaller than subsampling size (" + std::to_string(subsampling_sizes[i]) + ") * 2 - 1");
				res.dimension_sizes.push_back((in.dimension_sizes[i] - (subsampling_sizes[i] - 1)) / subsampling_sizes[i]);
				continue;
			}
			const int new_size = (static_cast<int>(in.dimension_sizes[i]) + static_cast<int>(strides[i]) - static_cast<int>(subsampling_sizes[i])
				+ (round_ups[i] ? static_cast<int>(subsampling_sizes[i]) - 1 : 0)) / static_cast<int>(strides[i]);
			if (new_size <= 0)
				throw neural_network_exception("Input configuration size (" + std::to_string(in.dimension_sizes[i]) + ") of dimension (" + std::to_string(i) + ") produces 0 output size");
			res.dimension_sizes.push_back(static_cast<unsigned int>(new_size));
		}
		return res;
	}

	tiling_factor max_subsampling_layer::get_tiling_factor() const
	{
		if (!tiling)
			return tiling_factor(entry_subsampling_size).get_inverse();
		tiling_factor res(1);
		for(const tiling_factor& t : get_tiling_factor_list())
			res *= t;
		return res;
	}

	std::vector<tiling_factor> max_subsampling_layer::get_tiling_factor_list() const
	{
		std::vector<tiling_factor> res;
		if (tiling)
			for(unsigned int s : subsampling_sizes)
				res.push_back(tiling_factor(s));
		return res;
	}

	float max_subsampling_layer::get_forward_flops_per_entry(const std::vector<layer_configuration_specific>& configs) const
	{
		const unsigned int neuron_count = get_output_layer_configuration_specific(configs).get_neuron_count();
		unsigned int per_item = feature_map_subsampling_size * entry_subsampling_size;
		for(unsigned int s : subsampling_sizes)
			per_item *= s;
		return static_cast<float>(neuron_count) * static_cast<float>(per_item - 1);
	}

	void max_subsampling_layer::read_proto(const void * layer_proto)
	{
		const schema_param_block * block = static_cast<const schema_param_block *>(layer_proto)->child("max_subsampling_param");
		if (block == nullptr)
			throw neural_network_exception("No max_subsampling_param specified for layer " + instance_name + " of type " + layer_type_name);
		subsampling_sizes.clear();
		round_ups.clear();
		strides.clear();
		for(const schema_param_block * dim : block->children("dimension_param"))
		{
			const unsigned int size = dim->require_uint("subsampling_size", "max_subsampling_param of layer " + instance_name);
			subsampling_sizes.push_back(size);
			round_ups.push_back(dim->get_bool("round_up", false));
			strides.push_back(dim->has("stride") ? dim->get_uint("stride", size) : size);
		}
		const std::vector<const schema_param_block *> fm = block->children("feature_map_param");
		feature_map_subsampling_size = fm.empty() ? 1 : fm[0]->require_uint("subsampling_size", "feature_map_param of layer " + instance_name);
		const std::vector<const schema_param_block *> en = block->children("entry_param");
		entry_subsampling_size = en.empty() ? 1 : en[0]->require_uint("subsampling_size", "entry_param of layer " + instance_name);
		tiling = block->get_bool("tiling", false);
		const std::string function = block->get_string("function", "MAX");
		if ((function != "MAX") && (function != "MIN"))
			throw neural_network_exception("Unknown function " + function + " in max_subsampling_param of layer " + instance_name);
		is_min = (function == "MIN");
		check();
	}

	void max_subsampling_layer::write_proto(void * layer_proto) const
	{
		schema_param_block& param = static_cast<schema_param_block *>(layer_proto)->add_block("max_subsampling_param");
		for(size_t i = 0; i < subsampling_sizes.size(); ++i)
		{
			schema_param_block& dim = param.add_block("dimension_param");
			dim.set("subsampling_size", std::to_string(subsampling_sizes[i]));
			if (round_ups[i])
				dim.set("round_up", "true");
			if (strides[i] != subsampling_sizes[i])
				dim.set("stride", std::to_string(strides[i]));
		}
		if (tiling)
			param.set("tiling", "true");
		if (feature_map_subsampling_size != 1)
			param.add_block("feature_map_param").set("subsampling_size", std::to_string(feature_map_subsampling_size));
		if (entry_subsampling_size != 1)
			param.add_block("entry_param").set("subsampling_size", std::to_string(entry_subsampling_size));
		if (is_min)
			param.set("function", "MIN");
	}

	std::vector<std::string> max_subsampling_layer::get_parameter_strings() const
	{
		std::stringstream ss;
		if (is_min)
			ss << "MIN";
		if (!subsampling_sizes.empty())
		{
			if (!ss.str().empty())
				ss << ", ";
			for(size_t i = 0; i < subsampling_sizes.size(); ++i)
				ss << (i == 0 ? "" : "x") << subsampling_sizes[i] << (round_ups[i] ? "_roundup_" : "");
		}
		if (strides != subsampling_sizes)
		{
			ss << ", stride ";
			for(size_t i = 0; i < strides.size(); ++i)
				ss << (i == 0 ? "" : "x") << strides[i];
		}
		if (feature_map_subsampling_size != 1)
			ss << (ss.str().empty() ? "" : ", ") << "fm " << feature_map_subsampling_size;
		if (entry_subsampling_size != 1)
			ss << (ss.str().empty() ? "" : ", ") << "samples " << entry_subsampling_size;
		if (tiling)
			ss << (ss.str().empty() ? "" : ", ") << "tiling";
		return std::vector<std::string>(1, ss.str());
	}
}
