#include "nnforge_hip/core.h"
#include "nnforge_hip/layers.h"

#include <algorithm>
#include <cstdlib>
#include <sstream>

namespace nnforge
{
	// nnforge/layer_action.h:56-78
	std::string layer_action::str() const
	{
		switch (at)
		{
		case forward: return "forward";
		case backward_weights: return "backward_weights";
		case backward_data_and_weights: return "backward_data_and_weights";
		case update_weights: return "update_weights";
		default: return "backward_data_" + std::to_string(backprop_index);
		}
	}

	namespace
	{
		template<class T> void write_pod(std::ostream& s, const T& v)
		{
			s.write(reinterpret_cast<const char *>(&v), sizeof(T));
		}

		template<class T> void read_pod(std::istream& s, T& v)
		{
			s.read(reinterpret_cast<char *>(&v), sizeof(T));
			if (!s)
				throw neural_network_exception("Unexpected end of stream while reading binary data");
		}
	}

	neural_network_exception::neural_network_exception(const std::string& message, const char * filename, int line_number)
		: std::runtime_error(message + " in " + filename + ":" + std::to_string(line_number))
	{
	}

	// ---- layer_configuration_specific ------------------------------------------------------

	void layer_configuration_specific::write(std::ostream& output_stream) const
	{
		write_pod(output_stream, feature_map_count);
		const unsigned int dimension_count = get_dimension_count();
		write_pod(output_stream, dimension_count);
		for(unsigned int size : dimension_sizes)
			write_pod(output_stream, size);
	}

	void layer_configuration_specific::read(std::istream& input_stream)
	{
		read_pod(input_stream, feature_map_count);
		unsigned int dimension_count;
		read_pod(input_stream, dimension_count);
		if (dimension_count > 16)
			throw neural_network_exception("Implausible dimension count " + std::to_string(dimension_count) + " in layer configuration");
		dimension_sizes.resize(dimension_count);
		for(unsigned int& size : dimension_sizes)
			read_pod(input_stream, size);
	}

	unsigned int layer_configuration_specific::get_neuron_count_per_feature_map() const
	{
		unsigned int neuron_count = 1;
		for(unsigned int size : dimension_sizes)
			neuron_count *= size;
		return neuron_count;
	}

	unsigned int layer_configuration_specific::get_neuron_count() const
	{
		return get_neuron_count_per_feature_map() * feature_map_count;
	}

	unsigned int layer_configuration_specific::get_pos(const std::vector<unsigned int>& offsets) const
	{
		if (offsets.size() != dimension_sizes.size())
			throw neural_network_exception("get_pos: " + std::to_string(offsets.size()) + " offsets for " + std::to_string(dimension_sizes.size()) + " dimensions");
		unsigned int res = 0;
		for(size_t i = dimension_sizes.size(); i-- > 0; )
			res = res * dimension_sizes[i] + offsets[i];
		return res;
	}

	std::vector<unsigned int> layer_configuration_specific::get_offsets(unsigned int pos) const
	{
		std::vector<unsigned int> res(dimension_sizes.size());
		for(size_t i = 0; i < dimension_sizes.size(); ++i)
		{
			res[i] = pos % dimension_sizes[i];
			pos /= dimension_sizes[i];
		}
		return res;
	}

	void layer_configuration_specific::check_equality(const layer_configuration_specific& other) const
	{
		if (feature_map_count != other.feature_map_count)
			throw neural_network_exception("Feature map count are not equal for layer configurations: " + std::to_string(feature_map_count) + " and " + std::to_string(other.feature_map_count));
		if (get_dimension_count() != other.get_dimension_count())
			throw neural_network_exception("Dimension count are not equal for layer configurations: " + std::to_string(get_dimension_count()) + " and " + std::to_string(other.get_dimension_count()));
		for(size_t i = 0; i < dimension_sizes.size(); ++i)
		{
			if (dimension_sizes[i] != other.dimension_sizes[i])
				throw neural_network_exception("Input configuration sizes of dimension (" + std::to_string(i) + ") are not equal: " + std::to_string(dimension_sizes[i]) + " and " + std::to_string(other.dimension_sizes[i]));
		}
	}

	void layer_configuration_specific::check_equality(unsigned int neuron_count) const
	{
		if (get_neuron_count() != neuron_count)
			throw neural_network_exception("Neuron count are not equal for layer configurations: " + std::to_string(get_neuron_count()) + " and " + std::to_string(neuron_count));
	}

	bool layer_configuration_specific::operator==(const layer_configuration_specific& other) const
	{
		return (feature_map_count == other.feature_map_count) && (dimension_sizes == other.dimension_sizes);
	}

	std::ostream& operator<<(std::ostream& out, const layer_configuration_specific& config)
	{
		out << config.feature_map_count << " fm";
		for(size_t i = 0; i < config.dimension_sizes.size(); ++i)
			out << (i == 0 ? " " : "x") << config.dimension_sizes[i];
		return out;
	}

	// ---- layer_data ------------------------------------------------------------------------

	void layer_data::write(std::ostream& binary_stream_to_write_to) const
	{
		write_pod(binary_stream_to_write_to, static_cast<unsigned int>(size()));
		for(const std::vector<float>& chunk : *this)
		{
			write_pod(binary_stream_to_write_to, static_cast<unsigned int>(chunk.size()));
			if (!chunk.empty())
				binary_stream_to_write_to.write(reinterpret_cast<const char *>(chunk.data()), sizeof(float) * chunk.size());
		}
	}

	void layer_data::read(std::istream& binary_stream_to_read_from)
	{
		unsigned int chunk_count;
		read_pod(binary_stream_to_read_from, chunk_count);
		if (chunk_count > 1024)
			throw neural_network_exception("Implausible weight chunk count " + std::to_string(chunk_count));
		resize(chunk_count);
		for(std::vector<float>& chunk : *this)
		{
			unsigned int weight_count;
			read_pod(binary_stream_to_read_from, weight_count);
			chunk.resize(weight_count);
			if (weight_count > 0)
			{
				binary_stream_to_read_from.read(reinterpret_cast<char *>(chunk.data()), sizeof(float) * weight_count);
				if (!binary_stream_to_read_from)
					throw neural_network_exception("Unexpected end of stream while reading " + std::to_string(weight_count) + " weights");
			}
		}
	}

	void layer_data::fill(float val)
	{
		for(std::vector<float>& chunk : *this)
			std::fill(chunk.begin(), chunk.end(), val);
	}

	// ---- schema_param_block ----------------------------------------------------------------

	float schema_param_block::get_float(const std::string& key, float default_value) const
	{
		std::map<std::string, std::string>::const_iterator it = scalars.find(key);
		if (it == scalars.end())
			return default_value;
		char * end = nullptr;
		const float v = std::strtof(it->second.c_str(), &end);
		if ((end == it->second.c_str()) || (*end != '\0'))
			throw neural_network_exception("Cannot parse \"" + it->second + "\" as a number for " + key);
		return v;
	}

	unsigned int schema_param_block::get_uint(const std::string& key, unsigned int default_value) const
	{
		std::map<std::string, std::string>::const_iterator it = scalars.find(key);
		if (it == scalars.end())
			return default_value;
		char * end = nullptr;
		const unsigned long v = std::strtoul(it->second.c_str(), &end, 10);
		if ((end == it->second.c_str()) || (*end != '\0'))
			throw neural_network_exception("Cannot parse \"" + it->second + "\" as an unsigned integer for " + key);
		return static_cast<unsigned int>(v);
	}

	unsigned int schema_param_block::require_uint(const std::string& key, const std::string& context) const
	{
		if (!has(key))
			throw neural_network_exception("No " + key + " specified for " + context);
		return get_uint(key, 0);
	}

	bool schema_param_block::get_bool(const std::string& key, bool default_value) const
	{
		std::map<std::string, std::string>::const_iterator it = scalars.find(key);
		if (it == scalars.end())
			return default_value;
		if ((it->second == "true") || (it->second == "True") || (it->second == "t") || (it->second == "1"))
			return true;
		if ((it->second == "false") || (it->second == "False") || (it->second == "f") || (it->second == "0"))
			return false;
		throw neural_network_exception("Cannot parse \"" + it->second + "\" as a boolean for " + key);
	}

	std::string schema_param_block::get_string(const std::string& key, const std::string& default_value) const
	{
		std::map<std::string, std::string>::const_iterator it = scalars.find(key);
		return (it == scalars.end()) ? default_value : it->second;
	}

	const schema_param_block * schema_param_block::child(const std::string& name) const
	{
		for(const std::pair<std::string, schema_param_block>& b : blocks)
			if (b.first == name)
				return &b.second;
		return nullptr;
	}

	void schema_param_block::set(const std::string& key, const std::string& value_text)
	{
		if (scalars.find(key) == scalars.end())
			scalar_order.push_back(key);
		scalars[key] = value_text;
	}

	schema_param_block& schema_param_block::add_block(const std::string& name)
	{
		blocks.push_back(std::make_pair(name, schema_param_block()));
		return blocks.back().second;
	}

	std::vector<const schema_param_block *> schema_param_block::children(const std::string& name) const
	{
		std::vector<const schema_param_block *> res;
		for(const std::pair<std::string, schema_param_block>& b : blocks)
			if (b.first == name)
				res.push_back(&b.second);
		return res;
	}

	// ---- layer -----------------------------------------------------------------------------

	// ---- tiling_factor (nnforge/tiling_factor.cpp:24-140) --------------------------------------

	tiling_factor::tiling_factor(unsigned int f, bool b_multiply)
		: f(f), b_multiply(b_multiply || (f == 1))
	{
	}

	tiling_factor::operator unsigned int() const
	{
		if (!b_multiply)
			throw neural_network_exception("Cannot convert tiling_factor " + str() + " to unsigned int");
		return f;
	}

	std::string tiling_factor::str() const
	{
		return b_multiply ? std::to_string(f) : ("1/" + std::to_string(f));
	}

	tiling_factor tiling_factor::get_inverse() const
	{
		return tiling_factor(f, !b_multiply);
	}

	tiling_factor& tiling_factor::operator *=(const tiling_factor& other)
	{
		if (b_multiply == other.b_multiply)
			f *= other.f;
		else if ((f >= other.f) && (f % other.f == 0))
			f /= other.f;
		else if ((f < other.f) && (other.f % f == 0))
		{
			f = other.f / f;
			b_multiply = !b_multiply;
		}
		else
			throw neural_network_exception("Cannot multiply tiling factor " + str() + " and " + other.str() + " ");
		if (f == 1)
			b_multiply = true;
		return *this;
	}

	tiling_factor operator *(const tiling_factor& t1, const tiling_factor& t2)
	{
		tiling_factor res = t1;
		res *= t2;
		return res;
	}

	bool operator ==(const tiling_factor& t1, const tiling_factor& t2)
	{
		return (t1.f == t2.f) && (t1.b_multiply == t2.b_multiply);
	}

	bool operator !=(const tiling_factor& t1, const tiling_factor& t2)
	{
		return !(t1 == t2);
	}

	layer_configuration_specific layer::get_output_layer_configuration_specific(
		const std::vector<layer_configuration_specific>& input_configuration_specific_list) const
	{
		if (input_configuration_specific_list.empty())
			throw neural_network_exception("Layer " + instance_name + " has no input configuration");
		return input_configuration_specific_list.front();
	}

	void layer::read_proto(const void *)
	{
	}

	void layer::write_proto(void *) const
	{
	}

	layer_data::ptr layer::create_layer_data() const
	{
		layer_data::ptr res(new layer_data());
		const data_config dc = get_data_config();
		res->resize(dc.size());
		for(size_t i = 0; i < dc.size(); ++i)
			(*res)[i].resize(dc[i], 0.0F);
		return res;
	}

	layer_data_custom::ptr layer::create_layer_data_custom() const
	{
		layer_data_custom::ptr res(new layer_data_custom());
		const data_custom_config dc = get_data_custom_config();
		res->resize(dc.size());
		for(size_t i = 0; i < dc.size(); ++i)
			(*res)[i].resize(dc[i], -1);
		return res;
	}

	void layer::check_layer_data_consistency(const layer_data& data) const
	{
		const data_config dc = get_data_config();
		if (dc.size() != data.size())
			throw neural_network_exception("data weight vector count " + std::to_string(data.size()) + " doesn't satisfy layer configuration " + std::to_string(dc.size()));
		for(size_t i = 0; i < dc.size(); ++i)
		{
			if (dc[i] != data[i].size())
				throw neural_network_exception("data weight count " + std::to_string(data[i].size()) + " for vector " + std::to_string(i) + " doesn't satisfy layer configuration " + std::to_string(dc[i]));
		}
	}

	void layer::check_layer_data_custom_consistency(const layer_data_custom& data_custom) const
	{
		const data_custom_config dc = get_data_custom_config();
		if (dc.size() != data_custom.size())
			throw neural_network_exception("custom data weight vector count " + std::to_string(data_custom.size()) + " doesn't satisfy layer configuration " + std::to_string(dc.size()));
		for(size_t i = 0; i < dc.size(); ++i)
		{
			if (dc[i] != data_custom[i].size())
				throw neural_network_exception("custom data weight count " + std::to_string(data_custom[i].size()) + " for vector " + std::to_string(i) + " doesn't satisfy layer configuration " + std::to_string(dc[i]));
		}
	}

	void layer::initialize_data(layer_data&) const
	{
	}

	// ---- layer_factory ---------------------------------------------------------------------

	bool layer_factory::register_layer(layer::const_ptr sample_layer)
	{
		return sample_name_layer_map.insert(std::make_pair(sample_layer->get_type_name(), sample_layer)).second;
	}

	bool layer_factory::unregister_layer(const std::string& layer_type_name)
	{
		return sample_name_layer_map.erase(layer_type_name) == 1;
	}

	bool layer_factory::is_registered(const std::string& layer_type_name) const
	{
		return sample_name_layer_map.find(layer_type_name) != sample_name_layer_map.end();
	}

	layer::ptr layer_factory::create_layer(const std::string& layer_type_name) const
	{
		std::map<std::string, layer::const_ptr>::const_iterator it = sample_name_layer_map.find(layer_type_name);
		if (it == sample_name_layer_map.end())
			throw neural_network_exception("No layer is registered with type " + layer_type_name);
		return it->second->clone();
	}

	layer_factory& layer_factory::get_singleton()
	{
		static layer_factory instance;
		return instance;
	}

	void init()
	{
		layer_factory& f = layer_factory::get_singleton();
		f.register_layer(layer::ptr(new data_layer()));
		f.register_layer(layer::ptr(new batch_norm_layer(1)));
		f.register_layer(layer::ptr(new rectified_linear_layer()));
		f.register_layer(layer::ptr(new parametric_rectified_linear_layer(1)));
		f.register_layer(layer::ptr(new exponential_linear_layer()));
		f.register_layer(layer::ptr(new sigmoid_layer()));
		f.register_layer(layer::ptr(new hyperbolic_tangent_layer()));
		f.register_layer(layer::ptr(new add_layer()));
		f.register_layer(layer::ptr(new softmax_layer()));
		f.register_layer(layer::ptr(new average_subsampling_layer(std::vector<unsigned int>(1, 1))));
		f.register_layer(layer::ptr(new absolute_layer()));
		f.register_layer(layer::ptr(new dropout_layer()));
		f.register_layer(layer::ptr(new concat_layer()));
		f.register_layer(layer::ptr(new maxout_layer(2)));
		f.register_layer(layer::ptr(new max_subsampling_layer(std::vector<unsigned int>(1, 1))));
	}
}
