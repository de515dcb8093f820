#include "nnforge_hip/data_streams.h"

#include <algorithm>
#include <cstdio>
#include <cstring>

namespace nnforge
{
	const unsigned char structured_data_stream_reader::guid[16] =
		{ 0x2c, 0x62, 0xe0, 0x5a, 0xc6, 0x21, 0x43, 0xb2, 0xa8, 0x2c, 0x85, 0xcd, 0x58, 0x58, 0x15, 0xd9 };

	namespace
	{
		std::string guid_text(const unsigned char * g)
		{
			char buf[40];
			std::snprintf(buf, sizeof(buf), "%02x%02x%02x%02x-%02x%02x-%02x%02x-%02x%02x-%02x%02x%02x%02x%02x%02x",
				g[0], g[1], g[2], g[3], g[4], g[5], g[6], g[7], g[8], g[9], g[10], g[11], g[12], g[13], g[14], g[15]);
			return buf;
		}
	}

	// ---- .dt reader ---------------------------------------------------------------------------

	structured_data_stream_reader::structured_data_stream_reader(std::shared_ptr<std::istream> input_stream)
		: in_stream(input_stream)
		, input_neuron_count(0)
		, entry_count(0)
	{
		if (!in_stream || !*in_stream)
			throw neural_network_exception("Cannot read structured data: the stream is not open");
		in_stream->exceptions(std::ios::eofbit | std::ios::failbit | std::ios::badbit);
		try
		{
			unsigned char guid_read[16];
			in_stream->read(reinterpret_cast<char *>(guid_read), sizeof(guid_read));
			if (std::memcmp(guid_read, guid, sizeof(guid)) != 0)
				throw neural_network_exception("Unknown structured data GUID encountered in input stream: " + guid_text(guid_read));
			input_configuration.read(*in_stream);
			input_neuron_count = input_configuration.get_neuron_count();
			in_stream->read(reinterpret_cast<char *>(&entry_count), sizeof(entry_count));
			first_entry_pos = in_stream->tellg();
		}
		catch (const std::ios_base::failure&)
		{
			throw neural_network_exception("Structured data stream ends inside its header");
		}
	}

	bool structured_data_stream_reader::read(unsigned int entry_id, float * data)
	{
		if (entry_id >= entry_count)
			return false;
		const std::istream::off_type entry_bytes = static_cast<std::istream::off_type>(sizeof(float)) * input_neuron_count;
		std::lock_guard<std::mutex> lock(stream_mutex);
		try
		{
			in_stream->seekg(first_entry_pos + static_cast<std::istream::off_type>(entry_id) * entry_bytes, std::ios::beg);
			in_stream->read(reinterpret_cast<char *>(data), entry_bytes);
		}
		catch (const std::ios_base::failure&)
		{
			in_stream->clear();
			throw neural_network_exception("Structured data stream holds fewer than the " + std::to_string(entry_count) + " entries its header announces: entry "
				+ std::to_string(entry_id) + " cannot be read");
		}
		return true;
	}

	// ---- .dt writer ---------------------------------------------------------------------------

	structured_data_stream_writer::structured_data_stream_writer(std::shared_ptr<std::ostream> output_stream, const layer_configuration_specific& config)
		: out_stream(output_stream)
		, neuron_count(config.get_neuron_count())
		, entry_count(0)
	{
		if (!out_stream || !*out_stream)
			throw neural_network_exception("Cannot write structured data: the stream is not open");
		out_stream->exceptions(std::ios::failbit | std::ios::badbit);
		out_stream->write(reinterpret_cast<const char *>(structured_data_stream_reader::guid), sizeof(structured_data_stream_reader::guid));
		config.write(*out_stream);
		entry_count_pos = out_stream->tellp();
		out_stream->write(reinterpret_cast<const char *>(&entry_count), sizeof(entry_count));
	}

	structured_data_stream_writer::~structured_data_stream_writer()
	{
		try
		{
			out_stream->seekp(entry_count_pos);
			out_stream->write(reinterpret_cast<const char *>(&entry_count), sizeof(entry_count));
			out_stream->seekp(0, std::ios::end);
			out_stream->flush();
		}
		catch (...)
		{
			// a destructor has nobody to tell: the file keeps an entry count of 0 and reads back as empty
		}
	}

	void structured_data_stream_writer::write(const float * neurons)
	{
		out_stream->write(reinterpret_cast<const char *>(neurons), sizeof(float) * neuron_count);
		++entry_count;
	}

	void structured_data_stream_writer::write(unsigned int entry_id, const float * neurons)
	{
		if (entry_id != entry_count)
			throw neural_network_exception("structured_data_stream_writer cannot write entry " + std::to_string(entry_id) + " when " + std::to_string(entry_count) + " written already");
		write(neurons);
	}

	// ---- constant reader ------------------------------------------------------------------------

	structured_data_constant_reader::structured_data_constant_reader(float val, const layer_configuration_specific& config, int entry_count)
		: val(val), config(config), entry_count(entry_count)
	{
	}

	bool structured_data_constant_reader::read(unsigned int entry_id, float * data)
	{
		if ((entry_count >= 0) && (entry_id >= static_cast<unsigned int>(entry_count)))
			return false;
		std::fill_n(data, config.get_neuron_count(), val);
		return true;
	}

	// ---- bunch of readers -----------------------------------------------------------------------

	structured_data_bunch_stream_reader::structured_data_bunch_stream_reader(
		const std::map<std::string, structured_data_reader::ptr>& data_reader_map,
		unsigned int multiple_epoch_count,
		unsigned int shuffle_block_size)
		: data_reader_map(data_reader_map)
		, total_entry_count(-1)
		, entry_count_list(std::max(1u, multiple_epoch_count), -1)
		, base_entry_count_list(std::max(1u, multiple_epoch_count), 0)
		, current_epoch(0)
		, current_chunk(0)
	{
		if (multiple_epoch_count == 0)
			throw neural_network_exception("structured_data_bunch_stream_reader: multiple_epoch_count cannot be 0");
		if (shuffle_block_size > 0)
			throw neural_network_exception("structured_data_bunch_stream_reader: shuffling blocks of entries is for training, which this backend does not do");
		for(const std::pair<const std::string, structured_data_reader::ptr>& r : data_reader_map)
		{
			const int count = r.second->get_entry_count();
			if (count < 0)
				continue;
			if (total_entry_count < 0)
				total_entry_count = count;
			else if (total_entry_count != count)
			{
				invalid_config_message = "Entry count mismatch: " + std::to_string(total_entry_count) + " and " + std::to_string(count);
				return;
			}
		}
		if (multiple_epoch_count == 1)
		{
			entry_count_list[0] = total_entry_count;
			return;
		}
		if (total_entry_count < 0)
		{
			invalid_config_message = "Multiple epoch count specified for structured_data_bunch_stream_reader while entry count cannot be determined";
			return;
		}
		// the first (total % parts) parts hold one entry more
		const unsigned int part = static_cast<unsigned int>(total_entry_count) / multiple_epoch_count;
		const unsigned int longer = static_cast<unsigned int>(total_entry_count) % multiple_epoch_count;
		for(unsigned int i = 0; i < multiple_epoch_count; ++i)
		{
			entry_count_list[i] = static_cast<int>(part + ((i < longer) ? 1 : 0));
			if (i > 0)
				base_entry_count_list[i] = base_entry_count_list[i - 1] + static_cast<unsigned int>(entry_count_list[i - 1]);
		}
	}

	structured_data_bunch_reader::ptr structured_data_bunch_stream_reader::get_narrow_reader(const std::set<std::string>& layer_names) const
	{
		std::map<std::string, structured_data_reader::ptr> narrow;
		for(const std::pair<const std::string, structured_data_reader::ptr>& r : data_reader_map)
			if (layer_names.find(r.first) != layer_names.end())
				narrow.insert(r);
		std::shared_ptr<structured_data_bunch_stream_reader> res(new structured_data_bunch_stream_reader(narrow, static_cast<unsigned int>(entry_count_list.size()), 0));
		res->set_epoch(current_epoch);
		return res;
	}

	std::map<std::string, layer_configuration_specific> structured_data_bunch_stream_reader::get_config_map() const
	{
		std::map<std::string, layer_configuration_specific> res;
		for(const std::pair<const std::string, structured_data_reader::ptr>& r : data_reader_map)
			res[r.first] = r.second->get_configuration();
		return res;
	}

	void structured_data_bunch_stream_reader::set_epoch(unsigned int epoch_id)
	{
		current_epoch = epoch_id;
		current_chunk = epoch_id % static_cast<unsigned int>(entry_count_list.size());
	}

	bool structured_data_bunch_stream_reader::read(unsigned int entry_id, const std::map<std::string, float *>& data_map)
	{
		if (!invalid_config_message.empty())
			throw neural_network_exception(invalid_config_message);
		if ((entry_count_list[current_chunk] >= 0) && (entry_id >= static_cast<unsigned int>(entry_count_list[current_chunk])))
			return false;
		const unsigned int global_entry_id = entry_id + base_entry_count_list[current_chunk];
		bool res = true;
		for(const std::pair<const std::string, float *>& dst : data_map)
		{
			std::map<std::string, structured_data_reader::ptr>::const_iterator r = data_reader_map.find(dst.first);
			if (r == data_reader_map.end())
				throw neural_network_exception("structured_data_bunch_stream_reader is requested to read " + dst.first + " data, while it doesn't have it");
			res = r->second->read(global_entry_id, dst.second) && res;
		}
		return res;
	}

	int structured_data_bunch_stream_reader::get_entry_count() const
	{
		return entry_count_list[current_chunk];
	}

	// ---- values in memory -------------------------------------------------------------------------

	neuron_value_set::neuron_value_set(unsigned int neuron_count)
		: neuron_count(neuron_count)
	{
	}

	neuron_value_set::neuron_value_set(unsigned int neuron_count, unsigned int entry_count)
		: neuron_count(neuron_count)
	{
		for(unsigned int i = 0; i < entry_count; ++i)
			neuron_value_list.push_back(std::make_shared<std::vector<float> >(neuron_count));
	}

	void neuron_value_set::add_entry(const float * new_data)
	{
		neuron_value_list.push_back(std::make_shared<std::vector<float> >(new_data, new_data + neuron_count));
	}

	void neuron_value_set::set_entry(unsigned int entry_id, const float * new_data)
	{
		// entries may arrive in any order: every slot up to this one exists afterwards (zeros until written)
		while (neuron_value_list.size() <= entry_id)
			neuron_value_list.push_back(std::make_shared<std::vector<float> >(neuron_count));
		std::copy(new_data, new_data + neuron_count, neuron_value_list[entry_id]->begin());
	}

	std::shared_ptr<std::vector<double> > neuron_value_set::get_average() const
	{
		std::shared_ptr<std::vector<double> > res(new std::vector<double>(neuron_count, 0.0));
		for(const std::shared_ptr<std::vector<float> >& entry : neuron_value_list)
			for(unsigned int i = 0; i < neuron_count; ++i)
				(*res)[i] += static_cast<double>((*entry)[i]);
		const double mult = 1.0 / static_cast<double>(neuron_value_list.size());
		for(double& v : *res)
			v *= mult;
		return res;
	}

	void neuron_value_set::add(const neuron_value_set& other, float alpha, float beta)
	{
		if ((other.neuron_count != neuron_count) || (other.neuron_value_list.size() < neuron_value_list.size()))
			throw neural_network_exception("neuron_value_set::add: the sets differ in size");
		for(size_t entry_id = 0; entry_id < neuron_value_list.size(); ++entry_id)
		{
			const std::vector<float>& src = *other.neuron_value_list[entry_id];
			std::vector<float>& dst = *neuron_value_list[entry_id];
			for(unsigned int i = 0; i < neuron_count; ++i)
				dst[i] = alpha * dst[i] + beta * src[i];
		}
	}

	void neuron_value_set::compact(unsigned int sample_count)
	{
		if (sample_count == 1)
			return;
		if ((sample_count == 0) || (neuron_value_list.size() % sample_count != 0))
			throw neural_network_exception("neuron_value_set::compact cannot operate on " + std::to_string(neuron_value_list.size())
				+ " entries no evenly divisible by sample count " + std::to_string(sample_count));
		const size_t new_entry_count = neuron_value_list.size() / sample_count;
		const float mult = 1.0F / static_cast<float>(sample_count);
		for(size_t dst_entry_id = 0; dst_entry_id < new_entry_count; ++dst_entry_id)
		{
			// entry dst_entry_id is overwritten only after it has been read: it is the first of its own group or lies before it
			std::vector<float>& dst = *neuron_value_list[dst_entry_id];
			for(unsigned int i = 0; i < neuron_count; ++i)
			{
				float sum = 0.0F;
				for(unsigned int sample_id = 0; sample_id < sample_count; ++sample_id)
					sum += (*neuron_value_list[dst_entry_id * sample_count + sample_id])[i];
				dst[i] = mult * sum;
			}
		}
		neuron_value_list.resize(new_entry_count);
	}

	// ---- writer into memory ---------------------------------------------------------------------

	void neuron_value_set_data_bunch_writer::set_config_map(const std::map<std::string, layer_configuration_specific> config_map)
	{
		layer_name_to_config_and_value_set_map.clear();
		for(const std::pair<const std::string, layer_configuration_specific>& c : config_map)
			layer_name_to_config_and_value_set_map[c.first] = std::make_pair(c.second, neuron_value_set::ptr(new neuron_value_set(c.second.get_neuron_count())));
	}

	void neuron_value_set_data_bunch_writer::write(unsigned int entry_id, const std::map<std::string, const float *>& data_map)
	{
		for(const std::pair<const std::string, const float *>& src : data_map)
		{
			std::map<std::string, std::pair<layer_configuration_specific, neuron_value_set::ptr> >::iterator it = layer_name_to_config_and_value_set_map.find(src.first);
			if (it == layer_name_to_config_and_value_set_map.end())
				throw neural_network_exception("neuron_value_set_data_bunch_writer has no configuration for layer " + src.first);
			it->second.second->set_entry(entry_id, src.second);
		}
	}
}
