// Data sets on disk and in memory, either side of forward_propagation::run: the ".dt" files the toolset reads
// its inputs from and dumps its outputs to, and the containers run_inference collects the outputs in.
#pragma once

#include "propagation.h"

#include <istream>
#include <memory>
#include <mutex>
#include <ostream>

namespace nnforge
{
	// One tensor per entry (nnforge/structured_data_reader.h:24-48).
	class structured_data_reader
	{
	public:
		typedef std::shared_ptr<structured_data_reader> ptr;
		virtual ~structured_data_reader() = default;
		// false when there is no such entry
		virtual bool read(unsigned int entry_id, float * data) = 0;
		virtual layer_configuration_specific get_configuration() const = 0;
		virtual int get_entry_count() const = 0; // -1: unknown

	protected:
		structured_data_reader() = default;
	};

	// nnforge/structured_data_writer.h:27-52
	class structured_data_writer
	{
	public:
		typedef std::shared_ptr<structured_data_writer> ptr;
		virtual ~structured_data_writer() = default;
		virtual void write(unsigned int entry_id, const float * neurons) = 0;

	protected:
		structured_data_writer() = default;
	};

	// The .dt file: 16 bytes {2C62E05A-C621-43B2-A82C-85CD585815D9}, the layer configuration (u32 feature maps, u32
	// dimension count, u32 per dimension), u32 entry count, then the entries, fp32, one after the other
	// (nnforge/structured_data_stream_reader.cpp:28-61, structured_data_stream_schema.cpp:21-27). Entries are
	// read by position, in any order, from several threads.
	class structured_data_stream_reader : public structured_data_reader
	{
	public:
		// switches the stream to throwing on failure
		explicit structured_data_stream_reader(std::shared_ptr<std::istream> input_stream);
		bool read(unsigned int entry_id, float * data) override;
		layer_configuration_specific get_configuration() const override { return input_configuration; }
		int get_entry_count() const override { return static_cast<int>(entry_count); }

		static const unsigned char guid[16];

	private:
		std::shared_ptr<std::istream> in_stream;
		layer_configuration_specific input_configuration;
		unsigned int input_neuron_count;
		unsigned int entry_count;
		std::istream::pos_type first_entry_pos;
		std::mutex stream_mutex;
	};

	// Writes the same file; entries must arrive in order. The entry count in the header is filled in when the
	// writer is destroyed (nnforge/structured_data_stream_writer.cpp:26-66).
	class structured_data_stream_writer : public structured_data_writer
	{
	public:
		structured_data_stream_writer(std::shared_ptr<std::ostream> output_stream, const layer_configuration_specific& config);
		~structured_data_stream_writer() override;
		void write(const float * neurons);
		void write(unsigned int entry_id, const float * neurons) override;

	private:
		std::shared_ptr<std::ostream> out_stream;
		unsigned int neuron_count;
		unsigned int entry_count;
		std::ostream::pos_type entry_count_pos;
	};

	// The same value everywhere (nnforge/structured_data_constant_reader.cpp:25-55); the toolset feeds the
	// "dataset_value" data layer with it.
	class structured_data_constant_reader : public structured_data_reader
	{
	public:
		structured_data_constant_reader(float val, const layer_configuration_specific& config, int entry_count = -1);
		bool read(unsigned int entry_id, float * data) override;
		layer_configuration_specific get_configuration() const override { return config; }
		int get_entry_count() const override { return entry_count; }

	private:
		float val;
		layer_configuration_specific config;
		int entry_count;
	};

	// A reader per data layer behind the bunch interface forward_propagation::run takes
	// (nnforge/structured_data_bunch_stream_reader.cpp:27-160). The readers must agree on the entry count (those
	// that know it). multiple_epoch_count > 1 cuts the data into that many parts, set_epoch() chooses one.
	// Shuffling of blocks belongs to training and is refused.
	class structured_data_bunch_stream_reader : public structured_data_bunch_reader
	{
	public:
		structured_data_bunch_stream_reader(
			const std::map<std::string, structured_data_reader::ptr>& data_reader_map,
			unsigned int multiple_epoch_count = 1,
			unsigned int shuffle_block_size = 0);
		std::map<std::string, layer_configuration_specific> get_config_map() const override;
		bool read(unsigned int entry_id, const std::map<std::string, float *>& data_map) override;
		void set_epoch(unsigned int epoch_id) override;
		int get_entry_count() const override;
		// the same data, only the given layers
		structured_data_bunch_reader::ptr get_narrow_reader(const std::set<std::string>& layer_names) const;

	private:
		std::map<std::string, structured_data_reader::ptr> data_reader_map;
		int total_entry_count;
		std::vector<int> entry_count_list;           // per part
		std::vector<unsigned int> base_entry_count_list;
		unsigned int current_epoch;
		unsigned int current_chunk;
		std::string invalid_config_message;          // thrown by read(), as the reference defers it
	};

	// Entries of one layer kept in memory (nnforge/neuron_value_set.h:26-68; the constructors that merge several
	// sets are the toolset's ensemble code and are not here).
	class neuron_value_set
	{
	public:
		typedef std::shared_ptr<neuron_value_set> ptr;
		typedef std::shared_ptr<const neuron_value_set> const_ptr;

		explicit neuron_value_set(unsigned int neuron_count);
		neuron_value_set(unsigned int neuron_count, unsigned int entry_count);

		void add_entry(const float * new_data);
		void set_entry(unsigned int entry_id, const float * new_data);
		// per neuron, over the entries, accumulated in double
		std::shared_ptr<std::vector<double> > get_average() const;
		// this = alpha * this + beta * other
		void add(const neuron_value_set& other, float alpha, float beta);
		// replaces every sample_count consecutive entries by their mean: folds the entries a tiling layer made of
		// each input entry (nnforge/neuron_value_set.cpp:174-197)
		void compact(unsigned int sample_count);

		unsigned int neuron_count;
		std::vector<std::shared_ptr<std::vector<float> > > neuron_value_list;
	};

	// Collects everything forward_propagation::run writes (nnforge/neuron_value_set_data_bunch_writer.cpp:21-39).
	class neuron_value_set_data_bunch_writer : public structured_data_bunch_writer
	{
	public:
		void set_config_map(const std::map<std::string, layer_configuration_specific> config_map) override;
		void write(unsigned int entry_id, const std::map<std::string, const float *>& data_map) override;

		std::map<std::string, std::pair<layer_configuration_specific, neuron_value_set::ptr> > layer_name_to_config_and_value_set_map;
	};
}
