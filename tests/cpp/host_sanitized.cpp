// Host-side code of the backend (schema reader and writer, layer configuration rules, launch and
// buffer planner, weight files) driven through the C bridge without a device. The tests build this
// program together with the backend's sources under AddressSanitizer and UndefinedBehaviorSanitizer:
// it feeds the reader well-formed and damaged text and must end with "ok" and no sanitizer report.
#include <nnforge_hip_backend.h>
#include <nnforge_hip/propagation.h>

#include <atomic>
#include <cstdio>
#include <cstddef>
#include <cstring>
#include <map>
#include <set>
#include <sstream>
#include <string>
#include <vector>

namespace
{
	const char * good_schema = R"(
name: "host_checks"
layer { type: "Data" name: "conv1" }
layer { type: "BatchNorm" name: "bn" input_layer_name: "conv1" batch_norm_param { feature_map_count: 8 } }
layer { type: "ReLU" name: "relu" input_layer_name: "bn" relu_param { negative_slope: 0.1 } }
layer { type: "MaxSubsampling" name: "pool1" input_layer_name: "relu"
	max_subsampling_param { dimension_param { subsampling_size: 3 stride: 2 round_up: true } dimension_param { subsampling_size: 3 stride: 2 round_up: true } } }
layer { type: "TanH" name: "tanh" input_layer_name: "pool1" tanh_param { scale: 1.7159 steepness: 0.6666 } }
layer { type: "Absolute" name: "abs" input_layer_name: "tanh" }
layer { type: "MaxSubsampling" name: "tiles" input_layer_name: "abs"
	max_subsampling_param { tiling: true dimension_param { subsampling_size: 2 } dimension_param { subsampling_size: 2 } } }
layer { type: "AverageSubsampling" name: "untile" input_layer_name: "tiles"
	average_subsampling_param { dimension_param { subsampling_size: 1 } dimension_param { subsampling_size: 1 } entry_param { subsampling_size: 4 } } }
layer { type: "AverageSubsampling" name: "pool2" input_layer_name: "untile"
	average_subsampling_param { dimension_param { subsampling_size: 2 } dimension_param { subsampling_size: 2 } } }
layer { type: "PReLU" name: "prelu" input_layer_name: "pool2" prelu_param { feature_map_count: 8 } }
layer { type: "Dropout" name: "drop" input_layer_name: "prelu" dropout_param { dropout_rate: 0.25 } }
layer { type: "Add" name: "sum" input_layer_name: "drop" input_layer_name: "pool2" add_param { alpha: 0.5 } }
layer { type: "Concat" name: "cat" input_layer_name: "sum" input_layer_name: "pool2" }
layer { type: "Maxout" name: "mo" input_layer_name: "cat" maxout_param { feature_map_subsampling_size: 2 } }
layer { type: "ELU" name: "elu" input_layer_name: "mo" }
layer { type: "Sigmoid" name: "sig" input_layer_name: "elu" }
layer { type: "Softmax" name: "prob" input_layer_name: "sig" }
)";

	int failures = 0;

	void expect(bool condition, const std::string& what)
	{
		if (!condition)
		{
			std::printf("FAILED: %s\n", what.c_str());
			++failures;
		}
	}

	int plan(const std::string& text, uint32_t width, uint32_t height, std::string& report, int fuse = 1)
	{
		const uint32_t dims[2] = { width, height };
		nnf_backend_input input = { "conv1", 8, 2, dims, nullptr };
		const char * outputs[1] = { "prob" };
		nnf_backend_options options;
		std::memset(&options, 0, sizeof(options));
		options.struct_size = sizeof(options);
		options.fuse = fuse;
		std::vector<char> buffer(1 << 16);
		const int rc = nnf_backend_plan_schema(text.c_str(), &input, 1, outputs, 1, &options, 1ull << 30, buffer.data(), buffer.size());
		report = buffer.data();
		return rc;
	}
}

int main(int argc, char ** argv)
{
	const std::string folder = (argc > 1) ? argv[1] : ".";
	const std::string good(good_schema);
	std::string report;

	// the whole schema plans, with and without fusion, at several input sizes
	for(uint32_t size : { 28u, 57u, 112u })
	{
		expect(plan(good, size, size, report, 1) == 0, "plan with fusion: " + report);
		expect(report.find("bn+relu+pool1") != std::string::npos, "the pooling layer takes the group in front of it along: " + report);
		expect(plan(good, size, size, report, 0) == 0, "plan without fusion: " + report);
	}
	// options without their size are refused; options of an older, shorter header are taken with the later members at their defaults
	{
		const uint32_t dims[2] = { 28, 28 };
		nnf_backend_input input = { "conv1", 8, 2, dims, nullptr };
		const char * outputs[1] = { "prob" };
		std::vector<char> buffer(1 << 16);
		nnf_backend_options options;
		std::memset(&options, 0xFF, sizeof(options)); // whatever lies behind a shorter structure must not be read
		options.struct_size = 0;
		expect(nnf_backend_plan_schema(good.c_str(), &input, 1, outputs, 1, &options, 1ull << 30, buffer.data(), buffer.size()) != 0, "options with struct_size 0 are refused");
		expect(std::string(buffer.data()).find("struct_size") != std::string::npos, std::string("the refusal names struct_size: ") + buffer.data());
		options.struct_size = offsetof(nnf_backend_options, max_entry_count) + sizeof(options.max_entry_count);
		options.fuse = 1;
		options.dont_share_buffers = 0;
		options.max_entry_count = 7;
		expect(nnf_backend_plan_schema(good.c_str(), &input, 1, outputs, 1, &options, 1ull << 30, buffer.data(), buffer.size()) == 0, std::string("options of a shorter header: ") + buffer.data());
		expect(std::string(buffer.data()).find("max_entry_count: 7") != std::string::npos, std::string("... are honoured as far as they go: ") + buffer.data());
		expect(std::string(buffer.data()).find(" #") != std::string::npos, std::string("... and the members behind them take their defaults (groups launched together): ") + buffer.data());
	}
	// what a subclass of the reference's base classes may touch: the action schema of a forward_propagation, every kind of
	// option list of a factory_generator
	{
		struct probe : public nnforge::forward_propagation
		{
			probe(const nnforge::network_schema& schema, const std::vector<std::string>& outputs)
				: nnforge::forward_propagation(schema, outputs, nnforge::debug_state::ptr(), nnforge::profile_state::ptr()) {}
			void actual_set_data(nnforge::network_data::const_ptr) override {}
			void actual_clear_data() override {}
			void actual_run(nnforge::structured_data_bunch_reader&, nnforge::structured_data_bunch_writer&, unsigned int&,
				std::map<nnforge::layer_name_with_action, float>&, float&) override {}
			void layer_config_map_modified() override {}
			const nnforge::network_action_schema& actions() const { return *action_schema; }
		};
		nnforge::init();
		std::istringstream in(good);
		nnforge::network_schema schema;
		schema.read_proto(in);
		probe fp(schema, std::vector<std::string>(1, "cat"));
		const nnforge::layer_action forward(nnforge::layer_action::forward);
		const std::vector<nnforge::layer_name_with_action> order = fp.actions().get_actions_in_execution_order();
		expect(order.size() == 12, "a forward action for each of the twelve layers between the data layer and cat, none for what cat does not need: " + std::to_string(order.size()));
		expect(!fp.actions().action_exists(nnforge::layer_name_with_action("conv1", forward)), "a data layer has no action");
		expect(!fp.actions().action_exists(nnforge::layer_name_with_action("prob", forward)), "a layer the outputs do not need has no action");
		expect(fp.actions().get_dependencies(nnforge::layer_name_with_action("bn", forward)).empty(), "the first layer waits for nothing");
		const std::vector<nnforge::layer_name_with_action> of_sum = fp.actions().get_dependencies(nnforge::layer_name_with_action("sum", forward));
		expect((of_sum.size() == 2) && (of_sum[0].get_name() == "drop") && (of_sum[1].get_name() == "pool2"), "the Add waits for both layers it reads");
		expect(fp.actions().dependency_exists(nnforge::layer_name_with_action("cat", forward), nnforge::layer_name_with_action("pool2", forward)), "cat waits for pool2");
		std::map<std::string, size_t> position;
		for(size_t i = 0; i < order.size(); ++i)
			position[order[i].get_name()] = i;
		bool ordered = true;
		for(const nnforge::layer_name_with_action& a : order)
			for(const nnforge::layer_name_with_action& d : fp.actions().get_dependencies(a))
				ordered = ordered && (position[d.get_name()] < position[a.get_name()]);
		expect(ordered, "execution order puts every action behind what it waits for");
		nnforge::network_action_schema copy(fp.actions());
		copy.drop_actions_not_required_to_do(std::set<nnforge::layer_name_with_action>{ nnforge::layer_name_with_action("abs", forward) });
		expect(copy.get_actions().size() == 5, "bn, relu, pool1, tanh, abs are what abs needs: " + std::to_string(copy.get_actions().size()));

		struct generator : public nnforge::factory_generator
		{
			void initialize() override {}
			nnforge::forward_propagation_factory::ptr create_forward_propagation_factory() const override { return nnforge::forward_propagation_factory::ptr(); }
			nnforge::backward_propagation_factory::ptr create_backward_propagation_factory() const override { return nnforge::backward_propagation_factory::ptr(); }
			void info() const override {}
			std::vector<nnforge::multi_string_option> get_multi_string_options() override
			{
				return std::vector<nnforge::multi_string_option>(1, nnforge::multi_string_option("device", &devices, "devices to use"));
			}
			std::vector<nnforge::path_option> get_path_options() override
			{
				return std::vector<nnforge::path_option>(1, nnforge::path_option("cache_folder", &cache, "/tmp/cache", "where to keep things"));
			}
			std::vector<std::string> devices = std::vector<std::string>(2, "stale");
			std::string cache = "stale";
		} g;
		expect(static_cast<nnforge::factory_generator&>(g).get_string_options().empty(), "option lists default to empty");
		g.apply_default_options();
		expect(g.devices.empty() && (g.cache == "/tmp/cache"), "defaults reach path options, and options that may repeat start empty");
	}
	// sizes the layers reject
	expect(plan(good, 2, 2, report) != 0, "an input smaller than the windows is refused");
	expect(plan(good, 0, 5, report) != 0, "an empty dimension is refused");

	// the text written back parses again to the same text
	std::vector<char> once(1 << 16), twice(1 << 16);
	expect(nnf_backend_rewrite_schema(good.c_str(), 0, once.data(), once.size()) == 0, "rewrite");
	expect(nnf_backend_rewrite_schema(once.data(), 0, twice.data(), twice.size()) == 0, "rewrite of the rewritten text");
	expect(std::strcmp(once.data(), twice.data()) == 0, "the writer's output is a fixed point of reader + writer");
	// a buffer that is too small is reported, not overrun
	std::vector<char> tiny(16);
	expect(nnf_backend_rewrite_schema(good.c_str(), 0, tiny.data(), tiny.size()) != 0, "a short output buffer is an error");

	// damaged text: every prefix of the schema, single characters replaced, blocks doubled
	int accepted = 0, refused = 0;
	for(size_t cut = 0; cut < good.size(); cut += 7)
		(plan(good.substr(0, cut), 28, 28, report) == 0) ? ++accepted : ++refused;
	const char replacements[] = { '{', '}', '"', ':', '-', '9', 'x', '\0', '#', '\n' };
	for(size_t at = 3; at < good.size(); at += 11)
	{
		for(char c : replacements)
		{
			std::string damaged = good;
			damaged[at] = c;
			(plan(damaged, 28, 28, report) == 0) ? ++accepted : ++refused;
		}
	}
	for(size_t at = 0; at + 40 < good.size(); at += 97)
	{
		std::string doubled = good;
		doubled.insert(at, good.substr(at, 40));
		(plan(doubled, 28, 28, report) == 0) ? ++accepted : ++refused;
	}
	expect(refused > accepted, "most damaged texts are refused (" + std::to_string(refused) + " refused, " + std::to_string(accepted) + " still well-formed)");

	// the job runner: every job posted runs exactly once, on one of its threads, also those still queued when it goes
	{
		constexpr int job_count = 5000;
		std::vector<int> ran(job_count, 0);
		std::atomic<int> total(0);
		{
			nnforge::threadpool_job_runner runner(4);
			expect(runner.thread_count == 4, "thread count as asked");
			for(int i = 0; i < job_count; ++i)
				runner.post([&ran, &total, i]() { ++ran[i]; total.fetch_add(1); });
		}
		bool once_each = true;
		for(int r : ran)
			once_each = once_each && (r == 1);
		expect(once_each && (total.load() == job_count), "every posted job ran exactly once before the runner was gone");
		nnforge::threadpool_job_runner at_least_one(0);
		expect(at_least_one.thread_count == 1, "a runner has at least one thread");
		expect(nnforge::get_available_processor_count() >= 1, "at least one processor");
	}

	// weight files: written, read back, read with wrong expectations
	{
		const std::vector<float> gamma = { 1.0f, 2.0f, 3.0f }, slopes = { 0.25f };
		const uint32_t bn_sizes[4] = { 3, 3, 3, 3 };
		const float * bn_chunks[4] = { gamma.data(), gamma.data(), gamma.data(), gamma.data() };
		const uint32_t prelu_sizes[1] = { 1 };
		const float * prelu_chunks[1] = { slopes.data() };
		nnf_backend_weights weights[2] = { { "bn", 4, bn_sizes, bn_chunks }, { "prelu", 1, prelu_sizes, prelu_chunks } };
		std::vector<char> buffer(4096);
		expect(nnf_backend_write_weights(folder.c_str(), weights, 2, buffer.data(), buffer.size()) == 0, std::string("write weights: ") + buffer.data());
		std::vector<float> back(12, -1.0f);
		float * back_chunks[4] = { back.data(), back.data() + 3, back.data() + 6, back.data() + 9 };
		expect(nnf_backend_read_weights(folder.c_str(), "bn", 4, bn_sizes, back_chunks, buffer.data(), buffer.size()) == 0, std::string("read weights: ") + buffer.data());
		expect((back[0] == 1.0f) && (back[5] == 3.0f) && (back[11] == 3.0f), "the weights read are the weights written");
		const uint32_t wrong_sizes[4] = { 3, 3, 2, 3 };
		expect(nnf_backend_read_weights(folder.c_str(), "bn", 4, wrong_sizes, back_chunks, buffer.data(), buffer.size()) != 0, "a chunk of another size is refused");
		expect(nnf_backend_read_weights(folder.c_str(), "bn", 3, bn_sizes, back_chunks, buffer.data(), buffer.size()) != 0, "another chunk count is refused");
		expect(nnf_backend_read_weights(folder.c_str(), "missing", 1, prelu_sizes, back_chunks, buffer.data(), buffer.size()) != 0, "a layer without a file is refused");
		expect(nnf_backend_read_weights((folder + "/nowhere").c_str(), "bn", 4, bn_sizes, back_chunks, buffer.data(), buffer.size()) != 0, "a missing folder is refused");
	}

	// data set files: a good one, every prefix of it, and headers that announce more than the file holds
	{
		const uint32_t header[5] = { 2, 2, 3, 2, 6 }; // 2 feature maps of 3 x 2, 6 entries
		const unsigned char guid[16] = { 0x2c, 0x62, 0xe0, 0x5a, 0xc6, 0x21, 0x43, 0xb2, 0xa8, 0x2c, 0x85, 0xcd, 0x58, 0x58, 0x15, 0xd9 };
		std::string bytes(reinterpret_cast<const char *>(guid), sizeof(guid));
		bytes.append(reinterpret_cast<const char *>(header), sizeof(header));
		for(int i = 0; i < 6 * 12; ++i)
		{
			const float v = 0.5f * static_cast<float>(i);
			bytes.append(reinterpret_cast<const char *>(&v), sizeof(v));
		}
		const std::string in_path = folder + "/in.dt", out_path = folder + "/out.dt";
		const auto store = [&in_path] (const std::string& content)
		{
			std::FILE * f = std::fopen(in_path.c_str(), "wb");
			std::fwrite(content.data(), 1, content.size(), f);
			std::fclose(f);
		};
		std::vector<char> buffer(1 << 16);
		store(bytes);
		expect(nnf_backend_rewrite_dataset(in_path.c_str(), out_path.c_str(), 1, 1, 0, buffer.data(), buffer.size()) == 0, std::string("rewrite dataset: ") + buffer.data());
		expect(std::string(buffer.data()).find("entries_read: 6 of 6") != std::string::npos, std::string("all entries read: ") + buffer.data());
		expect(nnf_backend_rewrite_dataset(in_path.c_str(), out_path.c_str(), 3, 2, 1, buffer.data(), buffer.size()) == 0, std::string("second half, groups of 3: ") + buffer.data());
		expect(std::string(buffer.data()).find("entries_written: 1") != std::string::npos, std::string("one group written: ") + buffer.data());
		expect(nnf_backend_rewrite_dataset(in_path.c_str(), out_path.c_str(), 4, 1, 0, buffer.data(), buffer.size()) != 0, "6 entries do not fold into groups of 4");
		int cut_refused = 0;
		for(size_t cut = 0; cut < bytes.size(); cut += 3)
		{
			store(bytes.substr(0, cut));
			if (nnf_backend_rewrite_dataset(in_path.c_str(), out_path.c_str(), 1, 1, 0, buffer.data(), buffer.size()) != 0)
				++cut_refused;
		}
		expect(cut_refused == static_cast<int>((bytes.size() + 2) / 3), "every cut data set file is refused");
		std::string huge = bytes;
		const uint32_t many = 0xFFFFFFFFu;
		huge.replace(16 + 4, 4, reinterpret_cast<const char *>(&many), 4); // dimension count
		store(huge);
		expect(nnf_backend_rewrite_dataset(in_path.c_str(), out_path.c_str(), 1, 1, 0, buffer.data(), buffer.size()) != 0, "an implausible dimension count is refused");
	}

	if (failures == 0)
		std::printf("ok\n");
	return failures == 0 ? 0 : 1;
}
