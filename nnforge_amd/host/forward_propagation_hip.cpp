// forward_propagation for one MI355X: plans the launches (fusing runs of element-wise layers),
// plans the device buffers (liveness-based sharing, in-place where a tester allows it), then
// streams packets of entries through the plan.
#include "nnforge_hip/hip_backend.h"

#include <algorithm>
#include <chrono>
#include <condition_variable>
#include <cstring>
#include <exception>
#include <iostream>
#include <mutex>
#include <sstream>

namespace nnforge
{
	namespace hip
	{
		bool get_add_alpha(const layer_tester_hip& tester, float& alpha); // hip_testers.cpp

		std::string forward_step::description() const
		{
			std::string s;
			for(size_t i = 0; i < layer_names.size(); ++i)
				s += (i == 0 ? "" : "+") + layer_names[i];
			s += " <- ";
			for(size_t i = 0; i < input_names.size(); ++i)
				s += (i == 0 ? "" : ", ") + input_names[i];
			return s;
		}

		namespace
		{
			// one input tensor of a group under construction and the layers applied to it before the join
			struct pending_arm
			{
				std::string source;
				std::vector<std::string> ops;
			};

			// a group of element-wise layers whose result has not been written to memory yet
			struct pending_group
			{
				std::vector<pending_arm> arms;
				std::string add_layer_name; // empty: no join
				std::vector<std::string> tail;

				size_t op_count() const
				{
					size_t n = tail.size();
					for(const pending_arm& a : arms)
						n += a.ops.size();
					return n;
				}
			};

			struct step_plan
			{
				forward_step info;
				std::string key;                     // layer names joined with '+': what reports show for the step
				layer_name_with_action action;       // the step's key in the per-action tables: its last layer, forward
				layer_tester_hip::ptr tester;        // single-layer steps
				nnf_hip_chain_desc desc;             // fused steps (entry_count filled per packet)
				std::vector<std::string> chunk_layers; // fused steps: layers whose weight chunks are concatenated into chunk_ptrs
				int output_buffer;
				std::vector<int> input_buffers;
				bool passes_input_on = false;        // every layer of the step is a Dropout
				bool prologue = false;               // desc holds element-wise layers that the tester (a subsampling layer) applies to its input
				// a fused group that writes into the output of the Concat layer behind it: where its feature maps start inside
				// an entry of that output, and how long such an entry is (floats); stride 0: an ordinary step
				uint32_t view_offset = 0, view_stride = 0;
				std::vector<bool> inputs_in_place;   // a Concat step: the inputs that lie in its output already
				unsigned int entry_factor = 1;       // entries of the step's output per entry read (the cumulative tiling factor of its last layer)
				bool launches_nothing() const        // Dropout layers only, in place: nothing to do at inference; a Concat with every input in place
				{
					if (!inputs_in_place.empty())
						return std::find(inputs_in_place.begin(), inputs_in_place.end(), false) == inputs_in_place.end();
					return passes_input_on && (output_buffer == input_buffers.at(0));
				}
			};

			bool is_unary_elementwise(const std::string& type)
			{
				return (type == batch_norm_layer::layer_type_name) || (type == rectified_linear_layer::layer_type_name)
					|| (type == parametric_rectified_linear_layer::layer_type_name) || (type == exponential_linear_layer::layer_type_name)
					|| (type == sigmoid_layer::layer_type_name) || (type == hyperbolic_tangent_layer::layer_type_name)
					|| (type == absolute_layer::layer_type_name) || (type == dropout_layer::layer_type_name);
			}

			struct pinned_buffer
			{
				explicit pinned_buffer(size_t bytes) : ptr(nullptr), bytes(bytes)
				{
					hip_safe_call(nnf_hip_host_malloc(&ptr, bytes));
				}
				~pinned_buffer()
				{
					if (ptr != nullptr)
						nnf_hip_host_free(ptr);
				}
				pinned_buffer(const pinned_buffer&) = delete;
				pinned_buffer& operator=(const pinned_buffer&) = delete;
				void * ptr;
				size_t bytes;
			};

			struct hip_event
			{
				hip_event() : ev(nullptr) { hip_safe_call(nnf_hip_event_create(&ev)); }
				~hip_event() { if (ev != nullptr) nnf_hip_event_destroy(ev); }
				hip_event(const hip_event&) = delete;
				hip_event& operator=(const hip_event&) = delete;
				void * ev;
			};
		}

		// What a run holds on the device and in pinned host memory: data and output layer buffers once per I/O
		// slot, the rest shared; the working buffers testers ask for, per step (steps on different streams may
		// run at the same time); pinned staging per slot; the states and the workspace of the statistics. Kept
		// in the object from one run to the next while the packet size, the kind of writer, the weights and the
		// plan stay the same, so that a caller who runs data set after data set allocates once.
		struct forward_propagation_hip::run_buffers
		{
			unsigned int packet = 0;
			int slot_count = 0;
			int staging_slot_count = 0;
			bool with_output_staging = false;
			bool stats_on_device = false;
			std::vector<std::vector<hip_linear_buffer_device::ptr> > buffers; // per slot
			std::vector<std::pair<hip_linear_buffer_device::ptr, hip_linear_buffer_device::ptr> > temporary;
			std::vector<std::vector<const float *> > chunk_ptrs; // weight pointers of the fused steps
			std::vector<std::map<std::string, std::unique_ptr<pinned_buffer> > > staging; // per staging slot
			std::map<std::string, hip_linear_buffer_device::ptr> stat_states, stat_workspaces;
			std::map<std::string, size_t> stat_workspace_bytes;
		};

		struct forward_propagation_hip::impl
		{
			std::vector<layer::const_ptr> exec_layers; // layers with inputs, execution order
			std::map<std::string, layer_tester_hip::ptr> testers;
			std::map<std::string, std::vector<hip_linear_buffer_device::const_ptr> > weights;
			std::map<std::string, std::vector<hip_linear_buffer_device::const_ptr> > weights_custom;    // integer side data
			std::map<std::string, std::vector<hip_linear_buffer_device::const_ptr> > persistent_working; // per tester, made at configuration
			network_data::const_ptr host_data;

			std::vector<step_plan> plans;
			std::vector<size_t> buffer_floats_per_entry;   // planned device buffers
			std::map<std::string, int> value_to_buffer;    // data layers, step outputs
			void * stream = nullptr;          // kernels: the main kernel stream, kernel_streams[0]
			std::vector<void *> kernel_streams; // as many as the plan uses (steps' stream_index); the ones behind [0] take steps that do not depend on what [0] is doing
			void * upload_stream = nullptr;   // host -> device copies
			void * download_stream = nullptr; // device -> host copies
			std::vector<std::unique_ptr<hip_event> > stream_done; // per kernel stream behind [0]: end of its part of a packet

			void create_streams(size_t kernel_stream_count)
			{
				if (upload_stream == nullptr)
				{
					hip_safe_call(nnf_hip_stream_create(&upload_stream));
					hip_safe_call(nnf_hip_stream_create(&download_stream));
				}
				while (kernel_streams.size() < std::max<size_t>(1, kernel_stream_count))
				{
					void * s = nullptr;
					hip_safe_call(nnf_hip_stream_create(&s));
					kernel_streams.push_back(s);
					if (kernel_streams.size() > 1)
						stream_done.emplace_back(new hip_event());
				}
				stream = kernel_streams[0];
			}

			// Enqueues the launch plan for one packet whose data layer buffers are filled: every step on its
			// kernel stream (steps that depend on each other share one). The caller has made every kernel stream wait for
			// whatever the packet itself waits for; on return kernel_streams[0] has been made to wait for the
			// others, so that whatever is enqueued on it next runs after the whole packet.
			void enqueue_plan(
				const std::vector<hip_linear_buffer_device::ptr>& buffers,
				unsigned int entries_read,
				const std::vector<std::vector<const float *> >& chunk_ptrs,
				const std::vector<std::pair<hip_linear_buffer_device::ptr, hip_linear_buffer_device::ptr> >& temporary_buffers,
				const std::vector<std::unique_ptr<hip_event> > * profile_events);

			~impl()
			{
				for(void * s : kernel_streams)
					nnf_hip_stream_destroy(s);
				if (upload_stream != nullptr)
					nnf_hip_stream_destroy(upload_stream);
				if (download_stream != nullptr)
					nnf_hip_stream_destroy(download_stream);
			}
		};

		void forward_propagation_hip::impl::enqueue_plan(
			const std::vector<hip_linear_buffer_device::ptr>& buffers,
			unsigned int entries_read,
			const std::vector<std::vector<const float *> >& chunk_ptrs,
			const std::vector<std::pair<hip_linear_buffer_device::ptr, hip_linear_buffer_device::ptr> >& temporary_buffers,
			const std::vector<std::unique_ptr<hip_event> > * profile_events)
		{
			const std::vector<hip_linear_buffer_device::const_ptr> none;
			std::vector<bool> stream_used(kernel_streams.size(), false);
			for(size_t i = 0; i < plans.size(); ++i)
			{
				step_plan& plan = plans[i];
				void * const step_stream = kernel_streams.at(plan.info.stream_index);
				const unsigned int step_entries = entries_read * plan.entry_factor; // nnforge/plain/forward_propagation_plain.cpp:185
				if (profile_events != nullptr)
					hip_safe_call(nnf_hip_event_record((*profile_events)[i]->ev, step_stream));
				if (plan.launches_nothing())
					continue;
				stream_used[plan.info.stream_index] = true;

				std::vector<hip_linear_buffer_device::const_ptr> inputs;
				for(int b : plan.input_buffers)
					inputs.push_back(buffers[b]);
				if (plan.info.batch_index >= 0)
				{
					// the first step of a run of independent fused groups launches all of them
					if ((i > 0) && (plans[i - 1].info.batch_index == plan.info.batch_index))
						continue;
					std::vector<nnf_hip_chain_desc> descs;
					std::vector<float *> outputs;
					std::vector<std::vector<const float *> > in_ptrs;
					std::vector<const float * const *> in_ptr_ptrs, chunk_ptr_ptrs;
					for(size_t m = i; (m < plans.size()) && (plans[m].info.batch_index == plan.info.batch_index); ++m)
					{
						step_plan& member = plans[m];
						member.desc.entry_count = entries_read * member.entry_factor;
						descs.push_back(member.desc);
						outputs.push_back(*buffers[member.output_buffer]);
						in_ptrs.push_back(std::vector<const float *>());
						for(int b : member.input_buffers)
							in_ptrs.back().push_back(static_cast<const float *>(*static_cast<hip_linear_buffer_device::const_ptr>(buffers[b])));
						chunk_ptr_ptrs.push_back(chunk_ptrs[m].empty() ? nullptr : chunk_ptrs[m].data());
					}
					for(const std::vector<const float *>& v : in_ptrs)
						in_ptr_ptrs.push_back(v.data());
					hip_safe_call(nnf_hip_chain_forward_batch(step_stream, static_cast<uint32_t>(descs.size()), descs.data(), outputs.data(),
						in_ptr_ptrs.data(), chunk_ptr_ptrs.data()));
				}
				else if (plan.prologue)
				{
					plan.desc.entry_count = step_entries;
					plan.tester->enqueue_forward_propagation_with_prologue(step_stream, buffers[plan.output_buffer], inputs, plan.desc,
						chunk_ptrs[i].empty() ? nullptr : chunk_ptrs[i].data(), step_entries);
				}
				else if (plan.info.fused && (plan.view_stride != 0))
				{
					// The groups that write into one Concat's output and follow one another in the plan go to the kernels in
					// one call: none of them reads what another writes (only the Concat reads them), their parts of the
					// output lie side by side. The first of them launches all; with per-action times wanted, each its own.
					if ((profile_events == nullptr) && (i > 0) && (plans[i - 1].view_stride != 0) && (plans[i - 1].info.writes_into == plan.info.writes_into)
						&& (plans[i - 1].info.stream_index == plan.info.stream_index) && (plans[i - 1].entry_factor == plan.entry_factor))
						continue;
					std::vector<nnf_hip_chain_desc> descs;
					std::vector<float *> outputs;
					std::vector<uint32_t> strides;
					std::vector<std::vector<const float *> > in_ptrs;
					std::vector<const float * const *> in_ptr_ptrs, chunk_ptr_ptrs;
					for(size_t m = i; m < plans.size(); ++m)
					{
						step_plan& member = plans[m];
						if ((m > i) && ((profile_events != nullptr) || (member.view_stride == 0) || (member.info.writes_into != plan.info.writes_into)
							|| (member.info.stream_index != plan.info.stream_index) || (member.entry_factor != plan.entry_factor)))
							break;
						member.desc.entry_count = step_entries;
						descs.push_back(member.desc);
						outputs.push_back(static_cast<float *>(*buffers[member.output_buffer]) + member.view_offset);
						strides.push_back(member.view_stride);
						in_ptrs.push_back(std::vector<const float *>());
						for(int b : member.input_buffers)
							in_ptrs.back().push_back(static_cast<const float *>(*static_cast<hip_linear_buffer_device::const_ptr>(buffers[b])));
						chunk_ptr_ptrs.push_back(chunk_ptrs[m].empty() ? nullptr : chunk_ptrs[m].data());
					}
					for(const std::vector<const float *>& v : in_ptrs)
						in_ptr_ptrs.push_back(v.data());
					hip_safe_call(nnf_hip_chain_forward_strided_batch(step_stream, static_cast<uint32_t>(descs.size()), descs.data(), outputs.data(),
						strides.data(), in_ptr_ptrs.data(), chunk_ptr_ptrs.data()));
				}
				else if (plan.info.fused)
				{
					plan.desc.entry_count = step_entries;
					std::vector<const float *> in_ptrs;
					for(const hip_linear_buffer_device::const_ptr& b : inputs)
						in_ptrs.push_back(static_cast<const float *>(*b));
					hip_safe_call(nnf_hip_chain_forward(step_stream, &plan.desc, *buffers[plan.output_buffer], in_ptrs.data(),
						chunk_ptrs[i].empty() ? nullptr : chunk_ptrs[i].data()));
				}
				else if (!plan.inputs_in_place.empty())
					plan.tester->enqueue_forward_propagation_with_inputs_in_place(step_stream, buffers[plan.output_buffer], inputs, plan.inputs_in_place, step_entries);
				else
				{
					const std::string& layer_name = plan.info.layer_names[0];
					const auto of_layer = [&layer_name, &none] (const std::map<std::string, std::vector<hip_linear_buffer_device::const_ptr> >& m)
						-> const std::vector<hip_linear_buffer_device::const_ptr>&
					{
						std::map<std::string, std::vector<hip_linear_buffer_device::const_ptr> >::const_iterator it = m.find(layer_name);
						return (it == m.end()) ? none : it->second;
					};
					plan.tester->enqueue_forward_propagation(step_stream, buffers[plan.output_buffer], none,
						of_layer(weights), of_layer(weights_custom), inputs, of_layer(persistent_working),
						temporary_buffers[i].first, temporary_buffers[i].second, step_entries);
				}
			}
			if (profile_events != nullptr)
				hip_safe_call(nnf_hip_event_record((*profile_events)[plans.size()]->ev, kernel_streams[0]));
			for(size_t s = 1; s < kernel_streams.size(); ++s)
			{
				if (!stream_used[s])
					continue;
				hip_safe_call(nnf_hip_event_record(stream_done[s - 1]->ev, kernel_streams[s]));
				hip_safe_call(nnf_hip_stream_wait_event(kernel_streams[0], stream_done[s - 1]->ev));
			}
		}

		forward_propagation_hip::forward_propagation_hip(
			const network_schema& schema,
			const std::vector<std::string>& output_layer_names,
			debug_state::ptr debug,
			profile_state::ptr profile,
			hip_running_configuration::const_ptr hip_config)
			: forward_propagation(schema, output_layer_names, debug, profile)
			, p(new impl())
			, hip_config(hip_config)
			, per_entry_bytes(0)
			, max_entry_count(0)
		{
			for(const layer::const_ptr& l : this->schema->get_layers_in_forward_propagation_order())
			{
				if (l->input_layer_instance_names.empty())
				{
					// a data layer, or a layer computed elsewhere (the base class hands those over without inputs):
					// either way the reader supplies its values
					if ((l->get_type_name() != data_layer::layer_type_name) && (dynamic_cast<const external_layer *>(l.get()) == nullptr))
						throw neural_network_exception("Layer " + l->instance_name + " of type " + l->get_type_name() + " has no inputs");
					continue;
				}
				// fails here, at construction, for a layer type without a registered tester
				layer_testing_schema_factory::get_singleton().create_testing_schema_layer(l);
				p->exec_layers.push_back(l);
			}
		}

		forward_propagation_hip::~forward_propagation_hip()
		{
		}

		void forward_propagation_hip::actual_set_data(network_data::const_ptr data)
		{
			kept_run.reset(); // it holds pointers to the weights
			p->host_data = data;
			p->weights.clear();
			p->weights_custom.clear();
			if (hip_config->is_offline())
				return;
			hip_config->set_device();
			// nnforge/cuda/forward_propagation_cuda.cpp:1016-1050: every tester uploads its own layer's data
			for(const layer::const_ptr& l : p->exec_layers)
			{
				std::map<std::string, layer_tester_hip::ptr>::const_iterator t = p->testers.find(l->instance_name);
				if (t == p->testers.end())
					continue;
				layer_data::ptr d = data->find(l->instance_name);
				if (d)
					p->weights[l->instance_name] = t->second->get_data(d);
				layer_data_custom::ptr dc = data->find_custom(l->instance_name);
				if (dc)
					p->weights_custom[l->instance_name] = t->second->set_get_data_custom(dc);
			}
		}

		void forward_propagation_hip::actual_clear_data()
		{
			kept_run.reset();
			p->host_data.reset();
			p->weights.clear();
			p->weights_custom.clear();
		}

		void forward_propagation_hip::layer_config_map_modified()
		{
			hip_config->set_device();
			kept_run.reset(); // sized for the plan that is about to be replaced

			// testers for the new shapes
			p->testers.clear();
			for(const layer::const_ptr& l : p->exec_layers)
			{
				std::vector<layer_configuration_specific> inputs;
				for(const std::string& input : l->input_layer_instance_names)
					inputs.push_back(layer_config_map[input]);
				layer_testing_schema::ptr ts = layer_testing_schema_factory::get_singleton().create_testing_schema_layer(l);
				p->testers[l->instance_name] = ts->create_tester(inputs, layer_config_map[l->instance_name], hip_config);
			}
			p->persistent_working.clear();
			if (!hip_config->is_offline())
				for(const std::pair<const std::string, layer_tester_hip::ptr>& t : p->testers)
					p->persistent_working[t.first] = t.second->get_persistent_working_data();
			if (p->host_data)
				actual_set_data(p->host_data);

			// ---- launch plan: fuse runs of element-wise layers ----------------------------------
			const std::set<std::string> outputs(output_layer_names.begin(), output_layer_names.end());
			std::map<std::string, pending_group> pending;
			std::vector<std::pair<std::string, pending_group> > groups; // materialized, in execution order
			std::vector<std::pair<std::string, bool> > step_order;      // (layer name, is_group)
			std::map<std::string, pending_group> prologues;             // subsampling layer -> the group it applies to its input
			std::vector<unsigned int> step_slots;                       // with runs of groups launched together: the slot of every step of step_order

			auto materialize = [&](const std::string& name)
			{
				std::map<std::string, pending_group>::iterator it = pending.find(name);
				if (it == pending.end())
					return;
				groups.push_back(std::make_pair(name, it->second));
				step_order.push_back(std::make_pair(name, true));
				pending.erase(it);
			};
			auto absorbable = [&](const std::string& producer, const layer_configuration_specific& consumer_config) -> bool
			{
				return hip_config->fuse_layers
					&& (pending.find(producer) != pending.end())
					&& (this->schema->get_consumer_count(producer) == 1)
					&& (outputs.find(producer) == outputs.end())
					&& (layer_config_map[producer] == consumer_config);
			};

			for(const layer::const_ptr& l : p->exec_layers)
			{
				const std::string& name = l->instance_name;
				const std::string type = l->get_type_name();
				const layer_configuration_specific& config = layer_config_map[name];
				bool grouped = false;

				if (is_unary_elementwise(type))
				{
					const std::string& producer = l->input_layer_instance_names.at(0);
					pending_group g;
					if (absorbable(producer, config) && (pending[producer].op_count() + 1 <= NNF_HIP_MAX_OPS))
					{
						g = pending[producer];
						pending.erase(producer);
						if (g.add_layer_name.empty())
							g.arms[0].ops.push_back(name);
						else
							g.tail.push_back(name);
					}
					else
					{
						materialize(producer);
						pending_arm a;
						a.source = producer;
						a.ops.push_back(name);
						g.arms.push_back(a);
					}
					pending[name] = g;
					grouped = true;
				}
				else if ((type == add_layer::layer_type_name) && (l->input_layer_instance_names.size() <= NNF_HIP_MAX_INPUTS) && hip_config->fuse_layers)
				{
					bool same_configs = true;
					for(const std::string& producer : l->input_layer_instance_names)
						same_configs = same_configs && (layer_config_map[producer] == config);
					pending_group g;
					g.add_layer_name = name;
					size_t ops = 0;
					for(const std::string& producer : l->input_layer_instance_names)
					{
						pending_arm a;
						a.source = producer;
						if (same_configs && absorbable(producer, config) && pending[producer].add_layer_name.empty()
							&& (ops + pending[producer].op_count() <= NNF_HIP_MAX_OPS))
						{
							a = pending[producer].arms[0];
							ops += a.ops.size();
							pending.erase(producer);
						}
						else
							materialize(producer);
						g.arms.push_back(a);
					}
					pending[name] = g;
					grouped = true;
				}

				if (!grouped)
				{
					// A subsampling layer takes the pending group that feeds it along: the group's layers are
					// applied to the values on their way into the subsampling kernel's staging buffer. A chain of
					// layers over one input goes with every subsampling kernel that stages its input; two chains
					// joined by an Add (the last block of a residual network) with the average over whole planes.
					if (hip_config->fuse_layers && (l->input_layer_instance_names.size() == 1))
					{
						const std::string& producer = l->input_layer_instance_names[0];
						std::map<std::string, pending_group>::iterator it = pending.find(producer);
						const bool chain = (it != pending.end()) && it->second.add_layer_name.empty() && (it->second.arms.size() == 1);
						const bool joined = (it != pending.end()) && !it->second.add_layer_name.empty() && (it->second.arms.size() == 2);
						if ((chain || joined) && p->testers[name]->can_apply_prologue(static_cast<unsigned int>(it->second.arms.size()))
							&& (this->schema->get_consumer_count(producer) == 1) && (outputs.find(producer) == outputs.end()))
						{
							unsigned int weighted = 0;
							bool only_dropout = chain; // such a group costs no launch on its own
							std::vector<std::string> op_layers = it->second.tail;
							for(const pending_arm& arm : it->second.arms)
								op_layers.insert(op_layers.end(), arm.ops.begin(), arm.ops.end());
							for(const std::string& op_layer : op_layers)
							{
								nnf_hip_op op;
								weighted += (p->testers[op_layer]->get_chain_op(op) > 0) ? 1u : 0u;
								only_dropout = only_dropout && (this->schema->get_layer(op_layer)->get_type_name() == dropout_layer::layer_type_name);
							}
							if ((weighted <= 2) && !only_dropout)
							{
								prologues[name] = it->second;
								pending.erase(it);
							}
						}
					}
					for(const std::string& producer : l->input_layer_instance_names)
						materialize(producer);
					step_order.push_back(std::make_pair(name, false));
				}
				else if ((outputs.find(name) != outputs.end()) || (this->schema->get_consumer_count(name) != 1))
					materialize(name);
			}
			// anything still pending feeds nothing (cannot happen for a reduced schema) - write it out anyway
			while (!pending.empty())
				materialize(pending.begin()->first);

			// ---- groups that write into the Concat layer behind them -----------------------------------------
			// A Concat layer only puts its inputs side by side, entry by entry (nnforge/plain/concat_layer_tester_plain.cpp:
			// 45-58). A fused group that nothing else reads can write its result there itself: its launch goes over
			// (tiles of an entry) x (entries) and steps from entry to entry by the Concat's neuron count
			// (nnf_hip_chain_forward_strided), the group's own tensor is never made, and the Concat copies only the inputs
			// that are not such groups - nothing at all when every input is one. What qualifies: a group with at most two
			// inputs, read by the Concat alone and no output itself, whose entries and whose place in the Concat's entry
			// start on 16-byte boundaries, and large enough per entry for a launch over entries to be worth it.
			struct concat_view
			{
				std::string concat;
				uint32_t offset, stride;
			};
			std::map<std::string, concat_view> view_of;                        // by the group's name (its last layer)
			std::map<std::string, std::vector<bool> > concat_inputs_in_place;  // by the Concat layer's name
			if (hip_config->fuse_layers && hip_config->concat_in_place)
			{
				constexpr unsigned int min_view_floats_per_entry = 1024;
				std::map<std::string, const pending_group *> group_named;
				for(const std::pair<std::string, pending_group>& g : groups)
					group_named[g.first] = &g.second;
				for(const std::pair<std::string, bool>& so : step_order)
				{
					if (so.second || (prologues.find(so.first) != prologues.end()))
						continue;
					layer::const_ptr l = this->schema->get_layer(so.first);
					if ((l->get_type_name() != concat_layer::layer_type_name) || !p->testers[so.first]->can_take_inputs_in_place())
						continue;
					const uint32_t stride = layer_config_map[so.first].get_neuron_count();
					std::vector<bool> flags;
					uint32_t offset = 0;
					bool any = false;
					for(const std::string& input : l->input_layer_instance_names)
					{
						const layer_configuration_specific& input_config = layer_config_map[input];
						const uint32_t count = input_config.get_neuron_count();
						bool in_place = false;
						std::map<std::string, const pending_group *>::const_iterator g = group_named.find(input);
						if ((g != group_named.end()) && (this->schema->get_consumer_count(input) == 1) && (outputs.find(input) == outputs.end())
							&& (view_of.find(input) == view_of.end()) && (count >= min_view_floats_per_entry) && ((offset % 4) == 0))
						{
							nnf_hip_chain_desc shape;
							std::memset(&shape, 0, sizeof(shape));
							shape.entry_count = 1;
							shape.feature_map_count = input_config.feature_map_count;
							shape.neuron_count_per_feature_map = input_config.get_neuron_count_per_feature_map();
							shape.input_count = static_cast<uint32_t>(g->second->arms.size());
							in_place = nnf_hip_chain_forward_strided_status(&shape, stride) == NNF_HIP_OK;
						}
						if (in_place)
						{
							view_of[input] = concat_view{ so.first, offset, stride };
							any = true;
						}
						flags.push_back(in_place);
						offset += count;
					}
					if (any)
						concat_inputs_in_place[so.first] = flags;
				}
			}

			// ---- order: which steps share a launch ---------------------------------------------------------
			// With independent groups launched together (see below) a run of such groups ends where a step depends on
			// one of them, so the order of the steps decides how many launches there are and how large each is. Every
			// step gets a slot: one behind the latest slot of the steps whose results it reads, or later if nothing that
			// follows needs it sooner. Steps that others wait for (in a residual network: the joins of a stage, one per
			// level of the graph) have no choice; the groups that could run at any time (one convolution's BatchNorm and
			// ReLU each) are spread over the slots so that each launch has about the same number of bytes to move - a
			// level with one join alone would be a small launch, and a small launch runs below the rate of a large one.
			// Measured on the ResNet-50 stack's 48 groups (MI355X, kernels only): levels as they come, groups of one kind
			// per launch, 9 launches 1015-1018 us at 64 entries, 151 us at 8, 45 us at 1; spread like this, 6 launches,
			// 1007, 149 and 37 us. Steps of a slot: those that wait for the slot before first, then the other groups, then
			// what is launched on its own, so that a slot is one run.
			if (hip_config->batch_independent_groups && !profile->is_profile())
			{
				std::map<std::string, const pending_group *> group_of;
				for(const std::pair<std::string, pending_group>& g : groups)
					group_of[g.first] = &g.second;
				const size_t count = step_order.size();
				std::map<std::string, size_t> step_of_value; // by the name of the layer whose output a step stores
				std::vector<std::vector<size_t> > producers(count), consumers(count);
				std::vector<unsigned int> level(count, 0);
				std::vector<bool> joins_launches(count, false);
				std::vector<double> bytes(count, 0.0);
				unsigned int max_level = 0;
				for(size_t i = 0; i < count; ++i)
				{
					const std::string& name = step_order[i].first;
					std::vector<std::string> sources;
					if (step_order[i].second)
					{
						const pending_group& g = *group_of[name];
						for(const pending_arm& a : g.arms)
							sources.push_back(a.source);
						// a single layer is its tester's launch; a group that writes into a Concat's output has a launch of its own
						joins_launches[i] = ((g.op_count() + (g.add_layer_name.empty() ? 0 : 1)) > 1) && (view_of.find(name) == view_of.end());
						bytes[i] = static_cast<double>(layer_config_map[name].get_neuron_count()) * static_cast<double>(g.arms.size() + 1);
					}
					else if (prologues.find(name) != prologues.end())
						for(const pending_arm& arm : prologues[name].arms)
							sources.push_back(arm.source);
					else
						sources = this->schema->get_layer(name)->input_layer_instance_names;
					for(const std::string& source : sources)
					{
						std::map<std::string, size_t>::const_iterator it = step_of_value.find(source);
						if (it == step_of_value.end())
							continue; // data layers are on no level
						producers[i].push_back(it->second);
						consumers[it->second].push_back(i);
						level[i] = std::max(level[i], level[it->second] + 1);
					}
					step_of_value[name] = i;
					max_level = std::max(max_level, level[i]);
				}
				// the latest slot that keeps every follower where it is
				std::vector<unsigned int> latest(count, max_level);
				for(size_t i = count; i-- > 0; )
				{
					for(size_t c : consumers[i])
						latest[i] = std::min(latest[i], latest[c] - 1);
					if (!joins_launches[i])
						latest[i] = level[i];
				}
				std::vector<double> slot_bytes(max_level + 1, 0.0);
				std::vector<unsigned int> slot_groups(max_level + 1, 0);
				for(size_t i = 0; i < count; ++i)
					if (joins_launches[i] && (latest[i] == level[i]))
					{
						slot_bytes[level[i]] += bytes[i];
						++slot_groups[level[i]];
					}
				std::vector<unsigned int> slot(count, 0);
				std::vector<unsigned int> rank_in_slot(count, 2);
				for(size_t i = 0; i < count; ++i)
				{
					unsigned int earliest = 0;
					for(size_t producer : producers[i])
						earliest = std::max(earliest, slot[producer] + 1);
					// a step nothing pins (latest beyond its level) may have been pushed by a producer that moved
					const unsigned int last = std::max(earliest, latest[i]);
					slot[i] = earliest;
					if (joins_launches[i] && (latest[i] != level[i]))
					{
						// the lightest slot, one with room in its launch before one without
						bool chosen_has_room = false;
						for(unsigned int candidate = earliest; candidate <= last; ++candidate)
						{
							const bool room = slot_groups[candidate] < NNF_HIP_MAX_GROUPS_PER_LAUNCH;
							const bool better = (candidate == earliest) || (room && !chosen_has_room)
								|| ((room == chosen_has_room) && (slot_bytes[candidate] < slot_bytes[slot[i]]));
							if (better)
							{
								slot[i] = candidate;
								chosen_has_room = room;
							}
						}
						slot_bytes[slot[i]] += bytes[i];
						++slot_groups[slot[i]];
					}
					if (joins_launches[i])
						rank_in_slot[i] = ((earliest == slot[i]) && (earliest > 0)) ? 0 : 1;
				}
				std::vector<size_t> order(count);
				for(size_t i = 0; i < count; ++i)
					order[i] = i;
				std::stable_sort(order.begin(), order.end(), [&slot, &rank_in_slot] (size_t a, size_t b)
					{ return (slot[a] != slot[b]) ? (slot[a] < slot[b]) : (rank_in_slot[a] < rank_in_slot[b]); });
				std::vector<std::pair<std::string, bool> > sorted;
				for(size_t i : order)
				{
					sorted.push_back(step_order[i]);
					step_slots.push_back(slot[i]);
				}
				step_order.swap(sorted);
			}

			// ---- steps ---------------------------------------------------------------------------
			p->plans.clear();
			steps.clear();
			action_flops_per_entry.clear();
			action_bytes_per_entry.clear();
			action_layer_names.clear();
			action_layer_types.clear();
			std::map<std::string, const pending_group *> group_by_name;
			for(const std::pair<std::string, pending_group>& g : groups)
				group_by_name[g.first] = &g.second;

			for(const std::pair<std::string, bool>& so : step_order)
			{
				step_plan plan;
				std::memset(&plan.desc, 0, sizeof(plan.desc));
				plan.output_buffer = -1;
				const std::string& name = so.first;
				const layer_configuration_specific& config = layer_config_map[name];
				// the group's layers as the kernels want them; shape: the tensors the group works on
				auto fill_desc = [&](const pending_group& g, const layer_configuration_specific& shape)
				{
					nnf_hip_chain_desc& d = plan.desc;
					d.feature_map_count = shape.feature_map_count;
					d.neuron_count_per_feature_map = shape.get_neuron_count_per_feature_map();
					d.input_count = static_cast<uint32_t>(g.arms.size());
					d.has_add = g.add_layer_name.empty() ? 0u : 1u;
					d.add_alpha = 1.0F;
					if (d.has_add)
						get_add_alpha(*p->testers[g.add_layer_name], d.add_alpha);
					uint32_t op_index = 0;
					int chunk_index = 0;
					auto push_op = [&](const std::string& layer_name)
					{
						nnf_hip_op& op = d.ops[op_index++];
						const int chunks = p->testers[layer_name]->get_chain_op(op);
						if (chunks < 0)
							throw neural_network_exception("Layer " + layer_name + " cannot be part of a fused group");
						op.chunk = chunk_index;
						if (chunks > 0)
						{
							plan.chunk_layers.push_back(layer_name);
							chunk_index += chunks;
						}
					};
					for(size_t j = 0; j < g.arms.size(); ++j)
					{
						d.arm_op_count[j] = static_cast<uint32_t>(g.arms[j].ops.size());
						for(const std::string& op : g.arms[j].ops)
							push_op(op);
					}
					d.tail_op_count = static_cast<uint32_t>(g.tail.size());
					for(const std::string& op : g.tail)
						push_op(op);
				};
				if (!so.second && (prologues.find(name) != prologues.end()))
				{
					const pending_group& g = prologues[name];
					for(const pending_arm& arm : g.arms)
					{
						plan.info.input_names.push_back(arm.source);
						plan.info.layer_names.insert(plan.info.layer_names.end(), arm.ops.begin(), arm.ops.end());
					}
					if (!g.add_layer_name.empty())
						plan.info.layer_names.push_back(g.add_layer_name);
					plan.info.layer_names.insert(plan.info.layer_names.end(), g.tail.begin(), g.tail.end());
					plan.info.layer_names.push_back(name);
					plan.info.fused = true;
					plan.prologue = true;
					plan.tester = p->testers[name];
					fill_desc(g, layer_config_map[g.arms[0].source]);
				}
				else if (!so.second)
				{
					layer::const_ptr l = this->schema->get_layer(name);
					plan.info.layer_names.push_back(name);
					plan.info.input_names = l->input_layer_instance_names;
					plan.info.fused = false;
					plan.tester = p->testers[name];
				}
				else
				{
					const pending_group& g = *group_by_name[name];
					const bool single_layer = (g.op_count() + (g.add_layer_name.empty() ? 0 : 1)) == 1;
					for(const pending_arm& a : g.arms)
					{
						plan.info.input_names.push_back(a.source);
						for(const std::string& op : a.ops)
							plan.info.layer_names.push_back(op);
					}
					if (!g.add_layer_name.empty())
						plan.info.layer_names.push_back(g.add_layer_name);
					for(const std::string& op : g.tail)
						plan.info.layer_names.push_back(op);
					std::map<std::string, concat_view>::const_iterator view = view_of.find(name);
					if (single_layer && (view == view_of.end()))
					{
						// a group of one layer is that layer's own tester
						plan.info.fused = false;
						plan.tester = p->testers[plan.info.layer_names[0]];
					}
					else
					{
						plan.info.fused = true;
						fill_desc(g, config);
					}
					if (view != view_of.end())
					{
						plan.view_offset = view->second.offset;
						plan.view_stride = view->second.stride;
						plan.info.writes_into = view->second.concat;
					}
				}
				if (!so.second && (concat_inputs_in_place.find(name) != concat_inputs_in_place.end()))
				{
					plan.inputs_in_place = concat_inputs_in_place[name];
					for(size_t j = 0; j < plan.inputs_in_place.size(); ++j)
						if (plan.inputs_in_place[j])
							plan.info.inputs_in_place.push_back(plan.info.input_names[j]);
				}
				// report bookkeeping: name, layer types, flops (the reference's model) and memory traffic per entry
				std::string types;
				float step_flops = 0.0F;
				plan.passes_input_on = true;
				plan.entry_factor = cumulative_tiling_factor_map.at(plan.info.layer_names.back());
				for(const std::string& n : plan.info.layer_names)
				{
					plan.key += (plan.key.empty() ? "" : "+") + n;
					layer::const_ptr l = this->schema->get_layer(n);
					plan.passes_input_on = plan.passes_input_on && (l->get_type_name() == dropout_layer::layer_type_name);
					types += (types.empty() ? "" : "+") + l->get_type_name();
					std::vector<layer_configuration_specific> inputs;
					for(const std::string& input : l->input_layer_instance_names)
						inputs.push_back(layer_config_map[input]);
					step_flops += l->get_forward_flops_per_entry(inputs) * static_cast<float>(cumulative_tiling_factor_map.at(n));
				}
				float step_bytes = static_cast<float>(config.get_neuron_count()) * sizeof(float) * static_cast<float>(plan.entry_factor);
				for(const std::string& input : plan.info.input_names)
					step_bytes += static_cast<float>(layer_config_map[input].get_neuron_count()) * sizeof(float) * static_cast<float>(cumulative_tiling_factor_map.at(input));
				// what a Concat finds in place it neither reads nor writes
				for(const std::string& input : plan.info.inputs_in_place)
					step_bytes -= 2.0F * static_cast<float>(layer_config_map[input].get_neuron_count()) * sizeof(float) * static_cast<float>(cumulative_tiling_factor_map.at(input));
				plan.action = layer_name_with_action(plan.info.layer_names.back(), layer_action(layer_action::forward));
				action_flops_per_entry[plan.action] = step_flops;
				action_bytes_per_entry[plan.action] = step_bytes;
				action_layer_names[plan.action] = plan.key;
				action_layer_types[plan.action] = types;

				p->plans.push_back(plan);
				steps.push_back(plan.info);
			}

			// ---- buffers: dedicated for data and output layers, shared by liveness for the rest --
			p->buffer_floats_per_entry.clear();
			p->value_to_buffer.clear();
			auto new_buffer = [&](size_t floats_per_entry) -> int
			{
				p->buffer_floats_per_entry.push_back(floats_per_entry);
				return static_cast<int>(p->buffer_floats_per_entry.size()) - 1;
			};
			for(const std::string& n : data_layer_names)
				p->value_to_buffer[n] = new_buffer(layer_config_map[n].get_neuron_count());

			std::map<std::string, size_t> last_use;
			for(size_t i = 0; i < p->plans.size(); ++i)
				for(const std::string& in : p->plans[i].info.input_names)
					last_use[in] = i;

			// With runs of groups launched together a buffer whose value dies in a slot is handed out again from the next slot
			// on: given to a step of the same slot it would make that step wait for the buffer's readers, and the run would
			// end there (device memory is not what this driver is short of).
			std::vector<int> free_buffers;
			std::vector<int> freed_in_this_slot;
			std::set<int> shareable; // buffers that hold intermediate values
			for(size_t i = 0; i < p->plans.size(); ++i)
			{
				step_plan& plan = p->plans[i];
				if (!step_slots.empty() && (i > 0) && (step_slots[i] != step_slots[i - 1]))
				{
					free_buffers.insert(free_buffers.end(), freed_in_this_slot.begin(), freed_in_this_slot.end());
					freed_in_this_slot.clear();
				}
				const std::string& out_name = plan.info.layer_names.back();
				// the value whose buffer the step writes: its own, or the output of the Concat layer it writes into
				const std::string& buffer_owner = plan.info.writes_into.empty() ? out_name : plan.info.writes_into;
				// per entry read: a layer behind a tiling layer holds several entries for each (nnforge/plain/forward_propagation_plain.cpp:281)
				const size_t out_floats = static_cast<size_t>(layer_config_map[buffer_owner].get_neuron_count()) * plan.entry_factor;
				for(const std::string& in : plan.info.input_names)
					plan.input_buffers.push_back(p->value_to_buffer.at(in));

				const bool dedicated = (outputs.find(buffer_owner) != outputs.end()) || hip_config->dont_share_buffers;
				int chosen = -1;
				// a Concat's buffer exists from the first group that writes into it
				const std::map<std::string, int>::const_iterator planned = p->value_to_buffer.find(buffer_owner);
				if (planned != p->value_to_buffer.end())
					chosen = planned->second;
				if (!dedicated && (chosen < 0))
				{
					// in place: the first input dies here, nothing else reads its buffer in this step, same size
					const int can_write = (plan.prologue || (plan.view_stride != 0)) ? -1 : (plan.info.fused ? 0 : plan.tester->get_input_index_layer_can_write());
					if (can_write == 0)
					{
						const int b0 = plan.input_buffers[0];
						const bool dies_here = last_use[plan.info.input_names[0]] == i;
						const bool unique = std::count(plan.input_buffers.begin(), plan.input_buffers.end(), b0) == 1;
						if (dies_here && unique && (shareable.find(b0) != shareable.end()) && (p->buffer_floats_per_entry[b0] == out_floats))
							chosen = b0;
					}
					if (chosen < 0)
					{
						// smallest free buffer that is large enough
						std::vector<int>::iterator best = free_buffers.end();
						for(std::vector<int>::iterator it = free_buffers.begin(); it != free_buffers.end(); ++it)
						{
							if (p->buffer_floats_per_entry[*it] < out_floats)
								continue;
							if ((best == free_buffers.end()) || (p->buffer_floats_per_entry[*it] < p->buffer_floats_per_entry[*best]))
								best = it;
						}
						if (best != free_buffers.end())
						{
							chosen = *best;
							free_buffers.erase(best);
						}
					}
				}
				if (chosen < 0)
				{
					chosen = new_buffer(out_floats);
					if (!dedicated)
						shareable.insert(chosen);
				}
				plan.output_buffer = chosen;
				p->value_to_buffer[out_name] = chosen;
				p->value_to_buffer[buffer_owner] = chosen;

				// inputs that die here return to the pool (unless just reused in place)
				for(size_t j = 0; j < plan.info.input_names.size(); ++j)
				{
					const int b = plan.input_buffers[j];
					std::vector<int>& released = step_slots.empty() ? free_buffers : freed_in_this_slot;
					if ((last_use[plan.info.input_names[j]] == i) && (b != chosen) && (shareable.find(b) != shareable.end())
						&& (std::find(released.begin(), released.end(), b) == released.end()))
						released.push_back(b);
				}
			}

			// ---- kernel streams: which steps may overlap --------------------------------------------
			// A step depends on the earlier steps that wrote the buffers it reads and, because buffers are
			// shared, on the earlier steps that read or wrote the buffer it writes. Steps connected by such
			// dependencies, directly or through other steps, go to one stream, in order; steps that have nothing to
			// do with each other take the streams in turn, so that the start of one overlaps the end of another.
			// No step ever waits for another stream: an event recorded behind a kernel and waited for on another
			// stream costs more than a small kernel takes (measured on MI355X, 51 launches of 1 to 25 MB: 198 us on
			// one stream, 146 us on two without events, 401 us on two with 17 such record / wait pairs), which is why
			// nnforge/cuda/forward_propagation_cuda.cpp:414-423's event per dependency is not taken over.
			// With per-action times wanted every step goes to one stream: overlapping actions have no time of their own.
			//
			// Better than overlapping the ends of launches is not to have them: runs of consecutive fused groups that do
			// not depend on each other are handed to the kernels in one call (nnf_hip_chain_forward_batch), which puts
			// groups of a kind into one launch. A step joins the run unless it depends on a step already in it (a
			// dependency through steps in between would have ended the run at those). Such runs take one stream.
			{
				const bool batching = hip_config->batch_independent_groups && !profile->is_profile();
				const size_t stream_count = (profile->is_profile() || batching) ? 1 : static_cast<size_t>(std::max(1, hip_config->kernel_stream_count));
				const size_t buffer_count = p->buffer_floats_per_entry.size();
				const size_t step_count = p->plans.size();
				std::vector<size_t> component(step_count);
				for(size_t i = 0; i < step_count; ++i)
					component[i] = i;
				const auto root_of = [&component] (size_t i)
				{
					while (component[i] != i)
						i = component[i] = component[component[i]];
					return i;
				};
				std::vector<int> last_writer(buffer_count, -1);
				std::vector<std::vector<int> > readers(buffer_count);
				std::vector<std::set<int> > depends_directly_on(step_count);
				for(size_t i = 0; i < step_count; ++i)
				{
					const step_plan& plan = p->plans[i];
					if (plan.launches_nothing())
						continue; // the value stays where it is: whoever reads it depends on its writer
					const auto depends_on = [&] (int earlier)
					{
						depends_directly_on[i].insert(earlier);
						// the smaller index becomes the root: a component is named after its first step
						const size_t a = root_of(i), b = root_of(static_cast<size_t>(earlier));
						component[std::max(a, b)] = std::min(a, b);
					};
					for(int b : plan.input_buffers)
						if (last_writer[b] >= 0)
							depends_on(last_writer[b]);
					const int out = plan.output_buffer;
					if (last_writer[out] >= 0)
						depends_on(last_writer[out]);
					for(int r : readers[out])
						depends_on(r);
					for(int b : plan.input_buffers)
						readers[b].push_back(static_cast<int>(i));
					last_writer[out] = static_cast<int>(i);
					readers[out].clear();
				}
				std::map<size_t, unsigned int> stream_of_component;
				unsigned int next_stream = 0;
				for(size_t i = 0; i < step_count; ++i)
				{
					const size_t c = root_of(i);
					std::map<size_t, unsigned int>::const_iterator known = stream_of_component.find(c);
					if (known == stream_of_component.end())
					{
						known = stream_of_component.insert(std::make_pair(c, next_stream)).first;
						next_stream = (next_stream + 1) % static_cast<unsigned int>(stream_count);
					}
					p->plans[i].info.stream_index = known->second;
				}

				int batch_count = 0;
				std::vector<int> run; // the steps of the batch being formed
				for(size_t i = 0; i < step_count; ++i)
				{
					step_plan& plan = p->plans[i];
					plan.info.batch_index = -1;
					if (plan.launches_nothing())
						continue; // no launch: neither joins a run nor ends one
					const bool can_join = batching && plan.info.fused && !plan.prologue && (plan.view_stride == 0);
					bool depends_on_run = false;
					for(int member : run)
						depends_on_run = depends_on_run || (depends_directly_on[i].find(member) != depends_directly_on[i].end());
					if (!can_join || depends_on_run)
					{
						batch_count += run.empty() ? 0 : 1;
						run.clear();
					}
					if (can_join)
					{
						plan.info.batch_index = batch_count;
						run.push_back(static_cast<int>(i));
					}
				}
				for(size_t i = 0; i < step_count; ++i)
					steps[i] = p->plans[i].info;
			}

			per_entry_bytes = 0;
			for(size_t floats : p->buffer_floats_per_entry)
				per_entry_bytes += floats * sizeof(float);

			// packet size from the memory budget (nnforge/plain/forward_propagation_plain.cpp:403-444)
			size_t weight_bytes = 0;
			for(const std::pair<const std::string, std::vector<hip_linear_buffer_device::const_ptr> >& w : p->weights)
				for(const hip_linear_buffer_device::const_ptr& b : w.second)
					weight_bytes += b->get_size();
			const size_t budget = hip_config->get_max_bytes();
			// data and output layers have a second device buffer, for the packet whose I/O overlaps the kernels
			std::set<int> io_buffers;
			for(const std::string& n : data_layer_names)
				io_buffers.insert(p->value_to_buffer.at(n));
			for(const std::string& n : output_layer_names)
				io_buffers.insert(p->value_to_buffer.at(n));
			size_t device_bytes_per_entry = per_entry_bytes;
			for(int b : io_buffers)
				device_bytes_per_entry += p->buffer_floats_per_entry[b] * sizeof(float);
			if ((per_entry_bytes == 0) || (budget <= weight_bytes) || ((budget - weight_bytes) / device_bytes_per_entry == 0))
				throw neural_network_exception("Insufficient memory to do forward prop for even one sample");
			const size_t fit = (budget - weight_bytes) / device_bytes_per_entry;
			max_entry_count = static_cast<unsigned int>(std::min<size_t>(fit, static_cast<size_t>(std::max(1, hip_config->max_entry_count))));
			// and no tensor of a packet may outgrow the kernels' 32-bit indices
			size_t largest_floats_per_entry = 1;
			for(size_t floats : p->buffer_floats_per_entry)
				largest_floats_per_entry = std::max(largest_floats_per_entry, floats);
			const size_t index_fit = static_cast<size_t>(NNF_HIP_MAX_ELEMENT_COUNT / largest_floats_per_entry);
			if (index_fit == 0)
				throw neural_network_exception("A single entry of " + std::to_string(largest_floats_per_entry) + " values in one layer is beyond the hip kernels' index range");
			max_entry_count = static_cast<unsigned int>(std::min<size_t>(max_entry_count, index_fit));
			// A run into a statistics writer also holds, per output layer, the running states and the workspace of the
			// reduction (a few KB to MB): where the budget is that tight, the packet gives them room
			{
				size_t stat_bytes = 0;
				for(const std::string& n : output_layer_names)
				{
					const layer_configuration_specific& c = layer_config_map[n];
					size_t workspace = 0;
					if (nnf_hip_feature_map_stat_workspace_bytes(max_entry_count * output_layers_tiling_factor, c.feature_map_count, c.get_neuron_count_per_feature_map(), &workspace) == NNF_HIP_OK)
						stat_bytes += workspace + static_cast<size_t>(c.feature_map_count) * sizeof(nnf_hip_running_stat);
				}
				const size_t used = weight_bytes + device_bytes_per_entry * max_entry_count;
				if ((used + stat_bytes > budget) && (max_entry_count > 1))
				{
					const size_t give_up = (used + stat_bytes - budget + device_bytes_per_entry - 1) / device_bytes_per_entry;
					max_entry_count = static_cast<unsigned int>(std::max<size_t>(1, max_entry_count - std::min<size_t>(give_up, max_entry_count - 1)));
				}
			}

			if (debug->is_debug())
			{
				std::cout << "forward prop hip: " << p->plans.size() << " launches, " << p->buffer_floats_per_entry.size() << " buffers, "
					<< per_entry_bytes << " bytes per entry, max " << max_entry_count << " entries per packet" << std::endl;
				for(const forward_step& s : steps)
					std::cout << "  " << (s.fused ? "[fused] " : "        ") << s.description() << std::endl;
			}
		}

		namespace
		{
			// Whatever ends a run - the normal return or an exception from the reader, the writer or a launch -
			// nothing the run owns (device buffers, pinned staging, events) may be released while copies or
			// kernels that use it are still in flight: declared after them, this guard is destroyed first and waits.
			struct drain_streams
			{
				std::vector<void *> streams;
				~drain_streams()
				{
					for(void * s : streams)
						nnf_hip_stream_synchronize(s);
				}
			};
		}

		forward_propagation_hip::run_buffers& forward_propagation_hip::prepare_run(unsigned int packet, int slot_count, bool with_output_staging, bool stats_on_device,
			int staging_slot_count)
		{
			hip_config->set_device();
			if (staging_slot_count <= 0)
				staging_slot_count = slot_count;
			if (kept_run && (kept_run->packet == packet) && (kept_run->slot_count == slot_count) && (kept_run->staging_slot_count == staging_slot_count)
				&& (kept_run->with_output_staging == with_output_staging) && (kept_run->stats_on_device == stats_on_device))
				return *kept_run;
			kept_run.reset(); // what the run before held goes first: both sets need not fit side by side
			std::unique_ptr<run_buffers> fresh(new run_buffers());
			run_buffers& r = *fresh;
			r.packet = packet;
			r.slot_count = slot_count;
			r.staging_slot_count = staging_slot_count;
			r.buffers.resize(static_cast<size_t>(slot_count));
			r.staging.resize(static_cast<size_t>(staging_slot_count));
			r.with_output_staging = with_output_staging;
			r.stats_on_device = stats_on_device;
			unsigned int stream_count = 1;
			for(const forward_step& step : steps)
				stream_count = std::max(stream_count, step.stream_index + 1);
			p->create_streams(stream_count);
			for(const layer::const_ptr& l : p->exec_layers)
				if (!l->is_empty_data() && (p->weights.find(l->instance_name) == p->weights.end()))
					throw neural_network_exception("No data found with layer name " + l->instance_name);

			std::set<int> io_buffers;
			for(const std::string& n : data_layer_names)
				io_buffers.insert(p->value_to_buffer.at(n));
			for(const std::string& n : output_layer_names)
				io_buffers.insert(p->value_to_buffer.at(n));
			for(size_t b = 0; b < p->buffer_floats_per_entry.size(); ++b)
			{
				const size_t bytes = p->buffer_floats_per_entry[b] * sizeof(float) * packet;
				r.buffers[0].push_back(hip_linear_buffer_device::ptr(new hip_linear_buffer_device(bytes)));
				for(int s = 1; s < slot_count; ++s)
				{
					if (io_buffers.find(static_cast<int>(b)) != io_buffers.end())
						r.buffers[s].push_back(hip_linear_buffer_device::ptr(new hip_linear_buffer_device(bytes)));
					else
						r.buffers[s].push_back(r.buffers[0].back());
				}
			}
			for(const step_plan& plan : p->plans)
			{
				std::pair<hip_linear_buffer_device::ptr, hip_linear_buffer_device::ptr> t;
				if (!plan.info.fused && plan.tester)
				{
					const size_t fixed = plan.tester->get_temporary_working_fixed_buffer_size().first;
					const size_t per_entry = plan.tester->get_temporary_working_per_entry_buffer_size();
					if (fixed > 0)
						t.first.reset(new hip_linear_buffer_device(fixed));
					if (per_entry > 0)
						t.second.reset(new hip_linear_buffer_device(per_entry * packet * plan.entry_factor));
				}
				r.temporary.push_back(t);
			}
			r.chunk_ptrs.assign(p->plans.size(), std::vector<const float *>());
			for(size_t i = 0; i < p->plans.size(); ++i)
				for(const std::string& layer_name : p->plans[i].chunk_layers)
					for(const hip_linear_buffer_device::const_ptr& b : p->weights.at(layer_name))
						r.chunk_ptrs[i].push_back(static_cast<const float *>(*b));

			// pinned staging per I/O slot: the data layers, and the output layers unless only their statistics are wanted
			for(int s = 0; s < staging_slot_count; ++s)
			{
				for(const std::string& n : data_layer_names)
					r.staging[s][n].reset(new pinned_buffer(static_cast<size_t>(layer_config_map[n].get_neuron_count()) * sizeof(float) * packet));
				if (with_output_staging)
					for(const std::string& n : output_layer_names)
						if (r.staging[s].find(n) == r.staging[s].end())
							r.staging[s][n].reset(new pinned_buffer(static_cast<size_t>(layer_config_map[n].get_neuron_count()) * sizeof(float) * packet * output_layers_tiling_factor));
			}
			if (stats_on_device)
			{
				for(const std::string& n : output_layer_names)
				{
					const layer_configuration_specific& c = layer_config_map[n];
					r.stat_states[n].reset(new hip_linear_buffer_device(static_cast<size_t>(c.feature_map_count) * sizeof(nnf_hip_running_stat)));
					size_t bytes = 0;
					hip_safe_call(nnf_hip_feature_map_stat_workspace_bytes(packet * output_layers_tiling_factor, c.feature_map_count, c.get_neuron_count_per_feature_map(), &bytes));
					r.stat_workspaces[n].reset(new hip_linear_buffer_device(bytes));
					r.stat_workspace_bytes[n] = bytes;
				}
			}
			kept_run = std::move(fresh);
			return *kept_run;
		}

		// Packets of entries flow through in-order queues with two I/O slots (the double buffering
		// of nnforge/cuda/forward_propagation_cuda.cpp:84-112, 147-316):
		//   the job runner's threads read packet i into the pinned staging of slot i % 2, one job per entry
		//                                                                (needs: upload of packet i-2 done)
		//   meanwhile the calling thread hands packet i-1 to the writer  (needs: download i-1 done)
		//   upload stream copies packet i to the slot's device input buffers (needs: kernels of packet i-2 done)
		//   kernel streams run the launch plan                           (needs: upload i, download i-2, kernels i-1 done)
		//   download stream copies the slot's output buffers to staging  (needs: kernels i done)
		// Data and output layers have a device buffer per slot; everything in between is shared, which is
		// safe because the kernels of one packet start after those of the packet before.
		void forward_propagation_hip::actual_run(
			structured_data_bunch_reader& reader,
			structured_data_bunch_writer& writer,
			unsigned int& entries_processed,
			std::map<layer_name_with_action, float>& action_seconds,
			float& idle_seconds)
		{
			if (hip_config->is_offline())
				throw neural_network_exception("This forward_propagation_hip was created for planning only (offline configuration): it cannot run");

			unsigned int packet = max_entry_count;
			const int reader_entry_count = reader.get_entry_count();
			if (reader_entry_count > 0)
				packet = std::min(packet, static_cast<unsigned int>(reader_entry_count));

			// A statistics writer (nnforge/stat_data_bunch_writer.h) only wants per-feature-map figures of the
			// outputs: they are reduced where they lie, in device memory, and nothing but the running
			// states (32 bytes per feature map) travels to the host at the end of the run.
			stat_data_bunch_writer * stat_writer = dynamic_cast<stat_data_bunch_writer *>(&writer);
			const bool stats_on_device = (stat_writer != nullptr);

			// Entries that come from the host and go back to it pass through pinned staging, and what the host does
			// with them (reading, writing) bounds the run, not the kernels: packets are kept small enough for reading,
			// copying, computing and writing of neighbouring packets to overlap. Measured with BatchNorm -> ReLU on
			// 64 x 56 x 56 entries (0.8 MB in, 0.8 MB out per entry), 1024 entries: 12.6 GB/s of input + output with 51 MB of
			// staging per slot, 13.3 with 103 MB, 8.8 with 205 MB, 3.7 with all 1024 entries as one packet. The bound
			// (hip_max_io_staging_mb) never makes a packet smaller than a few entries: a network with many or large data
			// layers would otherwise run its launch plan entry by entry, where launches are what a pass costs.
			if (hip_config->max_io_staging_bytes > 0)
			{
				size_t io_bytes_per_entry = 0;
				for(const std::string& n : data_layer_names)
					io_bytes_per_entry += static_cast<size_t>(layer_config_map[n].get_neuron_count()) * sizeof(float);
				if (!stats_on_device)
					for(const std::string& n : output_layer_names)
						io_bytes_per_entry += static_cast<size_t>(layer_config_map[n].get_neuron_count()) * sizeof(float) * output_layers_tiling_factor;
				const size_t fit = hip_config->max_io_staging_bytes / std::max<size_t>(1, io_bytes_per_entry);
				const unsigned int floor_entries = std::min(packet, hip_running_configuration::min_packet_entries_under_staging_bound);
				packet = std::max(floor_entries, std::min(packet, static_cast<unsigned int>(std::min<size_t>(fit, 0xFFFFFFFFu))));
			}
			packet_entry_count = packet;

			constexpr int slot_count = 2;
			run_buffers& r = prepare_run(packet, slot_count, !stats_on_device, stats_on_device);
			std::vector<std::map<std::string, std::unique_ptr<pinned_buffer> > >& staging = r.staging;
			std::map<std::string, hip_linear_buffer_device::ptr>& stat_states = r.stat_states;
			std::map<std::string, hip_linear_buffer_device::ptr>& stat_workspaces = r.stat_workspaces;
			std::map<std::string, size_t>& stat_workspace_bytes = r.stat_workspace_bytes;
			if (stats_on_device)
				for(const std::string& n : output_layer_names)
					hip_safe_call(nnf_hip_feature_map_stat_init(p->stream, static_cast<nnf_hip_running_stat *>(static_cast<void *>(*stat_states[n])), layer_config_map[n].feature_map_count));
			hip_event upload_done[slot_count], kernels_done[slot_count], download_done[slot_count];
			bool slot_used[slot_count] = { false, false };

			const bool profiling = profile->is_profile();
			std::vector<std::unique_ptr<hip_event> > step_events[slot_count];
			if (profiling)
				for(int s = 0; s < slot_count; ++s)
					for(size_t i = 0; i <= p->plans.size(); ++i)
						step_events[s].emplace_back(new hip_event());

			unsigned int read_total = 0;
			double idle = 0.0;
			action_seconds.clear();

			// what is in flight: at most the packet before the current one
			struct in_flight
			{
				bool valid;
				int slot;
				unsigned int first_entry;
				unsigned int entries;
			} previous = { false, 0, 0, 0 };

			auto finish = [&](const in_flight& f)
			{
				hip_safe_call(nnf_hip_event_synchronize(download_done[f.slot].ev));
				if (profiling)
				{
					for(size_t i = 0; i < p->plans.size(); ++i)
					{
						float ms = 0.0F;
						hip_safe_call(nnf_hip_event_elapsed_ms(&ms, step_events[f.slot][i]->ev, step_events[f.slot][i + 1]->ev));
						action_seconds[p->plans[i].action] += ms * 1.0e-3F;
					}
				}
				// every entry the output layers hold goes to the writer, numbered in sequence
				// (nnforge/cuda/forward_propagation_cuda.cpp:271-278)
				for(unsigned int e = 0; (e < f.entries * output_layers_tiling_factor) && !stats_on_device; ++e)
				{
					std::map<std::string, const float *> data_map;
					for(const std::string& n : output_layer_names)
						data_map[n] = static_cast<const float *>(staging[f.slot][n]->ptr) + static_cast<size_t>(e) * layer_config_map[n].get_neuron_count();
					writer.write(f.first_entry * output_layers_tiling_factor + e, data_map);
				}
			};

			drain_streams drain_on_exit;
			drain_on_exit.streams = p->kernel_streams;
			drain_on_exit.streams.push_back(p->upload_stream);
			drain_on_exit.streams.push_back(p->download_stream);

			// Reading: one job per entry on the configuration's job runner, as the reference posts them
			// (nnforge/cuda/forward_propagation_cuda.cpp:190-245), while this thread hands the packet before to the
			// writer. A reader is therefore asked for different entries from different threads at the same time, and
			// for entries beyond its last one (it answers false, as to a sequential caller).
			struct packet_reads
			{
				std::mutex m;
				std::condition_variable done;
				unsigned int pending = 0;
				std::vector<char> entry_read;
				std::vector<std::exception_ptr> errors;
				void wait()
				{
					std::unique_lock<std::mutex> lock(m);
					done.wait(lock, [this]() { return pending == 0; });
				}
				// nothing the jobs use (the staging, this object, the reader) may go while one of them still runs
				~packet_reads() { wait(); }
			} reads;
			threadpool_job_runner::ptr job_runner = hip_config->get_job_runner();

			for(unsigned int packet_id = 0; ; ++packet_id)
			{
				const int slot = static_cast<int>(packet_id % slot_count);
				// the staging of this slot is free once its previous upload has finished; its output
				// staging was consumed when that packet was handed to the writer
				if (slot_used[slot])
					hip_safe_call(nnf_hip_event_synchronize(upload_done[slot].ev));

				unsigned int to_read = packet;
				if (reader_entry_count >= 0)
					to_read = std::min(packet, static_cast<unsigned int>(reader_entry_count) - std::min(read_total, static_cast<unsigned int>(reader_entry_count)));
				reads.entry_read.assign(to_read, 0);
				reads.errors.assign(to_read, std::exception_ptr());
				for(unsigned int i = 0; i < to_read; ++i)
				{
					// counted before it is posted and taken back if posting fails: the destructor of `reads` waits for
					// exactly the jobs that exist
					{
						std::lock_guard<std::mutex> lock(reads.m);
						++reads.pending;
					}
					struct uncount_unless_posted
					{
						packet_reads& reads;
						bool posted = false;
						~uncount_unless_posted()
						{
							if (!posted)
							{
								std::lock_guard<std::mutex> lock(reads.m);
								--reads.pending;
							}
						}
					} guard{reads};
					job_runner->post([this, &reads, &reader, &staging, slot, i, read_total]()
					{
						try
						{
							std::map<std::string, float *> data_map;
							for(const std::string& n : data_layer_names)
								data_map[n] = static_cast<float *>(staging[slot].at(n)->ptr) + static_cast<size_t>(i) * layer_config_map.at(n).get_neuron_count();
							reads.entry_read[i] = reader.read(read_total + i, data_map) ? 1 : 0;
						}
						catch (...)
						{
							reads.errors[i] = std::current_exception();
						}
						std::lock_guard<std::mutex> lock(reads.m);
						if (--reads.pending == 0)
							reads.done.notify_all();
					});
					guard.posted = true;
				}

				// while the entries are read, the packet before goes to the writer
				if (previous.valid)
				{
					finish(previous);
					previous.valid = false;
				}

				const std::chrono::high_resolution_clock::time_point wait_start = std::chrono::high_resolution_clock::now();
				reads.wait();
				idle += std::chrono::duration<double>(std::chrono::high_resolution_clock::now() - wait_start).count();
				unsigned int entries_read = 0;
				for(unsigned int i = 0; i < to_read; ++i)
				{
					// what a sequential caller would have met first comes first: an entry that could not be read ends the
					// data, an exception ends the run
					if (reads.errors[i])
						std::rethrow_exception(reads.errors[i]);
					if (!reads.entry_read[i])
						break;
					++entries_read;
				}

				if (entries_read > 0)
				{
					// upload: the slot's input buffers may still be read by the kernels of packet i-2, or by
					// its download when a layer worked in place on a data layer's buffer
					if (slot_used[slot])
					{
						hip_safe_call(nnf_hip_stream_wait_event(p->upload_stream, kernels_done[slot].ev));
						hip_safe_call(nnf_hip_stream_wait_event(p->upload_stream, download_done[slot].ev));
					}
					for(const std::string& n : data_layer_names)
						hip_safe_call(nnf_hip_memcpy_h2d(*r.buffers[slot][p->value_to_buffer[n]], staging[slot][n]->ptr,
							static_cast<size_t>(layer_config_map[n].get_neuron_count()) * sizeof(float) * entries_read, p->upload_stream));
					hip_safe_call(nnf_hip_event_record(upload_done[slot].ev, p->upload_stream));

					// kernels: need this packet's inputs and the slot's output buffers drained. The kernels of the
					// packet before need no wait: all steps that touch a buffer share a kernel stream, which
					// runs in order
					for(size_t ks = 0; ks < p->kernel_streams.size(); ++ks)
					{
						hip_safe_call(nnf_hip_stream_wait_event(p->kernel_streams[ks], upload_done[slot].ev));
						if (slot_used[slot])
							hip_safe_call(nnf_hip_stream_wait_event(p->kernel_streams[ks], download_done[slot].ev));
					}
					p->enqueue_plan(r.buffers[slot], entries_read, r.chunk_ptrs, r.temporary, profiling ? &step_events[slot] : nullptr);
					if (stats_on_device)
					{
						for(const std::string& n : output_layer_names)
						{
							const layer_configuration_specific& c = layer_config_map[n];
							hip_safe_call(nnf_hip_feature_map_stat_accumulate(p->stream,
								static_cast<nnf_hip_running_stat *>(static_cast<void *>(*stat_states[n])), *stat_workspaces[n], stat_workspace_bytes[n],
								static_cast<const float *>(static_cast<const void *>(*r.buffers[slot][p->value_to_buffer.at(n)])),
								entries_read * output_layers_tiling_factor, c.feature_map_count, c.get_neuron_count_per_feature_map()));
						}
					}
					hip_safe_call(nnf_hip_event_record(kernels_done[slot].ev, p->stream));

					// download
					hip_safe_call(nnf_hip_stream_wait_event(p->download_stream, kernels_done[slot].ev));
					for(const std::string& n : output_layer_names)
						if (!stats_on_device)
						hip_safe_call(nnf_hip_memcpy_d2h(staging[slot][n]->ptr, *r.buffers[slot][p->value_to_buffer.at(n)],
							static_cast<size_t>(layer_config_map[n].get_neuron_count()) * sizeof(float) * entries_read * output_layers_tiling_factor, p->download_stream));
					hip_safe_call(nnf_hip_event_record(download_done[slot].ev, p->download_stream));
					slot_used[slot] = true;
				}

				previous.valid = entries_read > 0;
				previous.slot = slot;
				previous.first_entry = read_total;
				previous.entries = entries_read;
				read_total += entries_read;
				if (entries_read < packet)
					break;
			}
			if (previous.valid)
				finish(previous);
			hip_safe_call(nnf_hip_stream_synchronize(p->stream));

			if (stats_on_device)
			{
				static_assert(sizeof(stat_data_bunch_writer::running_stat) == sizeof(nnf_hip_running_stat), "running state layouts differ");
				for(const std::string& n : output_layer_names)
				{
					std::vector<stat_data_bunch_writer::running_stat> states(layer_config_map[n].feature_map_count);
					hip_safe_call(nnf_hip_memcpy_d2h(states.data(), *stat_states[n], states.size() * sizeof(nnf_hip_running_stat), nullptr));
					stat_writer->merge(n, states);
				}
				stat_writer->add_entries(read_total * output_layers_tiling_factor);
			}

			entries_processed = read_total;
			idle_seconds = static_cast<float>(idle);
		}

		forward_propagation_hip::kernel_timing forward_propagation_hip::time_kernels(
			structured_data_bunch_reader& reader, unsigned int entry_count, unsigned int warmup, unsigned int passes, unsigned int resident_packets,
			bool replay_recorded_plan)
		{
			if (hip_config->is_offline())
				throw neural_network_exception("This forward_propagation_hip was created for planning only (offline configuration): it cannot run");
			set_input_configuration_specific(reader.get_config_map());
			const unsigned int packet = std::min(std::max(1U, entry_count), max_entry_count);
			const int slot_count = static_cast<int>(std::max(1U, std::min(resident_packets, 64U)));
			run_buffers& r = prepare_run(packet, slot_count, false, false, 1);
			// recordings of the plan, released after the streams have drained (declared first, destroyed last)
			struct recorded_plans
			{
				std::vector<void *> graphs;
				~recorded_plans()
				{
					for(void * g : graphs)
						nnf_hip_graph_destroy(g);
				}
			} recorded;
			drain_streams drain_on_exit;
			drain_on_exit.streams = p->kernel_streams;

			// one packet, read once and uploaded to every slot
			unsigned int entries_read = 0;
			{
				std::map<std::string, std::unique_ptr<pinned_buffer> >& staging = r.staging[0];
				for(; entries_read < packet; ++entries_read)
				{
					std::map<std::string, float *> data_map;
					for(const std::string& n : data_layer_names)
						data_map[n] = static_cast<float *>(staging[n]->ptr) + static_cast<size_t>(entries_read) * layer_config_map[n].get_neuron_count();
					if (!reader.read(entries_read, data_map))
						break;
				}
				if (entries_read == 0)
					throw neural_network_exception("time_kernels: the reader holds no entries");
				for(int slot = 0; slot < slot_count; ++slot)
					for(const std::string& n : data_layer_names)
						hip_safe_call(nnf_hip_memcpy_h2d(*r.buffers[slot][p->value_to_buffer[n]], staging[n]->ptr,
							static_cast<size_t>(layer_config_map[n].get_neuron_count()) * sizeof(float) * entries_read, nullptr));
			}

			hip_event start, stop;
			// A pass after a pass needs no wait between them: all steps that touch a buffer share a kernel stream,
			// which runs in order. (Every pass still ends with the main stream waiting for the others, as a packet does.)
			unsigned int pass_id = 0;
			auto one_pass = [&]()
			{
				const unsigned int slot = pass_id % static_cast<unsigned int>(slot_count);
				if (!recorded.graphs.empty())
					hip_safe_call(nnf_hip_graph_launch(recorded.graphs[slot], p->stream));
				else
					p->enqueue_plan(r.buffers[slot], entries_read, r.chunk_ptrs, r.temporary, nullptr);
				++pass_id;
			};
			hip_safe_call(nnf_hip_device_synchronize());
			kernel_timing res;
			res.entry_count = entries_read;
			res.resident_packets = static_cast<unsigned int>(slot_count);
			res.plan_step_count = 0;
			for(const step_plan& plan : p->plans)
				res.plan_step_count += plan.launches_nothing() ? 0 : 1;
			// what a pass launches: the kernels the library starts from this thread while one pass is enqueued
			uint64_t launches_before = 0, launches_after = 0;
			hip_safe_call(nnf_hip_launch_count(&launches_before));
			one_pass();
			hip_safe_call(nnf_hip_launch_count(&launches_after));
			res.launch_count = static_cast<unsigned int>(launches_after - launches_before);
			if (replay_recorded_plan)
			{
				if (p->kernel_streams.size() != 1)
					throw neural_network_exception("time_kernels: a recorded plan takes one kernel stream");
				hip_safe_call(nnf_hip_device_synchronize());
				for(int slot = 0; slot < slot_count; ++slot)
				{
					hip_safe_call(nnf_hip_stream_begin_capture(p->stream));
					p->enqueue_plan(r.buffers[slot], entries_read, r.chunk_ptrs, r.temporary, nullptr);
					void * graph = nullptr;
					hip_safe_call(nnf_hip_stream_end_capture(p->stream, &graph));
					recorded.graphs.push_back(graph);
				}
			}
			for(unsigned int i = 0; i < warmup; ++i)
				one_pass();
			hip_safe_call(nnf_hip_device_synchronize());

			const std::chrono::high_resolution_clock::time_point t0 = std::chrono::high_resolution_clock::now();
			hip_safe_call(nnf_hip_event_record(start.ev, p->stream));
			for(size_t ks = 1; ks < p->kernel_streams.size(); ++ks)
				hip_safe_call(nnf_hip_stream_wait_event(p->kernel_streams[ks], start.ev));
			for(unsigned int i = 0; i < passes; ++i)
				one_pass();
			hip_safe_call(nnf_hip_event_record(stop.ev, p->stream));
			const std::chrono::duration<float> enqueued = std::chrono::high_resolution_clock::now() - t0;
			hip_safe_call(nnf_hip_device_synchronize());
			const std::chrono::duration<float> wall = std::chrono::high_resolution_clock::now() - t0;
			float ms = 0.0F;
			hip_safe_call(nnf_hip_event_elapsed_ms(&ms, start.ev, stop.ev));
			const float n = static_cast<float>(std::max(1U, passes));
			res.wall_seconds_per_pass = wall.count() / n;
			res.device_seconds_per_pass = ms * 1.0e-3F / n;
			res.host_seconds_per_pass = enqueued.count() / n;
			return res;
		}

		float forward_propagation_hip::get_max_bytes_per_second() const
		{
			return 8.0e12F; // MI355X HBM3E peak
		}

		// ---- factories -------------------------------------------------------------------------

		forward_propagation::ptr forward_propagation_hip_factory::create(
			const network_schema& schema,
			const std::vector<std::string>& output_layer_names,
			debug_state::ptr debug,
			profile_state::ptr profile) const
		{
			return forward_propagation::ptr(new forward_propagation_hip(schema, output_layer_names, debug, profile, hip_config));
		}

		factory_generator_hip::factory_generator_hip()
			: hip_device_id(0)
			, hip_max_global_memory_usage_ratio(0.9F)
			, hip_fuse(true)
			, hip_dont_share_buffers(false)
			, hip_single_command_stream(false)
			, hip_batch_independent_groups(true)
			, hip_kernel_stream_count(hip_running_configuration::default_kernel_stream_count)
			, hip_max_entry_count(4096)
			, hip_reserved_thread_count(1)
			, hip_max_io_staging_mb(64)
			, hip_concat_in_place(true)
		{
		}

		void factory_generator_hip::initialize()
		{
			hip::init();
			std::shared_ptr<hip_running_configuration> config(new hip_running_configuration(
				hip_device_id, hip_max_global_memory_usage_ratio, hip_fuse, hip_dont_share_buffers, hip_max_entry_count,
				hip_single_command_stream ? 1 : std::max(1, hip_kernel_stream_count), hip_batch_independent_groups,
				static_cast<unsigned int>(std::max(0, hip_reserved_thread_count))));
			config->max_io_staging_bytes = static_cast<size_t>(std::max(0, hip_max_io_staging_mb)) << 20;
			config->concat_in_place = hip_concat_in_place;
			hip_config = config;
		}

		forward_propagation_factory::ptr factory_generator_hip::create_forward_propagation_factory() const
		{
			if (!hip_config)
				throw neural_network_exception("factory_generator_hip::initialize() has not been called");
			return forward_propagation_factory::ptr(new forward_propagation_hip_factory(hip_config));
		}

		backward_propagation_factory::ptr factory_generator_hip::create_backward_propagation_factory() const
		{
			throw neural_network_exception("The hip backend implements inference only: backward propagation is not supported");
		}

		void factory_generator_hip::info() const
		{
			if (hip_config)
				std::cout << *hip_config;
		}

		std::vector<bool_option> factory_generator_hip::get_bool_options()
		{
			std::vector<bool_option> res;
			res.push_back(bool_option("hip_fuse", &hip_fuse, true, "Fuse runs of element-wise layers (BatchNorm, activations, Add) into single kernel launches"));
			res.push_back(bool_option("hip_dont_share_buffers", &hip_dont_share_buffers, false, "Don't share buffers between layers. Switch it on if you suspect a bug in there"));
			res.push_back(bool_option("hip_single_command_stream", &hip_single_command_stream, false, "Use single stream for kernels. Switch it on if you suspect a bug in there"));
			res.push_back(bool_option("hip_concat_in_place", &hip_concat_in_place, true, "Fused groups that only a Concat layer reads write their results into its output instead of having them copied there"));
			res.push_back(bool_option("hip_batch_independent_groups", &hip_batch_independent_groups, true, "Launch consecutive fused groups that do not depend on each other together (takes one kernel stream)"));
			return res;
		}

		std::vector<float_option> factory_generator_hip::get_float_options()
		{
			std::vector<float_option> res;
			res.push_back(float_option("hip_max_global_memory_usage_ratio,G", &hip_max_global_memory_usage_ratio, 0.9F, "Part of the global memory to be used by the backend"));
			return res;
		}

		std::vector<int_option> factory_generator_hip::get_int_options()
		{
			std::vector<int_option> res;
			res.push_back(int_option("hip_device_id,D", &hip_device_id, 0, "HIP device ID"));
			res.push_back(int_option("hip_max_entry_count", &hip_max_entry_count, 4096, "Upper bound of entries processed per packet"));
			res.push_back(int_option("hip_kernel_stream_count", &hip_kernel_stream_count, hip_running_configuration::default_kernel_stream_count, "Streams the kernels of independent layers are spread over"));
			res.push_back(int_option("hip_reserved_thread_count", &hip_reserved_thread_count, 1, "The number of hw threads not used for input data processing"));
			res.push_back(int_option("hip_max_io_staging_mb", &hip_max_io_staging_mb, 64, "Pinned staging per I/O slot, in MB, that bounds the entries of a packet (0: no bound)"));
			return res;
		}
	}
}
