#include "nnforge_hip/schema.h"
#include "nnforge_hip/layers.h"

#include <algorithm>
#include <cctype>
#include <cstring>
#include <dirent.h>
#include <fstream>
#include <sstream>
#include <sys/stat.h>

namespace nnforge
{
	namespace
	{
		// ---- tokenizer / parser of the protobuf text format subset ----------------------------
		// message := (field)* ; field := name ':' scalar | name [':'] '{' message '}'
		// scalar := "string" | bare token (numbers, true/false, enum names). '#' starts a comment.
		struct token
		{
			enum kind_t { end, name, string_literal, colon, open_brace, close_brace } kind;
			std::string text;
			int line;
		};

		class tokenizer
		{
		public:
			explicit tokenizer(std::istream& in) : in(in), line(1) {}

			token next()
			{
				skip_space_and_comments();
				token t;
				t.line = line;
				const int c = in.get();
				if (c == EOF)
				{
					t.kind = token::end;
					return t;
				}
				if (c == ':') { t.kind = token::colon; return t; }
				if ((c == '{') || (c == '<')) { t.kind = token::open_brace; return t; }
				if ((c == '}') || (c == '>')) { t.kind = token::close_brace; return t; }
				if ((c == '"') || (c == '\''))
				{
					t.kind = token::string_literal;
					for(;;)
					{
						const int d = in.get();
						if (d == EOF)
							throw neural_network_exception("Unterminated string in schema at line " + std::to_string(t.line));
						if (d == c)
							break;
						if (d == '\\')
						{
							const int e = in.get();
							if (e == 'n') t.text.push_back('\n');
							else if (e == 't') t.text.push_back('\t');
							else if (e != EOF) t.text.push_back(static_cast<char>(e));
							continue;
						}
						if (d == '\n')
							++line;
						t.text.push_back(static_cast<char>(d));
					}
					return t;
				}
				t.kind = token::name;
				t.text.push_back(static_cast<char>(c));
				for(;;)
				{
					const int d = in.peek();
					if ((d == EOF) || std::isspace(d) || (d == ':') || (d == '{') || (d == '}') || (d == '<') || (d == '>') || (d == '"') || (d == '#') || (d == ',') || (d == ';'))
						break;
					t.text.push_back(static_cast<char>(in.get()));
				}
				return t;
			}

		private:
			void skip_space_and_comments()
			{
				for(;;)
				{
					const int c = in.peek();
					if (c == EOF)
						return;
					if (c == '\n') { ++line; in.get(); continue; }
					if (std::isspace(c) || (c == ',') || (c == ';')) { in.get(); continue; }
					if (c == '#')
					{
						while ((in.peek() != EOF) && (in.peek() != '\n'))
							in.get();
						continue;
					}
					return;
				}
			}

			std::istream& in;
			int line;
		};

		// parses fields until the closing brace (or end of input at top level)
		void parse_message(tokenizer& tk, schema_param_block& block, bool top_level)
		{
			for(;;)
			{
				token t = tk.next();
				if (t.kind == token::end)
				{
					if (!top_level)
						throw neural_network_exception("Unexpected end of schema: missing '}'");
					return;
				}
				if (t.kind == token::close_brace)
				{
					if (top_level)
						throw neural_network_exception("Unexpected '}' in schema at line " + std::to_string(t.line));
					return;
				}
				if (t.kind != token::name)
					throw neural_network_exception("Field name expected in schema at line " + std::to_string(t.line));
				const std::string field = t.text;
				token v = tk.next();
				if (v.kind == token::colon)
					v = tk.next();
				if (v.kind == token::open_brace)
				{
					block.blocks.push_back(std::make_pair(field, schema_param_block()));
					parse_message(tk, block.blocks.back().second, false);
				}
				else if ((v.kind == token::name) || (v.kind == token::string_literal))
				{
					if (field == "input_layer_name") // the only repeated scalar: keep every occurrence, in order
					{
						block.blocks.push_back(std::make_pair(field, schema_param_block()));
						block.blocks.back().second.scalars["value"] = v.text;
					}
					else
					{
						block.set(field, v.text);
						if (v.kind == token::string_literal)
							block.quoted.insert(field);
					}
				}
				else
					throw neural_network_exception("Value expected for field " + field + " in schema at line " + std::to_string(v.line));
			}
		}

		const unsigned char data_guid[16] = { 0xd1, 0x19, 0x35, 0xb5, 0x30, 0x59, 0x49, 0xe2, 0x9c, 0x33, 0x1c, 0x43, 0x22, 0xf8, 0x13, 0x0d };

		bool ends_with(const std::string& s, const std::string& suffix)
		{
			return (s.size() >= suffix.size()) && (s.compare(s.size() - suffix.size(), suffix.size(), suffix) == 0);
		}
	}

	// ---- network_schema --------------------------------------------------------------------

	network_schema::network_schema(const std::vector<layer::const_ptr>& layer_list)
	{
		rebuild(layer_list);
	}

	void network_schema::rebuild(const std::vector<layer::const_ptr>& layer_list)
	{
		std::map<std::string, size_t> by_name;
		for(size_t i = 0; i < layer_list.size(); ++i)
		{
			if (layer_list[i]->instance_name.empty())
				throw neural_network_exception("Layer of type " + layer_list[i]->get_type_name() + " has no name");
			if (!by_name.insert(std::make_pair(layer_list[i]->instance_name, i)).second)
				throw neural_network_exception("Duplicate layer name " + layer_list[i]->instance_name + " in schema");
		}
		for(const layer::const_ptr& l : layer_list)
		{
			for(const std::string& input : l->input_layer_instance_names)
				if (by_name.find(input) == by_name.end())
					throw neural_network_exception("Layer " + l->instance_name + " has unknown input layer " + input);
		}

		// topological order, stable with respect to the given order
		std::vector<int> state(layer_list.size(), 0); // 0 new, 1 on the stack, 2 done
		std::vector<layer::const_ptr> ordered;
		std::vector<std::pair<size_t, size_t> > stack;
		for(size_t root = 0; root < layer_list.size(); ++root)
		{
			if (state[root] != 0)
				continue;
			stack.push_back(std::make_pair(root, static_cast<size_t>(0)));
			state[root] = 1;
			while (!stack.empty())
			{
				const size_t cur = stack.back().first;
				const std::vector<std::string>& inputs = layer_list[cur]->input_layer_instance_names;
				if (stack.back().second < inputs.size())
				{
					const size_t next = by_name[inputs[stack.back().second++]];
					if (state[next] == 1)
						throw neural_network_exception("Schema has a cycle through layer " + layer_list[next]->instance_name);
					if (state[next] == 0)
					{
						state[next] = 1;
						stack.push_back(std::make_pair(next, static_cast<size_t>(0)));
					}
				}
				else
				{
					state[cur] = 2;
					ordered.push_back(layer_list[cur]);
					stack.pop_back();
				}
			}
		}

		layers = ordered;
		name_to_index.clear();
		for(size_t i = 0; i < layers.size(); ++i)
			name_to_index[layers[i]->instance_name] = i;
	}

	void network_schema::read_proto(std::istream& stream_to_read_from, bool keep_unregistered_layers)
	{
		tokenizer tk(stream_to_read_from);
		schema_param_block root;
		parse_message(tk, root, true);

		name = root.has("name") ? root.scalars["name"] : std::string();
		std::vector<layer::const_ptr> layer_list;
		for(const schema_param_block * lb : root.children("layer"))
		{
			if (!lb->has("type"))
				throw neural_network_exception("Layer without type in schema");
			if (!lb->has("name"))
				throw neural_network_exception("Layer without name in schema");
			const std::string type = lb->scalars.find("type")->second;
			layer::ptr l = (keep_unregistered_layers && !layer_factory::get_singleton().is_registered(type))
				? layer::ptr(new external_layer(type)) : layer_factory::get_singleton().create_layer(type);
			l->instance_name = lb->scalars.find("name")->second;
			for(const schema_param_block * in : lb->children("input_layer_name"))
				l->input_layer_instance_names.push_back(in->scalars.find("value")->second);
			l->read_proto(lb);
			layer_list.push_back(l);
		}
		rebuild(layer_list);
	}

	namespace
	{
		// a scalar as the text format wants it: strings (what a reader found in quotes) in quotes again
		std::string scalar_text(const schema_param_block& block, const std::string& key)
		{
			const std::string& value = block.scalars.find(key)->second;
			return (block.quoted.find(key) != block.quoted.end()) ? "\"" + value + "\"" : value;
		}

		void write_inline(std::ostream& out, const schema_param_block& block)
		{
			for(const std::string& key : block.scalar_order)
				out << key << ": " << scalar_text(block, key) << " ";
			for(const std::pair<std::string, schema_param_block>& nested : block.blocks)
			{
				out << nested.first << " { ";
				write_inline(out, nested.second);
				out << "} ";
			}
		}

		// the fields of a message a layer wrote: nested messages first (a line each), then the scalars, as the
		// files this backend has always written
		void write_fields(std::ostream& out, const schema_param_block& block, const std::string& indent)
		{
			for(const std::pair<std::string, schema_param_block>& nested : block.blocks)
			{
				out << indent << nested.first << " { ";
				write_inline(out, nested.second);
				out << "}\n";
			}
			for(const std::string& key : block.scalar_order)
				out << indent << key << ": " << scalar_text(block, key) << "\n";
		}
	}

	void network_schema::write_proto(std::ostream& out) const
	{
		if (!name.empty())
			out << "name: \"" << name << "\"\n";
		for(const layer::const_ptr& l : layers)
		{
			out << "layer {\n";
			out << "\ttype: \"" << l->get_type_name() << "\"\n";
			out << "\tname: \"" << l->instance_name << "\"\n";
			for(const std::string& input : l->input_layer_instance_names)
				out << "\tinput_layer_name: \"" << input << "\"\n";
			// the layer adds its "<type>_param" message (if it has anything to say); nested messages of that go on one line
			schema_param_block message;
			l->write_proto(&message);
			for(const std::pair<std::string, schema_param_block>& param : message.blocks)
			{
				out << "\t" << param.first << " {\n";
				write_fields(out, param.second, "\t\t");
				out << "\t}\n";
			}
			out << "}\n";
		}
	}

	std::vector<layer::const_ptr> network_schema::get_required_layers(const std::vector<std::string>& output_layer_names) const
	{
		std::vector<bool> needed(layers.size(), false);
		std::vector<size_t> todo;
		for(const std::string& n : output_layer_names)
		{
			std::map<std::string, size_t>::const_iterator it = name_to_index.find(n);
			if (it == name_to_index.end())
				throw neural_network_exception("Layer not found: " + n);
			todo.push_back(it->second);
		}
		while (!todo.empty())
		{
			const size_t cur = todo.back();
			todo.pop_back();
			if (needed[cur])
				continue;
			needed[cur] = true;
			if (dynamic_cast<const external_layer *>(layers[cur].get()) != nullptr)
				continue; // its output comes from outside
			for(const std::string& input : layers[cur]->input_layer_instance_names)
				todo.push_back(name_to_index.find(input)->second);
		}
		std::vector<layer::const_ptr> res;
		for(size_t i = 0; i < layers.size(); ++i)
		{
			if (!needed[i])
				continue;
			if ((dynamic_cast<const external_layer *>(layers[i].get()) != nullptr) && !layers[i]->input_layer_instance_names.empty())
			{
				layer::ptr source = layers[i]->clone();
				source->input_layer_instance_names.clear();
				res.push_back(source);
			}
			else
				res.push_back(layers[i]);
		}
		return res;
	}

	bool network_schema::has_external_layers() const
	{
		for(const layer::const_ptr& l : layers)
			if (dynamic_cast<const external_layer *>(l.get()) != nullptr)
				return true;
		return false;
	}

	std::vector<layer::const_ptr> network_schema::get_data_layers() const
	{
		std::vector<layer::const_ptr> res;
		for(const layer::const_ptr& l : layers)
			if (l->input_layer_instance_names.empty())
				res.push_back(l);
		return res;
	}

	std::vector<layer::const_ptr> network_schema::get_layers_in_forward_propagation_order() const
	{
		return layers;
	}

	std::map<std::string, layer_configuration_specific> network_schema::get_layer_configuration_specific_map(
		const std::map<std::string, layer_configuration_specific>& input_configuration_specific_map) const
	{
		std::map<std::string, layer_configuration_specific> res;
		for(const layer::const_ptr& l : layers)
		{
			if (l->input_layer_instance_names.empty())
			{
				std::map<std::string, layer_configuration_specific>::const_iterator it = input_configuration_specific_map.find(l->instance_name);
				if (it == input_configuration_specific_map.end())
					throw neural_network_exception("No input configuration supplied for data layer " + l->instance_name);
				res[l->instance_name] = it->second;
				continue;
			}
			std::vector<layer_configuration_specific> inputs;
			for(const std::string& input : l->input_layer_instance_names)
				inputs.push_back(res[input]);
			res[l->instance_name] = l->get_output_layer_configuration_specific(inputs);
		}
		return res;
	}

	std::map<std::string, unsigned int> network_schema::get_cumulative_tiling_factor_map() const
	{
		std::map<std::string, unsigned int> res;
		for(const layer::const_ptr& l : layers)
		{
			if (l->input_layer_instance_names.empty())
			{
				res[l->instance_name] = 1;
				continue;
			}
			const unsigned int input_factor = res.at(l->input_layer_instance_names[0]);
			for(const std::string& input : l->input_layer_instance_names)
				if (res.at(input) != input_factor)
					throw neural_network_exception("Tiling factors mismatch for inputs of layer " + l->instance_name + ": "
						+ std::to_string(input_factor) + " and " + std::to_string(res.at(input)));
			// the conversion throws when the layer would leave a fraction of an entry
			res[l->instance_name] = static_cast<unsigned int>(tiling_factor(input_factor) * l->get_tiling_factor());
		}
		return res;
	}

	unsigned int network_schema::get_consumer_count(const std::string& instance_name) const
	{
		unsigned int count = 0;
		for(const layer::const_ptr& l : layers)
			for(const std::string& input : l->input_layer_instance_names)
				if (input == instance_name)
					++count;
		return count;
	}

	layer::const_ptr network_schema::find_layer(const std::string& instance_name) const
	{
		std::map<std::string, size_t>::const_iterator it = name_to_index.find(instance_name);
		return (it == name_to_index.end()) ? layer::const_ptr() : layers[it->second];
	}

	layer::const_ptr network_schema::get_layer(const std::string& instance_name) const
	{
		layer::const_ptr res = find_layer(instance_name);
		if (!res)
			throw neural_network_exception("Layer not found: " + instance_name);
		return res;
	}

	// ---- network_data ----------------------------------------------------------------------

	network_data::network_data(const std::vector<layer::const_ptr>& layer_list, float val)
	{
		for(const layer::const_ptr& l : layer_list)
		{
			layer_data::ptr data = l->create_layer_data();
			if (!data->empty())
			{
				data->fill(val);
				data_list[l->instance_name] = data;
			}
			layer_data_custom::ptr custom = l->create_layer_data_custom();
			if (!custom->empty())
				data_custom_list[l->instance_name] = custom;
		}
	}

	network_data::network_data(const std::vector<layer::const_ptr>& layer_list, const network_data& other)
	{
		for(const layer::const_ptr& l : layer_list)
		{
			if (!l->is_empty_data())
				data_list[l->instance_name] = other.get(l->instance_name);
			if (!l->is_empty_data_custom())
			{
				std::map<std::string, layer_data_custom::ptr>::const_iterator it = other.data_custom_list.find(l->instance_name);
				if (it == other.data_custom_list.end())
					throw neural_network_exception("No custom data found with layer name " + l->instance_name);
				data_custom_list[l->instance_name] = it->second;
			}
		}
	}

	void network_data::check_network_data_consistency(const std::vector<layer::const_ptr>& layer_list) const
	{
		for(const layer::const_ptr& l : layer_list)
		{
			if (!l->is_empty_data())
				l->check_layer_data_consistency(*get(l->instance_name));
		}
	}

	void network_data::initialize(const std::vector<layer::const_ptr>& layer_list)
	{
		for(const layer::const_ptr& l : layer_list)
		{
			layer_data::ptr d = find(l->instance_name);
			if (d)
				l->initialize_data(*d);
		}
	}

	void network_data::write(const std::string& folder_path) const
	{
		::mkdir(folder_path.c_str(), 0777);
		for(const std::pair<const std::string, layer_data::ptr>& item : data_list)
		{
			const std::string file_path = folder_path + "/" + item.first + ".data";
			std::ofstream out(file_path.c_str(), std::ios_base::out | std::ios_base::binary | std::ios_base::trunc);
			if (!out)
				throw neural_network_exception("Cannot open " + file_path + " for writing");
			out.write(reinterpret_cast<const char *>(data_guid), sizeof(data_guid));
			item.second->write(out);
		}
	}

	void network_data::read(const std::string& folder_path)
	{
		data_list.clear();
		DIR * dir = ::opendir(folder_path.c_str());
		if (dir == nullptr)
			throw neural_network_exception("Directory " + folder_path + " doesn't exist");
		std::vector<std::string> names;
		while (struct dirent * entry = ::readdir(dir))
		{
			const std::string file_name = entry->d_name;
			if (ends_with(file_name, ".data") && (file_name.size() > 5))
				names.push_back(file_name);
		}
		::closedir(dir);
		std::sort(names.begin(), names.end());
		for(const std::string& file_name : names)
		{
			const std::string file_path = folder_path + "/" + file_name;
			std::ifstream in(file_path.c_str(), std::ios_base::in | std::ios_base::binary);
			if (!in)
				throw neural_network_exception("Cannot open " + file_path);
			unsigned char guid[16];
			in.read(reinterpret_cast<char *>(guid), sizeof(guid));
			if (!in || (std::memcmp(guid, data_guid, sizeof(guid)) != 0))
				throw neural_network_exception("Unknown data GUID encountered in " + file_path);
			layer_data::ptr data(new layer_data());
			data->read(in);
			data_list[file_name.substr(0, file_name.size() - 5)] = data;
		}
	}

	layer_data::ptr network_data::find(const std::string& instance_name) const
	{
		std::map<std::string, layer_data::ptr>::const_iterator it = data_list.find(instance_name);
		return (it == data_list.end()) ? layer_data::ptr() : it->second;
	}

	layer_data_custom::ptr network_data::find_custom(const std::string& instance_name) const
	{
		std::map<std::string, layer_data_custom::ptr>::const_iterator it = data_custom_list.find(instance_name);
		return (it == data_custom_list.end()) ? layer_data_custom::ptr() : it->second;
	}

	layer_data::ptr network_data::get(const std::string& instance_name) const
	{
		layer_data::ptr res = find(instance_name);
		if (!res)
			throw neural_network_exception("No data found with layer name " + instance_name);
		return res;
	}

	void network_data::add(const std::string& instance_name, layer_data::ptr data)
	{
		data_list[instance_name] = data;
	}
}
