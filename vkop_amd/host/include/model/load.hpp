// Reader of the `.vkopbin` model file (model/load.hpp:18-67 for the types,
// model/load.cpp:98-285 for the order of the sections, writer
// model/pypi/onnx2vkop/dag.py:102-217).  Header only.
//
// Same types and field names as the reference's vkop::load, so code written
// against VkModel reads a model the same way.  Differences, on purpose:
//   * every length in the file is checked against the end of the file before it
//     is used (the reference trusts the attribute tag byte and the initializer
//     byte counts); a short or malformed file throws std::runtime_error naming
//     the field;
//   * the file is read into memory instead of mapped;
//   * nothing is printed while loading.
// Attribute values keep the reference's textual form (std::to_string of the
// number, lists as "[a, b]"): operators parse their attributes from text.
#ifndef VKOP_HIP_MODEL_LOAD_HPP_
#define VKOP_HIP_MODEL_LOAD_HPP_

#include <cstdint>
#include <cstring>
#include <fstream>
#include <iostream>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <unordered_set>
#include <vector>

namespace vkop {
namespace load {

struct Shape {
    std::string name;
    std::vector<uint32_t> dims;
};

struct Node {
    std::string op_type;
    std::string name;
    std::unordered_map<std::string, std::string> attributes;
    std::vector<Shape> inputs;
    std::vector<Shape> outputs;
    std::unordered_set<std::string> dependencies;
    std::unordered_set<std::string> dependents;
};

struct Initializer {
    std::string name;
    std::string dtype;
    std::vector<uint32_t> dims;
};

// One record of the "unified_metadata" / "rgba_conversion_metadata" tables (model/load.hpp:40-54).
struct PackedTensorRecord {
    int dtype;
    int name_len;
    int offset;
    int size;
    int dims[4];
};
using UnifiedMetadata = PackedTensorRecord;
using RGBAConversion = PackedTensorRecord;

class VkModel {
  public:
    std::vector<Shape> inputs;
    std::vector<Shape> outputs;
    std::vector<Node> nodes;
    std::unordered_map<std::string, Initializer> initializers;
    bool rgba = false;
    bool unified = false;
    std::unordered_map<std::string, size_t> initializer_offsets;  // into initializer_memory, 64-byte aligned
    std::unordered_map<std::string, size_t> initializer_bytes;
    std::vector<uint8_t> initializer_memory;
    std::vector<std::vector<std::string>> concurrent_execution_levels;

    explicit VkModel(const std::string &file_path) {
        std::ifstream f(file_path, std::ios::binary | std::ios::ate);
        if (!f) throw std::runtime_error("Failed to open file: " + file_path);
        const std::streamoff size = f.tellg();
        std::vector<uint8_t> bytes(static_cast<size_t>(size));
        f.seekg(0);
        if (size > 0 && !f.read(reinterpret_cast<char *>(bytes.data()), size))
            throw std::runtime_error("Failed to read file: " + file_path);
        parse(bytes.data(), bytes.size());
    }
    VkModel(const uint8_t *data, size_t size) { parse(data, size); }

    const std::vector<std::vector<std::string>> &getConcurrentExecutionLevels() const { return concurrent_execution_levels; }

    const uint8_t *initializer_data(const std::string &name) const {
        return initializer_memory.data() + initializer_offsets.at(name);
    }
    // The same, after checking that the initializer's data holds what its dimensions
    // promise (product of dims elements of elem_size bytes); throws if it is shorter.
    const uint8_t *initializer_data(const std::string &name, size_t elem_size) const {
        const auto &init = initializers.at(name);
        uint64_t elems = 1;
        for (uint32_t d : init.dims) {
            elems *= d;
            if (elems > (1ull << 40)) throw std::runtime_error("Initializer " + name + ": dimensions too large");
        }
        if (elems * elem_size > initializer_bytes.at(name))
            throw std::runtime_error("Initializer " + name + ": " + std::to_string(initializer_bytes.at(name)) + " bytes of data for " +
                                     std::to_string(elems) + " elements of " + std::to_string(elem_size) + " bytes");
        return initializer_data(name);
    }

    void dump_model(std::ostream &os = std::cout) const {
        auto shapes = [&os](const char *title, const std::vector<Shape> &list) {
            os << title;
            for (const auto &s : list) {
                os << " " << s.name << "[";
                for (size_t i = 0; i < s.dims.size(); ++i) os << (i ? "," : "") << s.dims[i];
                os << "]";
            }
            os << "\n";
        };
        shapes("Inputs:", inputs);
        shapes("Outputs:", outputs);
        for (const auto &n : nodes) {
            os << "Node " << n.name << " (" << n.op_type << ")";
            for (const auto &a : n.attributes) os << " " << a.first << "=" << a.second;
            os << "\n";
            shapes("  in:", n.inputs);
            shapes("  out:", n.outputs);
        }
        for (const auto &it : initializers) {
            os << "Initializer " << it.first << " " << it.second.dtype << " [";
            for (size_t i = 0; i < it.second.dims.size(); ++i) os << (i ? "," : "") << it.second.dims[i];
            os << "]\n";
        }
        for (size_t l = 0; l < concurrent_execution_levels.size(); ++l) {
            os << "Level " << l << ":";
            for (const auto &name : concurrent_execution_levels[l]) os << " " << name;
            os << "\n";
        }
    }

  private:
    // A position in the file that cannot leave it.
    class Cursor {
      public:
        Cursor(const uint8_t *data, size_t size) : at_(data), end_(data + size) {}
        const uint8_t *take(uint64_t n, const char *what) {
            if (n > static_cast<uint64_t>(end_ - at_)) throw std::runtime_error(std::string("Unexpected end of file in ") + what);
            const uint8_t *p = at_;
            at_ += n;
            return p;
        }
        template <typename V> V value(const char *what) {
            V v;
            std::memcpy(&v, take(sizeof(V), what), sizeof(V));
            return v;
        }
        uint32_t u32(const char *what) { return value<uint32_t>(what); }
        // A count of records of at least `each` bytes: refused when the rest of the file cannot hold them.
        uint32_t count(const char *what, size_t each) {
            const uint32_t n = u32(what);
            if (static_cast<uint64_t>(n) * each > static_cast<uint64_t>(end_ - at_))
                throw std::runtime_error(std::string("Count larger than the file in ") + what);
            return n;
        }
        std::string string(const char *what) {
            const uint32_t n = u32(what);
            const uint8_t *p = take(n, what);
            return std::string(reinterpret_cast<const char *>(p), n);
        }
        std::vector<uint32_t> dims() {
            std::vector<uint32_t> d(count("dims", 4));
            for (auto &v : d) v = u32("dim");
            return d;
        }
        std::vector<Shape> shapes() {
            std::vector<Shape> list(count("shape list", 8));
            for (auto &s : list) {
                s.name = string("tensor name");
                s.dims = dims();
            }
            return list;
        }

      private:
        const uint8_t *at_, *end_;
    };

    template <typename V, typename Read> static std::string list_text(Cursor &c, Read read) {
        const uint32_t n = c.count("attribute list", sizeof(V));
        std::string text = "[";
        for (uint32_t i = 0; i < n; ++i) text += (i ? ", " : "") + std::to_string(read(c));
        return text + "]";
    }

    // model/load.hpp:241-262: tag 0 string, 1 int64, 2 float, 3 list of uint32, 4 list of float.
    static std::unordered_map<std::string, std::string> dict(Cursor &c) {
        std::unordered_map<std::string, std::string> d;
        const uint32_t n = c.count("attribute dict", 5);
        for (uint32_t i = 0; i < n; ++i) {
            std::string key = c.string("attribute name");
            const uint8_t tag = c.value<uint8_t>("attribute tag");
            std::string text;
            switch (tag) {
            case 0: text = c.string("string attribute"); break;
            case 1: text = std::to_string(c.value<int64_t>("int attribute")); break;
            case 2: text = std::to_string(c.value<float>("float attribute")); break;
            case 3: text = list_text<uint32_t>(c, [](Cursor &cc) { return cc.u32("int list"); }); break;
            case 4: text = list_text<float>(c, [](Cursor &cc) { return cc.value<float>("float list"); }); break;
            default: throw std::runtime_error("Unknown attribute type tag " + std::to_string(tag) + " for " + key);
            }
            d[std::move(key)] = std::move(text);
        }
        return d;
    }

    static const char *dtype_name(int code) {  // ONNX TensorProto codes, as the writer maps them (dag.py:200-217)
        static const char *const names[] = {"none",   "float32", "uint8",  "int8",    "uint16", "int16",     "int32",      "int64",   "string",
                                            "bool",   "float16", "float64", "uint32", "uint64", "complex64", "complex128", "bfloat16"};
        return code >= 0 && code < 17 ? names[code] : "none";
    }

    void parse(const uint8_t *data, size_t size) {
        Cursor c(data, size);
        inputs = c.shapes();
        outputs = c.shapes();
        const uint32_t num_nodes = c.count("node list", 28);
        nodes.reserve(num_nodes);
        for (uint32_t i = 0; i < num_nodes; ++i) {
            Node n;
            n.op_type = c.string("op type");
            n.name = c.string("node name");
            n.attributes = dict(c);
            n.inputs = c.shapes();
            n.outputs = c.shapes();
            for (uint32_t j = c.count("dependencies", 4); j > 0; --j) n.dependencies.insert(c.string("dependency"));
            for (uint32_t j = c.count("dependents", 4); j > 0; --j) n.dependents.insert(c.string("dependent"));
            nodes.push_back(std::move(n));
        }
        // initializers, packed into one block at 64-byte steps (model/load.cpp:132-178)
        const uint32_t num_init = c.count("initializer list", 20);
        struct Piece {
            size_t at;  // where the piece goes in initializer_memory
            const uint8_t *bytes;
            size_t size;
        };
        std::vector<Piece> pieces;
        size_t total = 0;
        for (uint32_t i = 0; i < num_init; ++i) {
            Initializer init;
            init.name = c.string("initializer name");
            init.dtype = c.string("initializer dtype");
            init.dims = c.dims();
            const int64_t bytes = c.value<int64_t>("initializer size");
            if (bytes < 0) throw std::runtime_error("Negative size of initializer " + init.name);
            const uint8_t *p = c.take(static_cast<uint64_t>(bytes), "initializer data");
            // (two initializers of one name would leave one offset for two pieces of different sizes)
            if (initializers.count(init.name)) throw std::runtime_error("Initializer " + init.name + " appears twice");
            const size_t at = (total + 63) & ~static_cast<size_t>(63);
            initializer_offsets[init.name] = at;
            initializer_bytes[init.name] = static_cast<size_t>(bytes);
            total = at + static_cast<size_t>(bytes);
            pieces.push_back({at, p, static_cast<size_t>(bytes)});
            initializers[init.name] = std::move(init);
        }
        initializer_memory.assign(total, 0);
        for (const auto &p : pieces)
            if (p.size) std::memcpy(initializer_memory.data() + p.at, p.bytes, p.size);
        const uint32_t num_levels = c.count("level list", 4);
        concurrent_execution_levels.resize(num_levels);
        for (auto &level : concurrent_execution_levels)
            for (uint32_t j = c.count("level", 4); j > 0; --j) level.push_back(c.string("level node"));
        expand_unified();
        restore_rgba_shapes();
    }

    // The records and the concatenated names of one packed table, bounds-checked.
    bool packed_table(const char *meta_name, const char *names_name, std::vector<PackedTensorRecord> &records,
                      std::vector<std::string> &names) const {
        if (initializers.find(meta_name) == initializers.end() || initializers.find(names_name) == initializers.end()) return false;
        const auto &dims = initializers.at(meta_name).dims;
        const size_t n = dims.empty() ? 0 : dims[0] / 8;
        if (n * sizeof(PackedTensorRecord) > initializer_bytes.at(meta_name)) throw std::runtime_error(std::string(meta_name) + ": table larger than its data");
        records.resize(n);
        if (n) std::memcpy(records.data(), initializer_data(meta_name), n * sizeof(PackedTensorRecord));
        const char *text = reinterpret_cast<const char *>(initializer_data(names_name));
        size_t at = 0;
        for (const auto &r : records) {
            if (r.name_len < 0 || at + static_cast<size_t>(r.name_len) > initializer_bytes.at(names_name))
                throw std::runtime_error(std::string(names_name) + ": names run past their data");
            names.emplace_back(text + at, static_cast<size_t>(r.name_len));
            at += static_cast<size_t>(r.name_len);
        }
        return true;
    }

    // Many small tensors stored inside "unified_tensors" become initializers of their own (model/load.cpp:194-238).
    void expand_unified() {
        std::vector<PackedTensorRecord> records;
        std::vector<std::string> names;
        if (initializers.find("unified_tensors") == initializers.end() || !packed_table("unified_metadata", "unified_names", records, names)) return;
        const size_t base = initializer_offsets.at("unified_tensors"), room = initializer_bytes.at("unified_tensors");
        for (size_t i = 0; i < records.size(); ++i) {
            const auto &r = records[i];
            if (r.offset < 0 || r.size < 0 || static_cast<size_t>(r.offset) + static_cast<size_t>(r.size) > room)
                throw std::runtime_error("unified tensor " + names[i] + " lies outside unified_tensors");
            Initializer init;
            init.name = names[i];
            init.dtype = dtype_name(r.dtype);
            for (int d : r.dims) {
                if (d == 0) break;
                init.dims.push_back(static_cast<uint32_t>(d));
            }
            initializer_offsets[init.name] = base + static_cast<size_t>(r.offset);
            initializer_bytes[init.name] = static_cast<size_t>(r.size);
            initializers[init.name] = std::move(init);
        }
        unified = true;
    }

    // Weights stored as RGBA texels get their four original dimensions back (model/load.cpp:240-282).
    void restore_rgba_shapes() {
        std::vector<PackedTensorRecord> records;
        std::vector<std::string> names;
        if (!packed_table("rgba_conversion_metadata", "rgba_conversion_names", records, names)) return;
        for (size_t i = 0; i < records.size(); ++i) {
            auto it = initializers.find(names[i]);
            if (it == initializers.end()) continue;
            it->second.dims.assign(records[i].dims, records[i].dims + 4);
        }
        initializers.erase("rgba_conversion_metadata");
        initializers.erase("rgba_conversion_names");
        rgba = true;
    }
};

}  // namespace load
}  // namespace vkop
#endif  // VKOP_HIP_MODEL_LOAD_HPP_
