// Executor of the host mirror (see rg_mirror/executor.h).
#include "rg_mirror/executor.h"
#include <algorithm>
#include <cstring>
#include <filesystem>
#include <fstream>
#include <iomanip>
#include <map>

namespace refactor::python_ffi {
    using hardware::Device;

    static kernel::Allocator allocatorOf(std::string const &name) {
        return name == "flat" ? kernel::flatAllocate : kernel::reusableAllocate;
    }

    Arc<Device> findDevice(std::string type, int card) {
        std::transform(type.begin(), type.end(), type.begin(), [](unsigned char c) { return std::tolower(c); });
        auto const type_ = type == "cpu"   ? Device::Type::Cpu
                           : type == "amd" ? Device::Type::Amd
                                           : UNREACHABLEX(Device::Type, "Unknown device type: \"", type, '"');
        return hardware::device::init(type_, card, "");
    }

    // computation::Graph is not copyable (operators are owned): the executor keeps the one it was built from
    Executor::Executor(computation::Graph graph, runtime::Stream stream)
        : _graph(std::move(graph)), _stream(std::move(stream)) {}

    void Executor::dispatch(Arc<Device> device, std::string allocator) {
        auto stream = _graph.lower(device->type()).lower(std::move(device), allocatorOf(allocator));
        auto const &topology = _graph.internal().topology;
        std::vector<uint8_t> buffer;
        for (auto i : topology.globalInputs()) {// global inputs keep their indices through lowering
            auto const bytes = _graph.internal().edges[i].tensor->bytesSize();
            buffer.resize(bytes);
            if (_stream.copyData(i, buffer.data(), bytes)) stream.setData(i, buffer.data(), bytes);
        }
        _stream = std::move(stream);
    }

    void Executor::setInput(count_t i, void const *data, size_t bytes) {
        auto const edge = _stream.graph().topology.globalInputs().at(i);
        ASSERT(_graph.internal().edges[edge].tensor->bytesSize() == bytes, "input size mismatch");
        _stream.setData(edge, data, bytes);
    }
    void Executor::setInputBlob(count_t i, Arc<Device::Blob> blob) {
        auto const edge = _stream.graph().topology.globalInputs().at(i);
        ASSERT(_graph.internal().edges[edge].tensor->bytesSize() == blob->size(), "input size mismatch");
        _stream.setData(edge, std::move(blob));
    }
    void Executor::getOutput(count_t i, void *data, size_t bytes) const {
        auto const edge = _stream.graph().topology.globalOutputs().at(i);
        auto const original = _graph.internal().topology.globalOutputs().at(i);
        ASSERT(_graph.internal().edges[original].tensor->bytesSize() == bytes, "output size mismatch");
        ASSERT(_stream.copyData(edge, data, bytes), "the output has not been computed");
    }
    Arc<Device::Blob> Executor::getOutputBlob(count_t i) const {
        return _stream.getData(_stream.graph().topology.globalOutputs().at(i));
    }

    void Executor::run() { _stream.run(); }

    std::vector<std::pair<std::string, std::chrono::nanoseconds>> Executor::bench(bool sync) {
        static Device::Type current;
        current = _stream.device()->type();
        auto const times = _stream.bench(sync ? +[] { hardware::device::sync(current); } : nullptr);
        std::vector<std::pair<std::string, std::chrono::nanoseconds>> ans;
        // node names of the lowered graph are not kept by the stream: they are the operators' names, in
        // order, except where lowering merged nodes (then several operators share one time)
        auto const &nodes = _graph.internal().nodes;
        if (nodes.size() == times.size()) {
            for (size_t i = 0; i < times.size(); ++i) ans.emplace_back(nodes[i].name, times[i]);
        } else {
            for (size_t i = 0; i < times.size(); ++i) ans.emplace_back("node" + std::to_string(i), times[i]);
        }
        return ans;
    }

    static char const *npyType(DataType dt) {
        switch (dt) {
            case DataType::F32: return "<f4";
            case DataType::U8: return "|u1";
            case DataType::I8: return "|i1";
            case DataType::U16: return "<u2";
            case DataType::I16: return "<i2";
            case DataType::I32: return "<i4";
            case DataType::I64: return "<i8";
            case DataType::Bool: return "|b1";
            case DataType::FP16: return "<f2";
            case DataType::F64: return "<f8";
            case DataType::U32: return "<u4";
            case DataType::U64: return "<u8";
            default: return nullptr;// BF16 and the complex types have no numpy descriptor here
        }
    }

    // numpy format 1.0: magic, version, little-endian header length, a Python dict padded with spaces to a
    // multiple of 64 bytes and closed by a newline, then the data
    static void writeNpy(std::ofstream &os, char const *type, kernel::Shape const &shape, char const *data, size_t bytes) {
        std::string dict = "{'descr': '";
        dict += type;
        dict += "', 'fortran_order': False, 'shape': (";
        for (auto d : shape) dict += std::to_string(d) + ",";
        dict += "), }";
        auto const total = (10 + dict.size() + 1 + 63) / 64 * 64;
        std::string header(total, ' ');
        static constexpr char MAGIC[]{static_cast<char>(0x93), 'N', 'U', 'M', 'P', 'Y', 1, 0};
        std::memcpy(header.data(), MAGIC, sizeof MAGIC);
        header[8] = static_cast<char>((total - 10) & 0xff);
        header[9] = static_cast<char>((total - 10) >> 8);
        std::memcpy(header.data() + 10, dict.data(), dict.size());
        header[total - 1] = '\n';
        os.write(header.data(), static_cast<std::streamsize>(total));
        os.write(data, static_cast<std::streamsize>(bytes));
    }

    void Executor::trace(std::string path_, std::string format) {
        namespace fs = std::filesystem;
        auto const path = fs::path(std::move(path_));
        fs::create_directories(path);
        ASSERT(fs::is_directory(path), "Failed to create \"", path.string(), '"');

        // tensors by edge name, names that occur twice left out
        std::map<std::string, kernel::Tensor const *> byName;
        for (auto const &e : _graph.internal().edges) {
            if (!e.tensor) continue;
            auto [it, fresh] = byName.emplace(e.name, e.tensor.get());
            if (!fresh) it->second = nullptr;
        }
        auto const &lowered = _stream.graph();
        auto const device = _stream.device();
        size_t dataIdx = 0;
        std::vector<char> buffer;
        auto numbered = [](char const *stem, size_t i, std::string const &ext) {
            std::ostringstream os;
            os << stem << std::setw(6) << std::setfill('0') << i << '.' << ext;
            return os.str();
        };
        _stream.trace([&](count_t nodeIdx, void const *const *inputs, void const *const *outputs) {
            hardware::device::sync(device->type());
            auto const node = lowered.topology.node(nodeIdx);
            auto dump = [&](count_t edgeIdx, void const *address) -> std::string {
                if (!address) return "";
                auto it = byName.find(lowered.edges[edgeIdx].name);
                if (it == byName.end() || !it->second) return "";
                auto const &tensor = *it->second;
                auto const bytes = tensor.bytesSize();
                buffer.resize(bytes);
                device->copyOut(buffer.data(), address, bytes);
                auto const *type = npyType(tensor.dataType);
                auto const asNpy = format == "npy" && type;
                auto const file = path / numbered("data", dataIdx++, asNpy ? "npy" : format == "npy" ? "bin" : format);
                std::ofstream os(file, std::ios::binary | std::ios::trunc);
                if (asNpy) {
                    writeNpy(os, type, tensor.shape, buffer.data(), bytes);
                } else {
                    os.write(buffer.data(), static_cast<std::streamsize>(bytes));
                }
                return file.string();
            };
            std::ostringstream meta;
            meta << "node\t" << nodeIdx << '\n';
            for (size_t i = 0; i < node.inputs.size(); ++i)
                meta << "input\t" << i << '\t' << lowered.edges[node.inputs[i]].name << '\t' << dump(node.inputs[i], inputs[i]) << '\n';
            for (size_t i = 0; i < node.outputs.size(); ++i)
                meta << "output\t" << i << '\t' << lowered.edges[node.outputs[i]].name << '\t' << dump(node.outputs[i], outputs[i]) << '\n';
            std::ofstream(path / numbered("node", nodeIdx, "meta")) << meta.str();
        });
    }

    Arc<Executor> compileOn(computation::Graph graph, Arc<Device> device, std::string allocator) {
        auto stream = graph.lower(device->type()).lower(std::move(device), allocatorOf(allocator));
        return std::make_shared<Executor>(std::move(graph), std::move(stream));
    }

    Arc<Executor> compile(computation::Graph graph, std::string target, std::string allocator) {
        auto const target_ = target == "cpu"   ? Device::Type::Cpu
                             : target == "hip" ? Device::Type::Amd
                                               : UNREACHABLEX(Device::Type, "Unknown target: ", target);
        return compileOn(std::move(graph), hardware::device::fetch(target_), std::move(allocator));
    }

}// namespace refactor::python_ffi
