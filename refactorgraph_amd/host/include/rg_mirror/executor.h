// What the reference's Python binding does in C++ once a graph exists, without the binding:
// findDevice / compile / Executor of src/09python_ffi/src/{import.cpp:10-22, compiler.cc:60-103,
// executor.h:10-27, executor.cc:12-248}, with "amd" (device) and "hip" (target) as the new names and
// host pointers where the binding takes numpy arrays.  Inputs and outputs are addressed by their
// position among the graph's global inputs / outputs.
#pragma once

#include "rg_mirror/computation.h"

namespace refactor::python_ffi {

    // "cpu" | "amd" (any case); initialises the device on first use
    Arc<hardware::Device> findDevice(std::string type, int card);

    class Executor {
        computation::Graph _graph;
        runtime::Stream _stream;

    public:
        Executor(computation::Graph, runtime::Stream);
        // lowers the graph again for another device / allocator; inputs that were set are carried over
        void dispatch(Arc<hardware::Device>, std::string allocator);
        void setInput(count_t, void const *data, size_t bytes);
        void setInputBlob(count_t, Arc<hardware::Device::Blob>);
        void getOutput(count_t, void *data, size_t bytes) const;
        Arc<hardware::Device::Blob> getOutputBlob(count_t) const;
        void run();
        // (node name, host time) per node; with `sync` every node is waited for
        std::vector<std::pair<std::string, std::chrono::nanoseconds>> bench(bool sync);
        // One node<index>.meta per node and one data<counter>.<format> per tensor it read or wrote, in
        // `path`; format "npy" or anything else for raw bytes.  Tensors are matched to the graph's
        // edges by name (lowering may renumber edges); an edge whose name is not unique gets no file.
        void trace(std::string path, std::string format);
        runtime::Stream &stream() noexcept { return _stream; }
    };

    // target: "cpu" | "hip" (on the device of that kind that was initialised first, card 0 otherwise);
    // allocator: "flat" or anything else for the reusing one
    Arc<Executor> compileOn(computation::Graph, Arc<hardware::Device>, std::string allocator);
    Arc<Executor> compile(computation::Graph, std::string target, std::string allocator);

}// namespace refactor::python_ffi
