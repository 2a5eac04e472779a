#include "rg_mirror/attributes.h"
#include <algorithm>
#include <numeric>

namespace refactor::kernel {

    SoftmaxInfo::SoftmaxInfo(Tensor const &data, dim_t axis) noexcept
        : pre(1), mid(data.shape[axis]), post(1), type(data.dataType) {
        for (dim_t i = 0; i < axis; ++i) { pre *= data.shape[i]; }
        for (size_t i = axis + 1; i < data.shape.size(); ++i) { post *= data.shape[i]; }
    }

    // The shapes are right-aligned and walked from the last dimension to the first.  A dimension
    // is described by which inputs really extend along it (size != 1); a run of dimensions with
    // the same description collapses into one entry.
    Broadcaster::Broadcaster(std::vector<std::vector<dim_t>> const &inputShapes)
        : strides{}, outputsCount(1), inputsCount(static_cast<dim_t>(inputShapes.size())) {
        ASSERT(inputsCount > 0, "Broadcaster: no inputs");
        size_t rank = 0;
        for (auto const &s : inputShapes) { rank = std::max(rank, s.size()); }

        std::vector<bool> pattern(inputsCount, false), here(inputsCount);
        std::vector<dim_t> extent(inputsCount, 1);// elements each input spans so far
        std::vector<std::vector<dim_t>> entries;  // innermost first: per-input strides + output stride
        for (size_t back = 0; back < rank; ++back) {
            dim_t size = 1;
            for (dim_t i = 0; i < inputsCount; ++i) {
                auto const &s = inputShapes[i];
                dim_t d = back < s.size() ? s[s.size() - 1 - back] : 1;
                here[i] = d != 1;
                if (d != 1) {
                    ASSERT(size == 1 || size == d, "Broadcaster: shape mismatch");
                    size = d;
                }
            }
            if (size == 1) { continue; }
            if (here != pattern) {
                pattern = here;
                std::vector<dim_t> entry(inputsCount + 1, 0);
                for (dim_t i = 0; i < inputsCount; ++i) {
                    if (pattern[i]) { entry[i] = extent[i]; }
                }
                entry[inputsCount] = outputsCount;
                entries.push_back(std::move(entry));
            }
            for (dim_t i = 0; i < inputsCount; ++i) {
                if (pattern[i]) { extent[i] *= size; }
            }
            outputsCount *= size;
        }
        // a single entry where every input walks with the output: nothing is broadcast
        if (entries.size() == 1 && std::all_of(entries[0].begin(), entries[0].end(), [](dim_t x) { return x == 1; })) {
            return;
        }
        for (auto it = entries.rbegin(); it != entries.rend(); ++it) {
            strides.insert(strides.end(), it->begin(), it->end());
        }
    }

    Broadcaster::Broadcaster(TensorRefs const &inputs)
        : Broadcaster([&] {
              std::vector<std::vector<dim_t>> shapes;
              for (auto const &t : inputs) { shapes.emplace_back(t.get().shape.begin(), t.get().shape.end()); }
              return shapes;
          }()) {}

    void Broadcaster::locate(dim_t k, dim_t ans[]) const noexcept {
        if (strides.empty()) {
            std::fill_n(ans, inputsCount, k);
            return;
        }
        std::fill_n(ans, inputsCount, 0);
        auto const width = inputsCount + 1;
        for (size_t at = 0; at < strides.size(); at += width) {
            auto const q = k / strides[at + inputsCount];
            k %= strides[at + inputsCount];
            for (dim_t j = 0; j < inputsCount; ++j) { ans[j] += strides[at + j] * q; }
        }
    }

    MatMulIntegerInfo::Input::Input(TensorRefs const &inputs, size_t i) noexcept
        : withZeroPoint(false), signed_(true), scalar(true) {
        if (inputs.size() <= i + 2) { return; }
        auto const &zp = inputs[i + 2].get();
        auto const count = zp.elementsSize();
        if (zp.data) {
            // a constant zero point of all zeros needs no work
            auto bytes = zp.data->get<uint8_t>();
            if (std::all_of(bytes, bytes + count, [](uint8_t x) { return x == 0; })) { return; }
        }
        withZeroPoint = true;
        signed_ = zp.dataType == DataType::I8;
        scalar = count == 1;
    }

    static std::vector<dim_t> batchDims(Tensor const &t) {
        return std::vector<dim_t>(t.shape.begin(), t.shape.end() - 2);
    }

    MatMulInfo::MatMulInfo(Tensor const &a, Tensor const &b, std::optional<std::reference_wrapper<Tensor const>> c,
                           bool transA_, bool transB_, float alpha_, float beta_)
        // src/04kernel/src/attributes/mat_mul_info.cc:27-43
        : dataType(a.dataType),
          alpha(alpha_), beta(beta_),
          transA(transA_), transB(transB_),
          m(transA ? a.shape.rbegin()[0] : a.shape.rbegin()[1]),
          k(transA ? a.shape.rbegin()[1] : a.shape.rbegin()[0]),
          n(transB ? b.shape.rbegin()[1] : b.shape.rbegin()[0]),
          hasBias(c.has_value()), biasSupported(true),
          biasStrideBatch(0), biasStrideM(0), biasStrideN(0),
          broadcaster({batchDims(a), batchDims(b)}) {
        auto kB = transB ? b.shape.rbegin()[0] : b.shape.rbegin()[1];
        ASSERT(k == kB, "MatMul: input shape not matched.");
        if (!c) { return; }
        // the bias broadcasts unidirectionally to [batch dims..., m, n] (mat_mul_info.cc:5-25)
        std::vector<dim_t> out(std::max(a.shape.size(), b.shape.size()) - 2);
        {
            auto const da = a.shape.size() - 2, db = b.shape.size() - 2;
            for (size_t i = 0; i < out.size(); ++i) {
                auto const a_ = i < da ? a.shape[da - i - 1] : 1, b_ = i < db ? b.shape[db - i - 1] : 1;
                out[out.size() - 1 - i] = std::max(a_, b_);
            }
        }
        auto const &cs = c->get().shape;
        auto at = [&](size_t fromEnd) -> dim_t { return fromEnd < cs.size() ? cs.rbegin()[fromEnd] : 1; };
        auto const cn = at(0), cm = at(1);
        if ((cn != 1 && cn != n) || (cm != 1 && cm != m) || cs.size() > out.size() + 2) {
            biasSupported = false;
            return;
        }
        biasStrideN = cn == n ? 1 : 0;
        biasStrideM = cm == m ? cn : 0;
        bool allOne = true, same = cs.size() == out.size() + 2;
        for (size_t i = 2; i < cs.size(); ++i) {
            allOne = allOne && at(i) == 1;
            same = same && at(i) == out[out.size() + 1 - i];
        }
        if (allOne) {
            biasStrideBatch = 0;
        } else if (same) {
            biasStrideBatch = static_cast<size_t>(cm) * cn;
        } else {
            // some batch dimensions broadcast and others do not: expanded into a workspace first, if the shapes
            // broadcast at all
            for (size_t i = 2; i < cs.size(); ++i) {
                if (at(i) != 1 && at(i) != out[out.size() + 1 - i]) {
                    biasSupported = false;
                    return;
                }
            }
            biasExpandFrom.assign(cs.begin(), cs.end());
            biasExpandTo = out;
            biasExpandTo.push_back(m);
            biasExpandTo.push_back(n);
            biasStrideN = 1;
            biasStrideM = n;
            biasStrideBatch = static_cast<size_t>(m) * n;
        }
    }

    MatMulIntegerInfo::MatMulIntegerInfo(TensorRefs const &inputs) noexcept
        : a(inputs, 0),
          b(inputs, 1),
          m(inputs[0].get().shape.rbegin()[1]),
          k(inputs[0].get().shape.rbegin()[0]),
          n(inputs[1].get().shape.rbegin()[0]),
          broadcaster({batchDims(inputs[0].get()), batchDims(inputs[1].get())}) {}

    // ------------------------------------------------------------------ TransposeInfo

    TransposeInfo::TransposeInfo(DataType dt, std::vector<dim_t> const &shape_, Permutation const &perm_)
        : dims{}, blockSize(static_cast<dim_t>(dt.size())), blockCount(1) {
        ASSERT(perm_.size() == shape_.size(), "a permutation names every dimension once");
        for (auto d : shape_) blockCount *= d;
        // runs of input dimensions (size 1 left out) that stay neighbours in the output, in output order
        std::vector<std::vector<dim_t>> runs;
        for (auto p : perm_) {
            ASSERT(p < shape_.size(), "a permutation names every dimension once");
            if (shape_[p] == 1) continue;
            // the previous kept dimension of the input, skipping size-1 ones
            bool follows = false;
            if (!runs.empty()) {
                auto last = runs.back().back();
                follows = p > last;
                for (auto q = last + 1; follows && q < p; ++q) follows = shape_[q] == 1;
            }
            if (follows) {
                runs.back().push_back(p);
            } else {
                runs.push_back({p});
            }
        }
        auto whole = [this] {
            dims = {{1, 1}};
            blockSize *= blockCount;
            blockCount = 1;
        };
        if (runs.size() <= 1) {
            whole();
            return;
        }
        auto extent = [&](std::vector<dim_t> const &run) {
            dim_t n = 1;
            for (auto d : run) n *= shape_[d];
            return n;
        };
        // input stride of a run, in blocks of the element size: everything behind its last dimension
        auto strideIn = [&](std::vector<dim_t> const &run) {
            dim_t n = 1;
            for (auto d = run.back() + 1; d < shape_.size(); ++d) n *= shape_[d];
            return n;
        };
        // the run that holds the input's last kept dimension, if it is also the output's last: part of the block
        dim_t inner = 1;
        if (strideIn(runs.back()) == 1) {
            inner = extent(runs.back());
            blockSize *= inner;
            blockCount /= inner;
            runs.pop_back();
        }
        dims.resize(runs.size());
        dim_t strideO = 1;
        for (auto i = runs.size(); i-- > 0;) {
            dims[i] = {strideIn(runs[i]) / inner, strideO};
            strideO *= extent(runs[i]);
        }
    }

    dim_t TransposeInfo::locate(dim_t i) const noexcept {
        dim_t ans = 0;
        for (auto [strideI, strideO] : dims) {
            ans += i / strideO * strideI;
            i %= strideO;
        }
        return ans;
    }

    // ------------------------------------------------------------------ SplitInfo

    SplitInfo::SplitInfo(dim_t axis, TensorRefs const &parts) : blockCount(1), sum(0), segments() {
        ASSERT(!parts.empty(), "SplitInfo: no parts");
        auto const &shape = parts[0].get().shape;
        ASSERT(axis < shape.size(), "SplitInfo: axis out of range");
        for (size_t d = 0; d < axis; ++d) { blockCount *= shape[d]; }
        dim_t postfix = static_cast<dim_t>(parts[0].get().dataType.size());
        for (size_t d = axis + 1; d < shape.size(); ++d) { postfix *= shape[d]; }
        segments.reserve(parts.size());
        for (auto const &part : parts) {
            segments.push_back(part.get().shape[axis] * postfix);
            sum += segments.back();
        }
    }

    // ------------------------------------------------------------------ ExpandInfo

    ExpandInfo::ExpandInfo(DataType dataType, std::vector<dim_t> const &input, std::vector<dim_t> const &output)
        : strides(), blockCount(1), blockSize(static_cast<dim_t>(dataType.size())) {
        ASSERT(input.size() <= output.size(), "ExpandInfo: the input has more dimensions than the output");
        // from the innermost dimension outwards: a run of dimensions that are all kept or all broadcast is one
        // stride pair; `kept` tells what the innermost run so far is (it starts as a kept run of extent 1)
        std::vector<Dim> reversed;
        bool kept = true, any = false;
        dim_t stride = 1;
        auto i = input.size();
        for (auto o = output.size(); o != 0;) {
            auto const i_ = i == 0 ? dim_t(1) : input[--i], o_ = output[--o];
            if (o_ == 1) { continue; }
            if (i_ == 1) {
                if (kept) { reversed.push_back({0, blockCount}); kept = false; any = true; }
            } else {
                ASSERT(i_ == o_, "ExpandInfo: shapes do not broadcast");
                if (!kept) { reversed.push_back({stride, blockCount}); kept = true; }
                stride *= i_;
            }
            blockCount *= o_;
        }
        if (!any) {// nothing is broadcast: one block
            blockSize *= blockCount;
            blockCount = 1;
            return;
        }
        strides.assign(reversed.rbegin(), reversed.rend());
        // the innermost pair is a broadcast one (a kept innermost run is implicit): it becomes the block
        auto const tail = strides.back();
        blockSize *= tail.o;
        blockCount /= tail.o;
        for (auto &s : strides) {
            s.i /= tail.o;
            s.o /= tail.o;
        }
    }

    ExpandInfo::ExpandInfo(Tensor const &input, Tensor const &output)
        : ExpandInfo(input.dataType, input.shape, output.shape) {}

}// namespace refactor::kernel
