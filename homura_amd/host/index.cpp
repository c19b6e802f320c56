// Gathering and scattering through index tensors: the checks of the front end
// (ref: src/tensor/index.rs:712-755, src/ops/scatter.rs:13-234).
#include "homura.hpp"

namespace homura {

namespace {

void check_index_dtype(const char *op, const Tensor &index) {
    if (index.dtype() != DType::I32 && index.dtype() != DType::I64) {
        throw Error(std::string(op) + "(): Expected dtype i32 or i64 for index, got " + name_of(index.dtype()));
    }
}

void same_device(std::initializer_list<const Tensor *> tensors) {
    const Tensor *first = *tensors.begin();
    for (const Tensor *t : tensors) {
        if (t->device() != first->device()) {
            throw Error("Expected all tensors to be on the same device, but found at least two devices, " + first->device().str() +
                        " and " + t->device().str() + "!");
        }
    }
}

// A zero-dimensional layout seen as a one-dimensional one of one element, as gather and scatter_add treat scalars.
TensorData at_least_1d(const TensorData &data) {
    if (!data.layout.shape.empty()) return data;
    TensorData d = data;
    d.layout.shape = Shape{1};
    d.layout.strides = Strides{1};
    return d;
}

TensorData copy_of(const Tensor &t) {
    // A new contiguous tensor with the elements of `t`.
    Tensor fresh = Tensor::uninit_on(t.shape(), t.dtype(), t.device());
    backend::copy(fresh.data(), t.data());
    return fresh.data();
}

}  // namespace

Tensor Tensor::index_select(int64_t dim, const Tensor &index) const {
    if (index.num_dims() > 1) throw Error("index_select(): Index is supposed to be a vector");
    check_index_dtype("index_select", index);
    const size_t nd = num_dims();
    if (nd == 0) throw Error("index_select() cannot be applied to a 0-dim tensor.");
    same_device({this, &index});
    const size_t d = normalize_dim(dim, nd);
    Tensor flat = index.reshape({-1}).to(DType::I64).contiguous();
    Shape shape = d_.layout.shape;
    shape[d] = flat.num_elements();
    Tensor out = Tensor::uninit_on(shape, d_.dtype, device());
    backend::index_select(out.data(), d_, d, flat.data(), Bounds::NonNegative);
    return out;
}

Tensor Tensor::gather(int64_t dim, const Tensor &index) const {
    same_device({this, &index});
    check_index_dtype("gather", index);
    const size_t d = normalize_dim(dim, num_dims());
    const TensorData src = at_least_1d(d_), idx = at_least_1d(index.data());
    const Shape &shape = src.layout.shape, &index_shape = idx.layout.shape;
    if (index_shape.size() != shape.size()) throw Error("Index tensor must have the same number of dimensions as input tensor");
    for (size_t k = 0; k < shape.size(); ++k) {
        if (k != d && index_shape[k] > shape[k]) {
            throw Error("Size does not match at dimension " + std::to_string(k) + " expected index " + shape_str(index.shape()) +
                        " to be no larger than self " + shape_str(this->shape()) + " apart from dimension " + std::to_string(d));
        }
    }
    Tensor out = Tensor::uninit_on(index.shape(), d_.dtype, device());
    backend::gather(at_least_1d(out.data()), src, d, idx);
    return out;
}

Tensor Tensor::index_add(int64_t dim, const Tensor &index, const Tensor &source) const {
    same_device({this, &index, &source});
    if (index.num_dims() > 1) throw Error("index_add(): Index is supposed to be a vector");
    check_index_dtype("index_add", index);
    const Shape &shape = this->shape(), &src_shape = source.shape();
    const size_t nd = shape.size();
    if (nd == 0) throw Error("index_add() cannot be applied to a 0-dim tensor.");
    const size_t d = normalize_dim(dim, nd);
    if (dtype() != source.dtype()) {
        throw Error(std::string("index_add(): self (") + name_of(dtype()) + ") and source (" + name_of(source.dtype()) +
                    ") must have the same scalar type");
    }
    const int64_t count = index.num_elements();
    int64_t src_size = 1;
    if (!src_shape.empty()) {
        if (d >= src_shape.size()) {
            throw Error("index_add(): Indexing dim " + std::to_string(d) + " is out of bounds of the source tensor with dim " +
                        std::to_string(src_shape.size()));
        }
        src_size = src_shape[d];
    }
    if (count != src_size) {
        throw Error("index_add(): Number of indices (" + std::to_string(count) + ") should be equal to source.size(dim): (" +
                    std::to_string(src_size) + "), for dim: " + std::to_string(d));
    }
    bool same = src_shape.size() == nd;
    for (size_t k = 0; same && k < nd; ++k) same = k == d || src_shape[k] == shape[k];
    if (!same) {
        throw Error("source tensor shape must match self tensor shape, excluding the specified dimension. Got self.shape = " +
                    shape_str(shape) + " source.shape = " + shape_str(src_shape));
    }
    TensorData out = copy_of(*this);
    backend::index_add(out, d, index.data(), source.data(), Bounds::NonNegative);
    return Tensor(out);
}

Tensor Tensor::scatter_add(int64_t dim, const Tensor &index, const Tensor &src) const {
    same_device({this, &index, &src});
    check_index_dtype("scatter_add", index);
    if (dtype() != src.dtype()) throw Error("scatter_add(): Expected self.dtype to be equal to src.dtype");
    const size_t d = normalize_dim(dim, num_dims());
    const TensorData idx = at_least_1d(index.data()), source = at_least_1d(src.data());
    const Shape shape = at_least_1d(d_).layout.shape;
    const Shape &index_shape = idx.layout.shape, &src_shape = source.layout.shape;
    if (index_shape.size() != shape.size()) throw Error("Index tensor must have the same number of dimensions as self tensor");
    if (src_shape.size() != shape.size()) throw Error("Index tensor must have the same number of dimensions as src tensor");
    for (size_t k = 0; k < shape.size(); ++k) {
        if ((k != d && index_shape[k] > shape[k]) || index_shape[k] > src_shape[k]) {
            throw Error("Expected index " + shape_str(index.shape()) + " to be no larger than self " + shape_str(this->shape()) +
                        " apart from dimension " + std::to_string(d) + " and to be no larger size than src " + shape_str(src.shape()));
        }
    }
    TensorData out = copy_of(*this);
    backend::scatter_add(at_least_1d(out), d, idx, source);
    return Tensor(out);
}

}  // namespace homura
