// Gathering and scattering through index tensors: the checks of the front end
// (ref: src/tensor/index.rs:712-755, src/ops/scatter.rs:13-234).
#include <algorithm>

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

// ---- advanced indexing (ref: src/ops/advanced_index.rs) ---------------------------------------------------------
//
// Masks are expanded into one coordinate vector per dimension they cover, the indices are broadcast together, and
// when the indexed dimensions are not adjacent they move to the front of the result. Reading and writing both
// fold the target, its dimensions in that order, into [before, indexed, after] and pick or write slices along
// the middle dimension at the linear positions the indices give in the indexed subspace.

namespace {

// One index after masks are expanded: positions on the device of the target.
struct Coords {
    Shape shape;
    TensorData values;
};

// nullopt if the shapes don't broadcast together (ref: advanced_index.rs:79-97).
std::optional<Shape> broadcast_of(const Shape &a, const Shape &b) {
    const size_t n = std::max(a.size(), b.size());
    auto dim = [&](const Shape &s, size_t i) { return i < n - s.size() ? int64_t{1} : s[i - (n - s.size())]; };
    Shape out;
    for (size_t i = 0; i < n; ++i) {
        const int64_t x = dim(a, i), y = dim(b, i);
        if (x == y || y == 1) out.push_back(x);
        else if (x == 1) out.push_back(y);
        else return std::nullopt;
    }
    return out;
}

// Indices on the CPU are copied to the target's device first (ref: advanced_index.rs:46-57).
TensorData on_device(const TensorData &data, Device device) {
    if (data.device() == Device::cpu() && device != Device::cpu()) return Tensor(data).to(device).data();
    return data;
}

int64_t product(const Shape &s, size_t from, size_t to) {
    int64_t n = 1;
    for (size_t k = from; k < to; ++k) n *= s[k];
    return n;
}

class AdvancedIndex {
  public:
    // ref: advanced_index.rs:99-231 (ATen's make_info): index dtypes, then devices, mask shapes, the number of
    // indices, broadcasting, and indices into empty dimensions.
    // `one_value`: the caller is about to assign a single value without accumulating. A mask that stands alone
    // then needs neither positions nor its count (one value fits any number of selected elements): the slots of its
    // dimensions take the mask's size as a stand-in, and scatter() selects.
    AdvancedIndex(const TensorData &target, const std::vector<std::optional<Tensor>> &indices, bool one_value = false) {
        const Device device = target.device();
        const Shape &shape = target.layout.shape;
        const size_t nd = shape.size();
        for (const auto &t : indices) {
            if (!t) continue;
            const DType d = t->dtype();
            if (d != DType::I64 && d != DType::I32 && d != DType::Bool) {
                throw Error(std::string("tensors used as indices must be i64, i32 or bool tensors, got ") + name_of(d) +
                            (d == DType::U8 ? "; use a bool tensor for a mask" : ""));
            }
        }
        for (const auto &t : indices) {
            if (t && t->device() != Device::cpu() && t->device() != device) {
                throw Error("indices should be either on cpu or on the same device as the indexed tensor (" + device.str() + ")");
            }
        }
        size_t count = 0;
        for (const auto &t : indices) count += t && t->dtype() == DType::Bool ? t->num_dims() : 1;
        if (count > nd) {
            throw Error("too many indices for tensor of dimension " + std::to_string(nd) + " (got " + std::to_string(count) + ")");
        }
        size_t defined_indices = 0;
        for (const auto &t : indices) defined_indices += t ? 1 : 0;
        std::vector<std::optional<Coords>> slots;
        for (const auto &t : indices) {
            if (!t) {
                slots.push_back(std::nullopt);
                continue;
            }
            const TensorData &data = t->data();
            if (t->dtype() != DType::Bool) {
                slots.push_back(Coords{data.layout.shape, on_device(data, device)});
                continue;
            }
            const Shape &mask_shape = data.layout.shape;
            if (mask_shape.empty()) throw Error("indexing with a zero-dimensional bool tensor is not supported");
            const size_t start = slots.size();
            for (size_t j = 0; j < mask_shape.size(); ++j) {
                if (mask_shape[j] != shape[start + j]) {
                    throw Error("The shape of the mask " + shape_str(mask_shape) + " at index " + std::to_string(j) +
                                " does not match the shape of the indexed tensor " + shape_str(shape) + " at index " +
                                std::to_string(start + j));
                }
            }
            if (defined_indices == 1) {
                // The only index: with its elements in order, the coordinates of the flattened mask are the
                // linear positions in the subspace it covers. They are in range by construction, so neither a
                // check nor a pass per dimension follows. Only the count is taken here: it shapes the result;
                // the positions are written when a read or a write asks for them.
                // (A mask that is a view is laid out in order first, a copy of a byte per element - unless only a
                // select follows, which walks any layout.)
                const TensorData dense = one_value || data.layout.is_contiguous() ? data : Tensor(data).contiguous().data();
                TensorData flat = dense;
                flat.layout = Layout::contiguous(Shape{dense.layout.num_elements()});
                flat.layout.offset = dense.layout.offset;
                mask_ = dense;
                int64_t count = flat.layout.num_elements();
                if (one_value) {
                    select_only_ = true;
                } else {
                    counted_ = backend::mask_count(flat);
                    count = counted_->count;
                }
                // The slots of the mask's dimensions keep the shape; their values are never read.
                for (size_t j = 0; j < mask_shape.size(); ++j) slots.push_back(Coords{Shape{count}, flat});
                continue;
            }
            for (const TensorData &values : backend::mask_coordinates(data)) {
                slots.push_back(Coords{values.layout.shape, on_device(values, device)});
            }
        }
        while (!slots.empty() && !slots.back()) slots.pop_back();
        std::vector<size_t> defined;
        for (size_t k = 0; k < slots.size(); ++k) {
            if (slots[k]) defined.push_back(k);
        }
        if (defined.empty()) throw Error("advanced indexing needs at least one index tensor");
        bool adjacent = true;
        for (size_t k = defined.front(); k <= defined.back(); ++k) adjacent = adjacent && slots[k].has_value();
        slots.resize(nd);
        if (adjacent) {
            for (size_t k = 0; k < nd; ++k) perm_.push_back(k);
            first_ = defined.front();
        } else {
            perm_ = defined;
            for (size_t k = 0; k < nd; ++k) {
                if (!slots[k]) perm_.push_back(k);
            }
            first_ = 0;
        }
        for (size_t k : perm_) shape_.push_back(shape[k]);
        for (size_t k : perm_) {
            if (slots[k]) coords_.push_back(std::move(*slots[k]));
        }
        std::optional<Shape> together = Shape{};
        for (const Coords &c : coords_) {
            together = broadcast_of(*together, c.shape);
            if (!together) {
                std::string shapes;
                for (const Coords &each : coords_) shapes += (shapes.empty() ? "" : ", ") + shape_str(each.shape);
                throw Error("shape mismatch: indexing tensors could not be broadcast together with shapes " + shapes);
            }
        }
        broadcast_ = *together;
        const size_t n = coords_.size();
        bool empty_dimension = false;
        for (size_t k = first_; k < first_ + n; ++k) empty_dimension = empty_dimension || shape_[k] == 0;
        if (product(broadcast_, 0, broadcast_.size()) > 0 && empty_dimension) {
            throw Error("index is out of bounds for dimension with size 0");
        }
        out_shape_.assign(shape_.begin(), shape_.begin() + first_);
        out_shape_.insert(out_shape_.end(), broadcast_.begin(), broadcast_.end());
        out_shape_.insert(out_shape_.end(), shape_.begin() + first_ + n, shape_.end());
    }

    const Shape &out_shape() const { return out_shape_; }

    // The indexing result: a new contiguous tensor of out_shape (ref: advanced_index.rs:293-316).
    Tensor gather(const TensorData &target) const {
        Tensor out = Tensor::uninit_on(out_shape_, target.dtype, target.device());
        if (out.num_elements() == 0) {
            check_and_place(nullptr);
            return out;
        }
        const Tensor src = Tensor(permuted(target)).reshape(folded());
        TensorData shaped = out.data();
        if (coords_.size() == 1 && !mask_ && coords_[0].values.layout.is_contiguous()) {
            // One index tensor: its elements are the positions along the one indexed dimension, the negative ones
            // counted from the end, which the row lookup does by itself. The check stays (and its message, which
            // names the dimension as the caller sees it); the pass that writes positions is not needed.
            check_and_place(nullptr);
            TensorData ids = coords_[0].values;
            const int64_t count = ids.layout.num_elements();
            const int64_t offset = ids.layout.offset;
            ids.layout = Layout::contiguous(Shape{count});
            ids.layout.offset = offset;
            shaped.layout = Layout::contiguous(Shape{before(), count, after()});
            backend::index_select(shaped, src.data(), 1, ids, Bounds::ValidWrap);
            return out;
        }
        const TensorData where = positions(target.device());
        const int64_t count = where.layout.num_elements();
        shaped.layout = Layout::contiguous(Shape{before(), count, after()});
        backend::index_select(shaped, src.data(), 1, where, Bounds::Valid);
        return out;
    }

    // ref: advanced_index.rs:318-343
    void check_values(const TensorData &target, const TensorData &values) const {
        if (values.dtype != target.dtype) {
            throw Error(std::string("Index put requires the source and destination dtypes match, got ") + name_of(target.dtype) +
                        " for the destination and " + name_of(values.dtype) + " for the source.");
        }
        if (values.device() != target.device()) {
            throw Error("Expected all tensors to be on the same device, but found at least two devices, " + target.device().str() +
                        " and " + values.device().str() + "!");
        }
        const Shape &v = values.layout.shape, &o = out_shape_;
        bool fits = v.size() <= o.size();
        for (size_t k = 0; fits && k < v.size(); ++k) {
            const int64_t b = o[o.size() - v.size() + k];
            fits = v[k] == b || v[k] == 1;
        }
        if (!fits) {
            throw Error("shape mismatch: value tensor of shape " + shape_str(v) + " cannot be broadcast to indexing result of shape " +
                        shape_str(o));
        }
    }

    // A copy of the target with `values` written at the indexed positions: added with `accumulate`, otherwise
    // copied, the last of repeated positions winning. The work happens on a contiguous copy with the dimensions
    // in the order of perm, which the result sees in the original order (ref: advanced_index.rs:345-387).
    Tensor scatter(const TensorData &target, const TensorData &values, bool accumulate) const {
        if (mask_ && !accumulate && values.layout.num_elements() == 1) {
            // One value for every element a mask selects: an element-wise choice between the value and the target,
            // with the mask broadcast over the dimensions behind it. No positions, no copy of the target first.
            const Shape &shape = target.layout.shape;
            const TensorData moved = on_device(*mask_, target.device());  // any layout: the select walks it
            TensorData cond = moved;
            cond.layout.shape = shape;
            cond.layout.strides.assign(shape.size(), 0);
            for (size_t j = 0; j < moved.layout.shape.size(); ++j) cond.layout.strides[first_ + j] = moved.layout.strides[j];
            Tensor out = Tensor::uninit_on(shape, target.dtype, target.device());
            backend::where_(out.data(), cond, values.expand_to(shape), target);
            return out;
        }
        const TensorData work = copy_of(Tensor(permuted(target)));
        if (product(out_shape_, 0, out_shape_.size()) == 0) {
            check_and_place(nullptr);
        } else {
            const TensorData where = positions(target.device());
            const int64_t count = where.layout.num_elements();
            TensorData shaped = work;
            shaped.layout = Layout::contiguous(folded());
            const Tensor src = Tensor(values.expand_to(out_shape_)).reshape(Shape{before(), count, after()});
            if (accumulate) backend::index_add(shaped, 1, where, src.data(), Bounds::Valid);
            else backend::index_overwrite(shaped, 1, where, src.data());
        }
        const size_t nd = perm_.size();
        TensorData result = work;
        result.layout.shape.assign(nd, 0);
        result.layout.strides.assign(nd, 0);
        for (size_t k = 0; k < nd; ++k) {
            result.layout.shape[perm_[k]] = work.layout.shape[k];
            result.layout.strides[perm_[k]] = work.layout.strides[k];
        }
        return Tensor(result);
    }

  private:
    int64_t before() const { return product(shape_, 0, first_); }
    int64_t indexed() const { return product(shape_, first_, first_ + coords_.size()); }
    int64_t after() const { return product(shape_, first_ + coords_.size(), shape_.size()); }
    Shape folded() const { return Shape{before(), indexed(), after()}; }

    // Checks every position to be in range along its dimension, the indices in order; with `out`, then writes
    // the linear position in the indexed subspace of every element of the broadcast shape (ref: :241-262).
    void check_and_place(const TensorData *out) const {
        if (mask_ && out == nullptr) return;  // the coordinates of a mask need no check
        std::vector<TensorData> values;
        for (const Coords &c : coords_) values.push_back(c.values);
        const std::vector<int64_t> sizes(shape_.begin() + first_, shape_.begin() + first_ + coords_.size());
        if (auto bad = backend::index_positions(out, values, sizes)) {
            throw Error(backend::out_of_bounds(bad->second, bad->first, sizes[bad->first]));
        }
    }

    // ref: advanced_index.rs:264-279
    TensorData positions(Device device) const {
        if (select_only_) throw Error("advanced indexing: the positions of an uncounted mask were asked for");
        if (counted_) return on_device(backend::mask_coordinates(*counted_).front(), device);
        const int64_t n = product(broadcast_, 0, broadcast_.size());
        const TensorData out = Tensor::uninit_on(Shape{n}, DType::I64, device).data();
        TensorData shaped = out;
        shaped.layout = Layout::contiguous(broadcast_);
        check_and_place(&shaped);
        return out;
    }

    TensorData permuted(const TensorData &data) const {
        TensorData d = data;
        d.layout.shape.clear();
        d.layout.strides.clear();
        for (size_t k : perm_) {
            d.layout.shape.push_back(data.layout.shape[k]);
            d.layout.strides.push_back(data.layout.strides[k]);
        }
        return d;
    }

    std::vector<size_t> perm_;  // the target's dimensions in working order: the indexed ones first unless adjacent
    Shape shape_;               // the target's shape in that order
    size_t first_ = 0;          // the first indexed dimension in shape_
    std::vector<Coords> coords_;
    std::optional<backend::MaskCount> counted_;  // set when one contiguous mask is the only index: its flattening, counted
    std::optional<TensorData> mask_;             // and the mask itself
    bool select_only_ = false;                   // the mask was not counted: only scatter()'s select may follow
    Shape broadcast_;           // what the indices broadcast to
    Shape out_shape_;           // before + broadcast + after
};

}  // namespace

Tensor Tensor::index_tensors(const std::vector<std::optional<Tensor>> &indices) const {
    const AdvancedIndex info(d_, indices);
    return info.gather(d_);
}

Tensor Tensor::index_put_tensors(const std::vector<std::optional<Tensor>> &indices, const Tensor &values, bool accumulate) const {
    const bool one_value = !accumulate && values.num_elements() == 1 && values.num_dims() <= 1;
    const AdvancedIndex info(d_, indices, one_value);
    info.check_values(d_, values.data());
    return info.scatter(d_, values.data(), accumulate);
}

}  // namespace homura
