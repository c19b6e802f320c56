// The ops front end: argument checks, type promotion, broadcasting, output allocation and the
// call into the backend. See homura.hpp for the map to the reference's files.
#include <algorithm>
#include <cmath>
#include <cstring>
#include <optional>

#include "homura.hpp"

namespace homura {

namespace {

bool g_fused_promotion = true;

// ---- helpers of src/ops/mod.rs ---------------------------------------------------------------------------

Device common_device(const std::vector<const TensorData *> &tensors) {
    std::optional<Device> device;
    for (const TensorData *t : tensors) {
        if (!device) device = t->device();
        else if (*device != t->device()) {
            throw Error("Expected all tensors to be on the same device, but found at least two devices, " +
                        device->str() + " and " + t->device().str() + "!");
        }
    }
    if (!device) throw Error("expected at least one tensor");
    return *device;
}

TensorData uninit_data(const Shape &shape, DType dtype, Device device) {
    Layout l = Layout::contiguous(shape);
    size_t nbytes = static_cast<size_t>(l.num_elements()) * size_in_bytes(dtype);
    return TensorData{std::make_shared<Storage>(device, nbytes), l, dtype};
}

// `data` converted to `dtype` (a copy only when the dtype differs): ref src/ops/mod.rs:175-195.
TensorData cast_data(const TensorData &data, DType dtype) {
    if (data.dtype == dtype) return data;
    TensorData out = uninit_data(data.layout.shape, dtype, data.device());
    backend::copy(out, data);
    return out;
}

TensorData clone_data(const TensorData &data) {
    TensorData out = uninit_data(data.layout.shape, data.dtype, data.device());
    backend::copy(out, data);
    return out;
}

TensorData reshape_data(const TensorData &data, const Shape &shape) {
    const Layout &l = data.layout;
    if (auto st = compute_view_strides(l.shape, l.strides, shape)) {
        return TensorData{data.storage, Layout{shape, *st, l.offset}, data.dtype};
    }
    TensorData c = clone_data(data);
    c.layout = Layout::contiguous(shape);
    return c;
}

TensorData scalar_data(Scalar value, DType dtype, Device device) {
    TensorData out = uninit_data({}, dtype, device);
    backend::fill(out, value);
    return out;
}

Scalar fill_value(Scalar value, DType dtype) {
    if (auto v = value.checked_to(dtype)) return *v;
    throw Error(std::string("value cannot be converted to type ") + name_of(dtype) + " without overflow");
}

// The value of a one-element tensor as a scalar of its kind; on a GPU the read waits for it
// (ref: src/ops/mod.rs:261-268).
Scalar scalar_value(const Tensor &t) {
    if (t.dtype() == DType::Bool) {
        return Scalar::of_bool(t.to_bytes()[0] != 0);
    }
    if (is_floating_point(t.dtype())) {
        double v;
        std::memcpy(&v, t.to(DType::F64).to_bytes().data(), sizeof v);
        return Scalar::of_float(v);
    }
    int64_t v;
    std::memcpy(&v, t.to(DType::I64).to_bytes().data(), sizeof v);
    return Scalar::of_int(v);
}

// ---- Resolved operands (ref: src/ops/binary.rs:12-61) -----------------------------------------------

struct Resolved {
    std::optional<TensorData> tensor;
    Scalar scalar{};
    explicit Resolved(const Operand &o) {
        if (std::holds_alternative<Tensor>(o)) tensor = std::get<Tensor>(o).data();
        else scalar = std::get<Scalar>(o);
    }
    void add_to(ResultType &rt) const {
        if (tensor) rt.tensor(tensor->dtype, tensor->layout.shape.size());
        else rt.scalar(scalar);
    }
    bool is_bool() const { return tensor ? tensor->dtype == DType::Bool : scalar.kind == Scalar::K::Bool; }
    Shape shape() const { return tensor ? tensor->layout.shape : Shape{}; }
    TensorData materialize(DType dtype, Device device, const Shape &shape) const {
        if (tensor) return cast_data(*tensor, dtype).expand_to(shape);
        return scalar_data(scalar, dtype, device).expand_to(shape);
    }
};

const char *unary_debug_name(UnaryOp op) {
    static const char *names[] = {"Neg", "Abs", "Sign", "Relu", "Exp", "Log", "Sqrt", "Rsqrt", "Reciprocal", "Sin",
                                  "Cos", "Erf", "Tanh", "Sigmoid", "LogSigmoid", "Silu", "Gelu", "GeluTanh",
                                  "LogicalNot"};
    return names[static_cast<int>(op)];
}

bool is_comparison(BinaryOp op) { return op >= BinaryOp::Greater && op <= BinaryOp::NotEqual; }

// [`where_`] with the result's dtype given (ref: src/ops/binary.rs:178-216).
Tensor select_op(const Tensor &condition, const Operand &x_operand, const Operand &y_operand, DType dtype) {
    TensorData cond = condition.data();
    Resolved x(x_operand), y(y_operand);
    std::vector<const TensorData *> devices = {&cond};
    if (x.tensor) devices.push_back(&*x.tensor);
    if (y.tensor) devices.push_back(&*y.tensor);
    Device device = common_device(devices);
    Shape shape = broadcast_shapes(broadcast_shapes(cond.layout.shape, x.shape()), y.shape());
    TensorData out = uninit_data(shape, dtype, device);
    TensorData c = cond.expand_to(shape);
    if (x.tensor && y.tensor) {
        backend::where_(out, c, x.materialize(dtype, device, shape), y.materialize(dtype, device, shape));
    } else {
        std::optional<TensorData> xd, yd;
        if (x.tensor) xd = x.materialize(dtype, device, shape);
        if (y.tensor) yd = y.materialize(dtype, device, shape);
        backend::Branch bx{xd ? &*xd : nullptr, x.scalar}, by{yd ? &*yd : nullptr, y.scalar};
        backend::where_constant(out, c, bx, by);
    }
    return Tensor(out);
}

Shape reduced_shape(const Shape &shape, const std::vector<bool> &mask, bool keepdim) {
    Shape out;
    for (size_t d = 0; d < shape.size(); ++d) {
        if (!mask[d]) out.push_back(shape[d]);
        else if (keepdim) out.push_back(1);
    }
    return out;
}

// ref: src/ops/reduce.rs:55-90
Tensor reduce_op(ReduceOp op, const Tensor &x, const std::vector<int64_t> &dims, bool keepdim, const char *name) {
    const TensorData &src = x.data();
    DType dtype = src.dtype;
    std::vector<bool> mask = dims_mask(dims, src.layout.shape.size());
    DType out_dtype = dtype;
    if ((op == ReduceOp::Sum || op == ReduceOp::Prod) && !is_floating_point(dtype)) out_dtype = DType::I64;
    else if (op == ReduceOp::Mean && !is_floating_point(dtype)) {
        throw Error(std::string(name) + "(): could not infer output dtype. Input dtype must be either a floating "
                                        "point or complex dtype. Got: " + name_of(dtype));
    } else if ((op == ReduceOp::All || op == ReduceOp::Any) && dtype != DType::U8) out_dtype = DType::Bool;
    bool reduces_empty = false;
    for (size_t d = 0; d < mask.size(); ++d) reduces_empty = reduces_empty || (mask[d] && src.layout.shape[d] == 0);
    if ((op == ReduceOp::Max || op == ReduceOp::Min) && reduces_empty) {
        throw Error(std::string(name) + "(): Expected reduction dim to be specified for input.numel() == 0. Specify "
                                        "the reduction dim with the 'dim' argument.");
    }
    TensorData out = uninit_data(reduced_shape(src.layout.shape, mask, keepdim), out_dtype, src.device());
    backend::reduce(op, out, src, mask);
    return Tensor(out);
}

// ref: src/ops/reduce.rs:92-135
std::pair<std::optional<Tensor>, Tensor> arg_op(const Tensor &x, std::optional<int64_t> dim_in, bool keepdim,
                                                bool is_max, bool values, const char *name) {
    TensorData src = x.data();
    int64_t dim = 0;
    if (dim_in) {
        dim = *dim_in;
    } else {
        src = reshape_data(src, Shape{src.layout.num_elements()});
        keepdim = false;
    }
    size_t nd = src.layout.shape.size();
    size_t d = normalize_dim(dim, nd);
    int64_t size = nd == 0 ? 1 : src.layout.shape[d];
    if (size == 0) {
        throw Error(std::string(name) + "(): Expected reduction dim " + std::to_string(d) + " to have non-zero size.");
    }
    std::vector<bool> mask(nd, false);
    if (nd > 0) mask[d] = true;
    Shape shape = reduced_shape(src.layout.shape, mask, keepdim);
    std::optional<TensorData> vals;
    if (values) vals = uninit_data(shape, src.dtype, src.device());
    TensorData indices = uninit_data(shape, DType::I64, src.device());
    backend::arg_reduce(vals ? &*vals : nullptr, indices, src, d, is_max);
    return {vals ? std::optional<Tensor>(Tensor(*vals)) : std::nullopt, Tensor(indices)};
}

// ref: src/ops/reduce.rs:137-156
Tensor var_op(const Tensor &x, const std::vector<int64_t> &dims, int64_t correction, bool keepdim, bool take_sqrt) {
    const TensorData &src = x.data();
    if (!is_floating_point(src.dtype)) {
        throw Error(std::string("std and var only support floating point dtypes, got ") + name_of(src.dtype));
    }
    std::vector<bool> mask = dims_mask(dims, src.layout.shape.size());
    TensorData out = uninit_data(reduced_shape(src.layout.shape, mask, keepdim), src.dtype, src.device());
    backend::var(out, src, mask, static_cast<double>(correction), take_sqrt);
    return Tensor(out);
}

// ref: src/ops/composite.rs:10-27
Tensor softmax_op(const Tensor &x, int64_t dim, bool log) {
    const TensorData &src = x.data();
    if (!is_floating_point(src.dtype)) {
        throw Error(std::string(log ? "log_softmax" : "softmax") + " is not implemented for " + name_of(src.dtype) +
                    " tensors");
    }
    size_t d = normalize_dim(dim, src.layout.shape.size());
    TensorData out = uninit_data(src.layout.shape, src.dtype, src.device());
    backend::softmax(out, src, d, log);
    return Tensor(out);
}

// ref: src/ops/shape_ops.rs:181-196
Tensor triangle_op(const Tensor &x, int64_t diagonal, bool upper) {
    const TensorData &src = x.data();
    if (src.layout.shape.size() < 2) {
        throw Error(std::string(upper ? "triu" : "tril") + ": input tensor must have at least 2 dimensions");
    }
    TensorData out = uninit_data(src.layout.shape, src.dtype, src.device());
    backend::triangle(out, src, diagonal, upper);
    return Tensor(out);
}

// ref: src/optim/mod.rs:602-640
Tensor fused_op(Fused op, const Tensor &a, const Tensor &b, const Tensor *c) {
    DType dtype = a.dtype();
    DType converted = op.kind == Fused::ScaledAdd || dtype == DType::F64 ? dtype : DType::F32;
    if (!Scalar::of_float(op.scalar).checked_to(converted)) {
        throw Error(std::string("value cannot be converted to type ") + name_of(converted) + " without overflow");
    }
    TensorData out = uninit_data(a.shape(), dtype, a.device());
    backend::fused(op, out, a.data(), b.data(), c ? &c->data() : nullptr);
    return Tensor(out);
}

}  // namespace

void set_fused_promotion(bool on) { g_fused_promotion = on; }

// ---- creation and movement ------------------------------------------------------------------------------

Tensor Tensor::uninit_on(const Shape &shape, DType dtype, Device device) { return Tensor(uninit_data(shape, dtype, device)); }

Tensor Tensor::from_bytes(const void *bytes, DType dtype, const Shape &shape, Device device) {
    TensorData host = uninit_data(shape, dtype, Device::cpu());
    size_t nbytes = static_cast<size_t>(host.layout.num_elements()) * size_in_bytes(dtype);
    if (nbytes) std::memcpy(host.storage->ptr(), bytes, nbytes);
    Tensor t(host);
    return device == Device::cpu() ? t : t.to(device);
}

Tensor Tensor::full(const Shape &shape, Scalar value, DType dtype, Device device) {
    TensorData out = uninit_data(shape, dtype, device);
    backend::fill(out, fill_value(value, dtype));
    return Tensor(out);
}

Tensor Tensor::contiguous() const {
    if (d_.layout.is_contiguous()) return *this;
    return Tensor(clone_data(d_));
}

Tensor Tensor::to(DType dtype) const {
    if (dtype == d_.dtype) return *this;
    return Tensor(cast_data(d_, dtype));
}

Tensor Tensor::to(Device device) const {
    if (device == d_.device()) return *this;
    // A contiguous copy on the source device, then the transfer (device to device goes through
    // host memory, ref: src/backend/mod.rs:250-252).
    Tensor src = contiguous();
    if (d_.device().kind == Device::K::Rocm && device.kind == Device::K::Rocm) return src.to(Device::cpu()).to(device);
    TensorData out = uninit_data(src.shape(), d_.dtype, device);
    if (device.kind == Device::K::Rocm) backend::upload(out, src.data());
    else backend::download(out, src.data());
    return Tensor(out);
}

std::vector<uint8_t> Tensor::to_bytes() const {
    Tensor host = to(Device::cpu()).contiguous();
    size_t size = size_in_bytes(d_.dtype);
    size_t nbytes = static_cast<size_t>(host.num_elements()) * size;
    std::vector<uint8_t> out(nbytes);
    if (nbytes) {
        std::memcpy(out.data(), static_cast<const char *>(host.data().storage->ptr()) + host.storage_offset() * size,
                    nbytes);
    }
    return out;
}

// ---- unary (ref: src/ops/unary.rs:17-57) ---------------------------------------------------------------

Tensor Tensor::unary(UnaryOp op) const {
    const TensorData &src = d_;
    DType dtype = src.dtype;
    DType compute;
    switch (op) {
        case UnaryOp::LogicalNot: compute = dtype; break;
        case UnaryOp::Neg:
            if (dtype == DType::Bool) {
                throw Error("Negation, the `-` operator, on a bool tensor is not supported. If you are trying to "
                            "invert a mask, use `logical_not()` instead.");
            }
            compute = dtype;
            break;
        case UnaryOp::Abs:
        case UnaryOp::Relu:
            if (dtype == DType::Bool) throw Error(std::string(unary_debug_name(op)) + " is not supported for bool tensors");
            compute = dtype;
            break;
        case UnaryOp::Sign: compute = dtype; break;
        case UnaryOp::Silu:
        case UnaryOp::Gelu:
        case UnaryOp::GeluTanh:
        case UnaryOp::LogSigmoid:
            if (!is_floating_point(dtype)) {
                throw Error(std::string(unary_debug_name(op)) + " is not implemented for " + name_of(dtype) + " tensors");
            }
            compute = dtype;
            break;
        default: compute = is_floating_point(dtype) ? dtype : default_dtype(); break;
    }
    DType out_dtype = op == UnaryOp::LogicalNot ? DType::Bool : compute;
    TensorData out = uninit_data(src.layout.shape, out_dtype, src.device());
    backend::unary(op, out, cast_data(src, compute));
    return Tensor(out);
}

// ---- binary (ref: src/ops/binary.rs:68-143) -------------------------------------------------------------

Tensor binary_op(BinaryOp op, const Operand &lhs, const Operand &rhs) {
    Resolved a(lhs), b(rhs);
    std::vector<const TensorData *> tensors;
    if (a.tensor) tensors.push_back(&*a.tensor);
    if (b.tensor) tensors.push_back(&*b.tensor);
    Device device = common_device(tensors);
    ResultType rt;
    a.add_to(rt);
    b.add_to(rt);
    DType common = rt.result();
    DType compute = common;
    if (op == BinaryOp::Div && !is_floating_point(common)) compute = default_dtype();
    else if (op == BinaryOp::LogicalAnd || op == BinaryOp::LogicalOr) compute = DType::Bool;
    if (op == BinaryOp::Sub) {
        if (a.is_bool() && b.is_bool()) {
            throw Error("Subtraction, the `-` operator, with two bool tensors is not supported. Use `not_equal()` "
                        "(logical xor) instead.");
        }
        if (a.is_bool() || b.is_bool()) {
            throw Error("Subtraction, the `-` operator, with a bool tensor is not supported. If you are trying to "
                        "invert a mask, use `logical_not()` instead.");
        }
    }
    if (compute == DType::Bool && op == BinaryOp::Pow) throw Error("pow is not supported for bool tensors");
    if (is_integral(compute) && op == BinaryOp::Pow && !b.tensor && b.scalar.to_i64() < 0) {
        throw Error("Integers to negative integer powers are not allowed.");
    }
    if (op == BinaryOp::BitwiseAnd && is_floating_point(compute)) {
        throw Error(std::string("bitwise_and is not implemented for ") + name_of(compute) + " tensors");
    }
    DType out_dtype = (is_comparison(op) || op == BinaryOp::LogicalAnd || op == BinaryOp::LogicalOr) ? DType::Bool : compute;
    Shape shape = broadcast_shapes(a.shape(), b.shape());
    TensorData out = uninit_data(shape, out_dtype, device);
    bool keeps_scalar = (op == BinaryOp::Mul || op == BinaryOp::Div) && (compute == DType::F16 || compute == DType::BF16);
    if (a.tensor && b.tensor) {
        // On ROCm the library's hmr_binary accepts a half operand next to an F32 one and widens it
        // inside the kernel (exactly, so the bits are those of cast-then-op); the reference would
        // first write an F32 copy of the half tensor (cast_data) and read it back.
        auto half = [](DType d) { return d == DType::F16 || d == DType::BF16; };
        bool arithmetic = op == BinaryOp::Add || op == BinaryOp::Sub || op == BinaryOp::Mul || op == BinaryOp::Div;
        bool mixed = (half(a.tensor->dtype) && b.tensor->dtype == DType::F32) ||
                     (a.tensor->dtype == DType::F32 && half(b.tensor->dtype));
        if (g_fused_promotion && device.kind == Device::K::Rocm && compute == DType::F32 && arithmetic && mixed) {
            backend::binary(op, out, a.tensor->expand_to(shape), b.tensor->expand_to(shape));
        } else {
            backend::binary(op, out, a.materialize(compute, device, shape), b.materialize(compute, device, shape));
        }
    } else {
        bool scalar_first = !a.tensor;
        const Resolved &t = scalar_first ? b : a;
        Scalar s = scalar_first ? a.scalar : b.scalar;
        TensorData td = t.materialize(compute, device, shape);
        if (keeps_scalar) backend::binary_scalar(op, out, td, s.to_f64(), scalar_first);
        else backend::binary_constant(op, out, td, s, scalar_first);
    }
    return Tensor(out);
}

Tensor Tensor::binary(BinaryOp op, const Operand &other) const { return binary_op(op, Operand(*this), other); }

Tensor where_(const Tensor &condition, const Operand &x, const Operand &y) {
    if (condition.dtype() != DType::Bool) {
        throw Error(std::string("where expected condition to be a boolean tensor, but got a tensor with dtype ") +
                    name_of(condition.dtype()));
    }
    ResultType rt;
    Resolved(x).add_to(rt);
    Resolved(y).add_to(rt);
    return select_op(condition, x, y, rt.result());
}

// ref: src/ops/binary.rs:430-470
Tensor Tensor::masked_fill(const Tensor &mask, const Operand &value) const {
    if (mask.dtype() != DType::Bool) {
        throw Error(std::string("masked_fill only supports boolean masks, but got mask with dtype ") + name_of(mask.dtype()));
    }
    if (std::holds_alternative<Scalar>(value)) {
        return select_op(mask, Operand(fill_value(std::get<Scalar>(value), dtype())), Operand(*this), dtype());
    }
    const Tensor &t = std::get<Tensor>(value);
    if (t.num_dims() != 0) {
        throw Error("masked_fill only supports a 0-dimensional value tensor, but got tensor with " +
                    std::to_string(t.num_dims()) + " dimension(s).");
    }
    // The value must fit the dtype like a scalar one; a value of the same dtype always fits and is not read
    // (ref: src/ops/binary.rs:466-472).
    if (t.dtype() != dtype()) fill_value(scalar_value(t), dtype());
    return select_op(mask, Operand(t.to(dtype())), Operand(*this), dtype());
}

// ---- in-place operations (ref: src/ops/mod.rs:308-392, src/ops/binary.rs:594-692) -----------------------

namespace {

// Whether distinct indices of the layout might be one storage element: dimensions longer than 1 sorted by
// stride, each stride must exceed what the smaller ones reach (ref: src/tensor/mod.rs:258-287).
bool may_overlap_internally(const Layout &l) {
    std::vector<std::pair<int64_t, int64_t>> dims;
    for (size_t d = 0; d < l.shape.size(); ++d) {
        if (l.shape[d] == 0) return false;
        if (l.shape[d] > 1) dims.emplace_back(l.strides[d], l.shape[d]);
    }
    std::sort(dims.begin(), dims.end());
    int64_t reach = 0;
    for (const auto &[stride, n] : dims) {
        if (stride <= reach) return true;
        reach += (n - 1) * stride;
    }
    return false;
}

// The element offsets [first, end) a layout can touch; nothing for a layout without elements
// (ref: src/tensor/mod.rs:187-197).
std::optional<std::pair<int64_t, int64_t>> span_of(const Layout &l) {
    int64_t last = l.offset;
    for (size_t d = 0; d < l.shape.size(); ++d) {
        if (l.shape[d] == 0) return std::nullopt;
        last += (l.shape[d] - 1) * l.strides[d];
    }
    return std::make_pair(l.offset, last + 1);
}

// Whether two views may refer to the same memory without being the same view (ref: src/tensor/mod.rs:295-310).
bool partially_overlaps(const TensorData &a, const TensorData &b) {
    if (a.storage != b.storage) return false;
    const auto sa = span_of(a.layout), sb = span_of(b.layout);
    if (!sa || !sb) return false;
    const int64_t ea = static_cast<int64_t>(size_in_bytes(a.dtype)), eb = static_cast<int64_t>(size_in_bytes(b.dtype));
    const bool disjoint = sa->second * ea <= sb->first * eb || sb->second * eb <= sa->first * ea;
    const bool same = a.dtype == b.dtype && a.layout.offset == b.layout.offset && a.layout.shape == b.layout.shape &&
                      a.layout.strides == b.layout.strides;
    return !disjoint && !same;
}

// ref: src/ops/binary.rs:665-692
void check_writable(const TensorData &dst) {
    if (may_overlap_internally(dst.layout)) {
        throw Error("unsupported operation: more than one element of the written-to tensor may refer to a single memory "
                    "location. Please deep_clone() the tensor before performing the operation.");
    }
}

// The end of an in-place operation: `result` was computed out of place on self's device
// (ref: src/ops/mod.rs:317-392).
void finish_in_place(const Tensor &self, const Tensor &result) {
    if (self.shape() != result.shape()) {
        throw Error("output with shape " + shape_str(self.shape()) + " doesn't match the broadcast shape " + shape_str(result.shape()));
    }
    if (!can_cast(result.dtype(), self.dtype())) {
        throw Error(std::string("result type ") + name_of(result.dtype()) + " can't be cast to the desired output type " +
                    name_of(self.dtype()));
    }
    check_writable(self.data());
    backend::copy(self.data(), result.data());
}

}  // namespace

const Tensor &Tensor::binary_(BinaryOp op, const Operand &other) const {
    finish_in_place(*this, binary(op, other));
    return *this;
}

const Tensor &Tensor::clamp_(const Operand &min, const Operand &max) const {
    finish_in_place(*this, clamp(min, max));
    return *this;
}

const Tensor &Tensor::masked_fill_(const Tensor &mask, const Operand &value) const {
    finish_in_place(*this, masked_fill(mask, value));
    return *this;
}

const Tensor &Tensor::copy_(const Tensor &src) const {
    check_writable(d_);
    src.data().layout.expand_to(d_.layout.shape);  // checks that src broadcasts to self
    // The source on self's device: moved (and converted) if it is elsewhere, copied if it partially overlaps self.
    Tensor s = src;
    if (src.device() != device()) s = src.to(dtype()).to(device());
    else if (partially_overlaps(d_, src.data())) s = Tensor(clone_data(src.data()));
    backend::copy(d_, s.data());
    return *this;
}

const Tensor &Tensor::fill_(Scalar value) const {
    check_writable(d_);
    backend::fill(d_, fill_value(value, d_.dtype));
    return *this;
}

// ---- reductions (ref: src/ops/reduce.rs:175-405) --------------------------------------------------------

Tensor Tensor::sum() const { return reduce_op(ReduceOp::Sum, *this, {}, false, "sum"); }
Tensor Tensor::sum_dim(const std::vector<int64_t> &dims, bool keepdim) const {
    return reduce_op(ReduceOp::Sum, *this, dims, keepdim, "sum");
}

Tensor Tensor::sum_to_size(const Shape &size) const {
    const Shape &shape = d_.layout.shape;
    if (!is_expandable_to(size, shape)) {
        throw Error("size {" + shape_str(size) + "} is not expandable to size {" + shape_str(shape) + "}.");
    }
    size_t lead = shape.size() - size.size();
    std::vector<int64_t> dims;
    for (size_t d = 0; d < shape.size(); ++d) {
        if (d < lead || (size[d - lead] == 1 && shape[d] != 1)) dims.push_back(static_cast<int64_t>(d));
    }
    if (dims.empty()) return *this;
    Tensor summed = reduce_op(ReduceOp::Sum, *this, dims, true, "sum");
    return Tensor(reshape_data(summed.data(), size));
}

Tensor Tensor::mean() const { return reduce_op(ReduceOp::Mean, *this, {}, false, "mean"); }
Tensor Tensor::mean_dim(const std::vector<int64_t> &dims, bool keepdim) const {
    return reduce_op(ReduceOp::Mean, *this, dims, keepdim, "mean");
}
Tensor Tensor::prod() const { return reduce_op(ReduceOp::Prod, *this, {}, false, "prod"); }
Tensor Tensor::prod_dim(int64_t dim, bool keepdim) const { return reduce_op(ReduceOp::Prod, *this, {dim}, keepdim, "prod"); }
Tensor Tensor::max() const { return reduce_op(ReduceOp::Max, *this, {}, false, "max"); }
Tensor Tensor::min() const { return reduce_op(ReduceOp::Min, *this, {}, false, "min"); }

ValuesAndIndices Tensor::max_dim(int64_t dim, bool keepdim) const {
    auto r = arg_op(*this, dim, keepdim, true, true, "max");
    return ValuesAndIndices{*r.first, r.second};
}
ValuesAndIndices Tensor::min_dim(int64_t dim, bool keepdim) const {
    auto r = arg_op(*this, dim, keepdim, false, true, "min");
    return ValuesAndIndices{*r.first, r.second};
}
Tensor Tensor::argmax() const { return arg_op(*this, std::nullopt, false, true, false, "argmax").second; }
Tensor Tensor::argmin() const { return arg_op(*this, std::nullopt, false, false, false, "argmin").second; }
Tensor Tensor::argmax_dim(int64_t dim, bool keepdim) const { return arg_op(*this, dim, keepdim, true, false, "argmax").second; }
Tensor Tensor::argmin_dim(int64_t dim, bool keepdim) const { return arg_op(*this, dim, keepdim, false, false, "argmin").second; }

Tensor Tensor::var(int64_t correction) const { return var_op(*this, {}, correction, false, false); }
Tensor Tensor::var_dim(const std::vector<int64_t> &dims, int64_t correction, bool keepdim) const {
    return var_op(*this, dims, correction, keepdim, false);
}
Tensor Tensor::std(int64_t correction) const { return var_op(*this, {}, correction, false, true); }
Tensor Tensor::std_dim(const std::vector<int64_t> &dims, int64_t correction, bool keepdim) const {
    return var_op(*this, dims, correction, keepdim, true);
}

Tensor Tensor::all() const { return reduce_op(ReduceOp::All, *this, {}, false, "all"); }
Tensor Tensor::any() const { return reduce_op(ReduceOp::Any, *this, {}, false, "any"); }
Tensor Tensor::all_dim(const std::vector<int64_t> &dims, bool keepdim) const {
    return reduce_op(ReduceOp::All, *this, dims, keepdim, "all");
}
Tensor Tensor::any_dim(const std::vector<int64_t> &dims, bool keepdim) const {
    return reduce_op(ReduceOp::Any, *this, dims, keepdim, "any");
}

Tensor Tensor::softmax(int64_t dim) const { return softmax_op(*this, dim, false); }
Tensor Tensor::log_softmax(int64_t dim) const { return softmax_op(*this, dim, true); }

// ref: src/ops/reduce.rs:158-170
Tensor exclusive_cumprod(const Tensor &x, size_t dim, bool reverse) {
    const TensorData &src = x.data();
    if (!is_floating_point(src.dtype)) throw Error(std::string("expected a floating point dtype, got ") + name_of(src.dtype));
    if (dim >= src.layout.shape.size()) throw Error("exclusive_cumprod: dimension out of range");
    TensorData out = uninit_data(src.layout.shape, src.dtype, src.device());
    backend::exclusive_cumprod(out, src, dim, reverse);
    return Tensor(out);
}

// ---- triangles and flips (ref: src/ops/shape_ops.rs:181-263) ---------------------------------------------

Tensor Tensor::triu(int64_t diagonal) const { return triangle_op(*this, diagonal, true); }
Tensor Tensor::tril(int64_t diagonal) const { return triangle_op(*this, diagonal, false); }

Tensor Tensor::flip(const std::vector<int64_t> &dims) const {
    const size_t nd = d_.layout.shape.size();
    std::vector<bool> mask = dims.empty() ? std::vector<bool>(nd, false) : dims_mask(dims, nd);
    TensorData out = uninit_data(d_.layout.shape, d_.dtype, d_.device());
    backend::flip(out, d_, mask);
    return Tensor(out);
}

// ---- compositions (ref: src/ops/composite.rs:448-508) ----------------------------------------------------

Tensor Tensor::addcmul(const Tensor &tensor1, const Tensor &tensor2, Scalar value) const {
    return add(tensor1.mul(value).mul(tensor2));
}

Tensor Tensor::addcdiv(const Tensor &tensor1, const Tensor &tensor2, Scalar value) const {
    if (!is_floating_point(tensor1.dtype()) && !is_floating_point(tensor2.dtype())) {
        throw Error("Integer division with addcdiv is no longer supported. Use self.add(tensor1.div(tensor2).mul(value)) "
                    "instead.");
    }
    return add(tensor1.mul(value).div(tensor2));
}

const Tensor &Tensor::addcmul_(const Tensor &tensor1, const Tensor &tensor2, Scalar value) const {
    finish_in_place(*this, addcmul(tensor1, tensor2, value));
    return *this;
}
const Tensor &Tensor::addcdiv_(const Tensor &tensor1, const Tensor &tensor2, Scalar value) const {
    finish_in_place(*this, addcdiv(tensor1, tensor2, value));
    return *this;
}
const Tensor &Tensor::lerp_(const Tensor &end, const Operand &weight) const {
    finish_in_place(*this, lerp(end, weight));
    return *this;
}

Tensor Tensor::lerp(const Tensor &end, const Operand &weight) const {
    Tensor diff = end.sub(*this);
    if (std::holds_alternative<Scalar>(weight)) {
        Scalar w = std::get<Scalar>(weight);
        double wf = w.to_f64();
        if (std::fabs(wf) < 0.5) return add(diff.mul(w));
        return end.sub(diff.mul(Scalar::of_float(1.0 - wf)));
    }
    const Tensor &w = std::get<Tensor>(weight);
    Tensor low = add(w.mul(diff));
    Tensor high = end.sub(diff.mul(w.neg().add(Scalar::of_float(1.0))));
    return where_(w.abs().less(Scalar::of_float(0.5)), low, high);
}

// ---- addr (ref: src/ops/composite.rs:29-114, 210-249, 346-384) --------------------------------------------

namespace {
// ref: src/ops/composite.rs:38-65, rule Strict.
Scalar addr_coefficient(Scalar s, DType dtype, const char *name) {
    if (s.kind == Scalar::K::Bool && dtype != DType::Bool) {
        throw Error(std::string("Boolean ") + name + " only supported for Boolean results");
    }
    if (s.kind == Scalar::K::Float && !is_floating_point(dtype)) {
        throw Error(std::string("For integral input tensors, argument ") + name + " must not be a floating point number");
    }
    auto fits = s.checked_to(dtype);
    if (!fits) throw Error(std::string(name) + "=" + s.str() + " cannot be converted to " + name_of(dtype) + " without overflow");
    return *fits;
}

void check_dims(const Tensor &t, size_t n, const char *what) {
    if (t.num_dims() != n) {
        throw Error(std::string(what) + " must be a " + std::to_string(n) + "-D tensor, got " + std::to_string(t.num_dims()) +
                    "-D tensor");
    }
}
}  // namespace

Tensor Tensor::addr(const Tensor &vec1, const Tensor &vec2, Scalar beta, Scalar alpha) const {
    check_dims(vec1, 1, "vec1");
    check_dims(vec2, 1, "vec2");
    common_device({&d_, &vec1.data(), &vec2.data()});
    // `self` takes full part in the promotion even when it is zero-dimensional.
    const DType dtype = promote_types(promote_types(d_.dtype, vec1.dtype()), vec2.dtype());
    const Tensor input = to(dtype), v1 = vec1.to(dtype), v2 = vec2.to(dtype);
    const Shape shape{v1.shape()[0], v2.shape()[0]};
    const TensorData c = input.data().expand_to(shape);  // fails for an input that doesn't broadcast
    beta = addr_coefficient(beta, dtype, "beta");
    alpha = addr_coefficient(alpha, dtype, "alpha");
    if (is_floating_point(dtype)) {
        // Rounded to the dtype whatever kind of scalar they are (ref: src/ops/composite.rs:99-114).
        beta = Scalar::of_float(round_through(beta.to_f64(), dtype));
        alpha = Scalar::of_float(round_through(alpha.to_f64(), dtype));
    }
    TensorData out = uninit_data(shape, dtype, v1.device());
    backend::addr(out, v1.data(), v2.data(), c, alpha, beta);
    return Tensor(out);
}

// ---- the optimizers' steps (ref: src/optim/mod.rs:569-616) -----------------------------------------------

namespace optim {
Tensor scaled_add(const Tensor &a, const Tensor &b, double alpha) { return fused_op(Fused{Fused::ScaledAdd, alpha}, a, b, nullptr); }
Tensor lerp(const Tensor &a, const Tensor &b, double weight) { return fused_op(Fused{Fused::Lerp, weight}, a, b, nullptr); }
Tensor addcmul(const Tensor &a, const Tensor &b, const Tensor &c, double value) {
    return fused_op(Fused{Fused::Addcmul, value}, a, b, &c);
}
Tensor addcdiv(const Tensor &a, const Tensor &b, const Tensor &c, double value) {
    return fused_op(Fused{Fused::Addcdiv, value}, a, b, &c);
}

namespace {
DType computation(DType dtype) { return dtype == DType::F16 || dtype == DType::BF16 ? DType::F32 : dtype; }

// ref: src/optim/mod.rs:618-640
void check_coefficient(double value, DType dtype) {
    if (!Scalar::of_float(value).checked_to(dtype)) {
        throw Error(std::string("value cannot be converted to type ") + name_of(dtype) + " without overflow");
    }
}

void check_like(const Tensor &p, const Tensor &t, const char *what) {
    if (t.shape() != p.shape() || t.dtype() != p.dtype() || t.device() != p.device()) {
        throw Error(std::string(what) + " must have the parameter's shape, dtype and device");
    }
}
}  // namespace

Tensor sgd_step(const Tensor &p, const Tensor &grad_in, std::optional<Tensor> &momentum_buffer, const SgdOptions &o) {
    check_like(p, grad_in, "the gradient");
    if (o.nesterov && (o.momentum <= 0.0 || o.dampening != 0.0)) {
        throw Error("Nesterov momentum requires a momentum and zero dampening");
    }
    // ref: src/optim/sgd.rs:257-263, 275-299: every alpha of the step, in the parameter's dtype.
    check_coefficient(-o.lr, p.dtype());
    if (o.weight_decay != 0.0) check_coefficient(o.weight_decay, p.dtype());
    if (o.momentum != 0.0) {
        if (momentum_buffer) {
            check_like(p, *momentum_buffer, "the momentum buffer");
            check_coefficient(1.0 - o.dampening, p.dtype());
        }
        if (o.nesterov) check_coefficient(o.momentum, p.dtype());
    }
    Tensor grad = o.maximize ? grad_in.neg() : grad_in;
    if (o.weight_decay != 0.0) grad = scaled_add(grad, p, o.weight_decay);
    if (o.momentum != 0.0) {
        if (!momentum_buffer) {
            // A copy of its own: the gradient may be the caller's tensor.
            momentum_buffer = grad.mul(Scalar::of_int(1));
        } else {
            Tensor scaled = momentum_buffer->mul(Scalar::of_float(o.momentum));
            momentum_buffer = scaled_add(scaled, grad, 1.0 - o.dampening);
        }
        grad = o.nesterov ? scaled_add(grad, *momentum_buffer, o.momentum) : *momentum_buffer;
    }
    return scaled_add(p, grad, -o.lr);
}

Tensor adam_step(const Tensor &p_in, const Tensor &grad_in, std::optional<AdamState> &state, const AdamOptions &o,
                 bool decoupled_weight_decay) {
    check_like(p_in, grad_in, "the gradient");
    const DType dtype = p_in.dtype();
    const double next = static_cast<double>(static_cast<float>((state ? state->step : 0.0) + 1.0));
    auto step_size = [&](double step) { return o.lr / (1.0 - std::pow(o.beta1, step)); };
    // ref: src/optim/adam.rs:291-304
    check_coefficient(-step_size(next), computation(dtype));
    if (o.weight_decay != 0.0 && !decoupled_weight_decay) check_coefficient(o.weight_decay, dtype);
    if (state) {
        check_like(p_in, state->exp_avg, "exp_avg");
        check_like(p_in, state->exp_avg_sq, "exp_avg_sq");
        if (o.amsgrad) {
            if (!state->max_exp_avg_sq) throw Error("the state has no max_exp_avg_sq, but amsgrad is set");
            check_like(p_in, *state->max_exp_avg_sq, "max_exp_avg_sq");
        }
    } else {
        Tensor zeros = Tensor::full(p_in.shape(), Scalar::of_int(0), dtype, p_in.device());
        state = AdamState{0.0, zeros, zeros, o.amsgrad ? std::optional<Tensor>(zeros) : std::nullopt};
    }
    Tensor p = p_in;
    Tensor grad = o.maximize ? grad_in.neg() : grad_in;
    state->step = next;
    if (o.weight_decay != 0.0) {
        if (decoupled_weight_decay) p = p.mul(Scalar::of_float(1.0 - o.lr * o.weight_decay));
        else grad = scaled_add(grad, p, o.weight_decay);
    }
    state->exp_avg = lerp(state->exp_avg, grad, 1.0 - o.beta1);
    state->exp_avg_sq = addcmul(state->exp_avg_sq.mul(Scalar::of_float(o.beta2)), grad, grad, 1.0 - o.beta2);
    const double bias_correction2 = 1.0 - std::pow(o.beta2, next);
    const double bias_correction2_sqrt = std::pow(bias_correction2, 0.5);
    const Tensor *second = &state->exp_avg_sq;
    if (o.amsgrad && state->max_exp_avg_sq) {
        state->max_exp_avg_sq = state->max_exp_avg_sq->maximum(state->exp_avg_sq);
        second = &*state->max_exp_avg_sq;
    }
    Tensor denom = second->sqrt().div(Scalar::of_float(bias_correction2_sqrt)).add(Scalar::of_float(o.eps));
    return addcdiv(p, state->exp_avg, denom, -step_size(next));
}
}  // namespace optim

}  // namespace homura
