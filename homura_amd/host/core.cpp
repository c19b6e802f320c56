// dtype rules, shape algebra, layouts and views of the host layer. See homura.hpp for the map to
// the reference's files.
#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstring>
#include <sstream>

#include "../csrc/elem.hpp"
#include "homura.hpp"

namespace homura {

// ---- dtype (ref: src/dtype.rs) ---------------------------------------------------------------------------

Kind kind_of(DType d) {
    switch (d) {
        case DType::Bool: return Kind::Bool;
        case DType::F16:
        case DType::BF16:
        case DType::F32:
        case DType::F64: return Kind::Float;
        default: return Kind::Int;
    }
}

size_t size_in_bytes(DType d) { return static_cast<size_t>(hmr::dtype_size(static_cast<int>(d))); }

const char *name_of(DType d) {
    static const char *names[] = {"bool", "u8", "i8", "i16", "i32", "i64", "f16", "bf16", "f32", "f64"};
    return names[static_cast<int>(d)];
}

namespace {
std::atomic<int> g_default_dtype{static_cast<int>(DType::F32)};
}

DType default_dtype() { return static_cast<DType>(g_default_dtype.load()); }

void set_default_dtype(DType d) {
    if (!is_floating_point(d)) throw Error(std::string("the default dtype must be floating point, got ") + name_of(d));
    g_default_dtype.store(static_cast<int>(d));
}

double Scalar::to_f64() const { return kind == K::Float ? f : static_cast<double>(i); }

int64_t Scalar::to_i64() const { return kind == K::Float ? hmr::f64_to_i64_sat(f) : i; }

bool Scalar::to_bool() const { return kind == K::Float ? f != 0.0 : i != 0; }

DType Scalar::dtype() const {
    switch (kind) {
        case K::Bool: return DType::Bool;
        case K::Int: return DType::I64;
        default: return default_dtype();
    }
}

std::string Scalar::str() const {
    std::ostringstream s;
    if (kind == K::Bool) s << (i ? "true" : "false");
    else if (kind == K::Int) s << i;
    else s << f;
    return s.str();
}

double float_max(DType d) {
    switch (d) {
        case DType::F16: return 65504.0;
        case DType::BF16: return 3.3895313892515355e38;
        case DType::F32: return 3.4028234663852886e38;
        default: return 1.7976931348623157e308;
    }
}

void int_range(DType d, int64_t &lo, int64_t &hi) {
    switch (d) {
        case DType::Bool: lo = 0; hi = 1; break;
        case DType::U8: lo = 0; hi = 255; break;
        case DType::I8: lo = -128; hi = 127; break;
        case DType::I16: lo = -32768; hi = 32767; break;
        case DType::I32: lo = INT32_MIN; hi = INT32_MAX; break;
        default: lo = INT64_MIN; hi = INT64_MAX; break;
    }
}

std::optional<Scalar> Scalar::checked_to(DType dtype) const {
    switch (kind_of(dtype)) {
        case Kind::Bool: return Scalar::of_bool(to_bool());
        case Kind::Float: {
            double v = to_f64();
            if (std::isfinite(v) && std::fabs(v) > float_max(dtype)) return std::nullopt;
            return *this;
        }
        default: {
            int64_t lo, hi;
            int_range(dtype, lo, hi);
            if (kind == K::Bool) return Scalar::of_int(i);
            if (kind == K::Int) {
                int64_t min = dtype == DType::U8 ? -hi : lo;  // like PyTorch, -255..-1 wrap for U8
                if (i < min || i > hi) return std::nullopt;
                return Scalar::of_int(i);
            }
            // Floats must lie in [MIN, MAX + 1) before truncation; 2^63 exactly for I64.
            double upper = dtype == DType::I64 ? 9223372036854775808.0 : static_cast<double>(hi) + 1.0;
            if (!(f >= static_cast<double>(lo) && f < upper)) return std::nullopt;
            return Scalar::of_int(hmr::f64_to_i64_sat(f));
        }
    }
}

DType promote_types(DType a, DType b) {
    if (a == b) return a;
    Kind ka = kind_of(a), kb = kind_of(b);
    if (ka == Kind::Bool) return b;
    if (kb == Kind::Bool) return a;
    if (ka == Kind::Float && kb == Kind::Float) return (a == DType::F64 || b == DType::F64) ? DType::F64 : DType::F32;
    if (ka == Kind::Float) return a;
    if (kb == Kind::Float) return b;
    auto rank = [](DType d) {
        switch (d) {
            case DType::I8: return 1;
            case DType::I16: return 2;
            case DType::I32: return 3;
            case DType::I64: return 4;
            default: return 0;
        }
    };
    if ((a == DType::U8 && b == DType::I8) || (a == DType::I8 && b == DType::U8)) return DType::I16;
    if (a == DType::U8) return b;
    if (b == DType::U8) return a;
    return rank(a) >= rank(b) ? a : b;
}

bool can_cast(DType from, DType to) {
    return !((is_floating_point(from) && !is_floating_point(to)) || (from != DType::Bool && to == DType::Bool));
}

namespace {
void update(std::optional<DType> &slot, DType d) { slot = slot ? promote_types(*slot, d) : d; }

std::optional<DType> combine(std::optional<DType> higher, std::optional<DType> lower) {
    if (!higher) return lower;
    if (!lower) return higher;
    if (is_floating_point(*higher)) return higher;
    if (*higher == DType::Bool || is_floating_point(*lower)) return promote_types(*higher, *lower);
    return higher;
}
}  // namespace

ResultType &ResultType::tensor(DType dtype, size_t num_dims) {
    update(num_dims == 0 ? zero_dim_ : dim_, dtype);
    return *this;
}

ResultType &ResultType::scalar(Scalar s) {
    update(scalar_, s.dtype());
    return *this;
}

DType ResultType::result() const {
    auto r = combine(dim_, combine(zero_dim_, scalar_));
    if (!r) throw Error("result_type needs at least one operand");
    return *r;
}

namespace {
template <class T>
uint64_t bits_of(T v) {
    uint64_t b = 0;
    std::memcpy(&b, &v, sizeof v);
    return b;
}

template <class T>
uint64_t scalar_bits_as(Scalar s) {
    switch (s.kind) {
        case Scalar::K::Bool: return bits_of(hmr::Conv<T>::from_bool(s.i != 0));
        case Scalar::K::Int: return bits_of(hmr::Conv<T>::from_i64(s.i));
        default: return bits_of(hmr::Conv<T>::from_f64(s.f));
    }
}
}  // namespace

uint64_t scalar_bits(Scalar value, DType dtype) {
    switch (dtype) {
        case DType::Bool: return scalar_bits_as<hmr::bool_t>(value);
        case DType::U8: return scalar_bits_as<uint8_t>(value);
        case DType::I8: return scalar_bits_as<int8_t>(value);
        case DType::I16: return scalar_bits_as<int16_t>(value);
        case DType::I32: return scalar_bits_as<int32_t>(value);
        case DType::I64: return scalar_bits_as<int64_t>(value);
        case DType::F16: return scalar_bits_as<hmr::f16_t>(value);
        case DType::BF16: return scalar_bits_as<hmr::bf16_t>(value);
        case DType::F32: return scalar_bits_as<float>(value);
        default: return scalar_bits_as<double>(value);
    }
}

double round_through(double value, DType dtype) {
    const float narrow = static_cast<float>(value);
    switch (dtype) {
        case DType::F16: return hmr::Conv<hmr::f16_t>::to_f64(hmr::f16_round(narrow));
        case DType::BF16: return hmr::Conv<hmr::bf16_t>::to_f64(hmr::bf16_round(narrow));
        case DType::F32: return static_cast<double>(narrow);
        default: return value;
    }
}

// ---- shapes (ref: src/shape.rs) --------------------------------------------------------------------------

std::string shape_str(const Shape &s) {
    std::ostringstream o;
    o << "[";
    for (size_t i = 0; i < s.size(); ++i) o << (i ? ", " : "") << s[i];
    o << "]";
    return o.str();
}

size_t normalize_dim(int64_t dim, size_t num_dims) {
    int64_t n = static_cast<int64_t>(num_dims == 0 ? 1 : num_dims);  // a 0-dim tensor takes 0 and -1
    if (dim < -n || dim >= n) {
        std::ostringstream m;
        m << "Dimension out of range (expected to be in range of [" << -n << ", " << n - 1 << "], but got " << dim
          << ")";
        throw Error(m.str());
    }
    return static_cast<size_t>(dim < 0 ? dim + n : dim);
}

std::vector<bool> dims_mask(const std::vector<int64_t> &dims, size_t num_dims) {
    if (dims.empty()) return std::vector<bool>(num_dims, true);
    std::vector<bool> mask(std::max<size_t>(num_dims, 1), false);
    for (int64_t d : dims) {
        size_t k = normalize_dim(d, num_dims);
        if (mask[k]) throw Error("dim " + std::to_string(k) + " appears multiple times in the list of dims");
        mask[k] = true;
    }
    mask.resize(num_dims);
    return mask;
}

Strides contiguous_strides(const Shape &shape) {
    Strides st(shape.size(), 0);
    int64_t acc = 1;
    for (size_t i = shape.size(); i-- > 0;) {
        st[i] = acc;
        if (__builtin_mul_overflow(acc, std::max<int64_t>(shape[i], 1), &acc)) {
            throw Error("shape " + shape_str(shape) + " has too many elements");
        }
    }
    return st;
}

bool is_contiguous(const Shape &shape, const Strides &strides) {
    for (int64_t n : shape) {
        if (n == 0) return true;
    }
    int64_t expected = 1;
    for (size_t i = shape.size(); i-- > 0;) {
        if (shape[i] == 1) continue;
        if (strides[i] != expected) return false;
        expected *= shape[i];
    }
    return true;
}

bool is_expandable_to(const Shape &shape, const Shape &desired) {
    if (shape.size() > desired.size()) return false;
    size_t lead = desired.size() - shape.size();
    for (size_t i = 0; i < shape.size(); ++i) {
        if (shape[i] != desired[lead + i] && shape[i] != 1) return false;
    }
    return true;
}

Shape broadcast_shapes(const Shape &a, const Shape &b) {
    size_t n = std::max(a.size(), b.size());
    Shape out(n, 0);
    for (size_t i = 0; i < n; ++i) {
        int64_t da = i < n - a.size() ? 1 : a[i - (n - a.size())];
        int64_t db = i < n - b.size() ? 1 : b[i - (n - b.size())];
        if (da == db || db == 1) out[i] = da;
        else if (da == 1) out[i] = db;
        else {
            std::ostringstream m;
            m << "The size of tensor a (" << da << ") must match the size of tensor b (" << db
              << ") at non-singleton dimension " << i;
            throw Error(m.str());
        }
    }
    return out;
}

Shape infer_size(const std::vector<int64_t> &spec, int64_t num_elements) {
    auto invalid = [&]() -> Error {
        return Error("shape '" + shape_str(spec) + "' is invalid for input of size " + std::to_string(num_elements));
    };
    std::optional<size_t> infer;
    int64_t known = 1;
    for (size_t i = 0; i < spec.size(); ++i) {
        int64_t d = spec[i];
        if (d == -1) {
            if (infer) throw Error("only one dimension can be inferred");
            infer = i;
        } else if (d < 0) {
            throw Error("invalid shape dimension " + std::to_string(d));
        } else if (__builtin_mul_overflow(known, d, &known)) {
            throw invalid();
        }
    }
    Shape out(spec.size());
    for (size_t i = 0; i < spec.size(); ++i) out[i] = std::max<int64_t>(spec[i], 0);
    if (infer) {
        if (known == 0 || num_elements % known != 0) throw invalid();
        out[*infer] = num_elements / known;
    } else if (known != num_elements) {
        throw invalid();
    }
    return out;
}

// PyTorch's computeStride, as ref: src/shape.rs:686-742 restates it.
std::optional<Strides> compute_view_strides(const Shape &old_shape, const Strides &old_strides, const Shape &new_shape) {
    if (old_shape.empty()) return Strides(new_shape.size(), 1);
    int64_t numel = 1;
    for (int64_t n : old_shape) numel *= n;
    if (numel == 0 && old_shape == new_shape) return old_strides;
    Strides ns(new_shape.size(), 0);
    if (numel == 0) {
        for (size_t d = new_shape.size(); d-- > 0;) {
            if (d == new_shape.size() - 1) ns[d] = 1;
            else if (__builtin_mul_overflow(std::max<int64_t>(new_shape[d + 1], 1), ns[d + 1], &ns[d])) return std::nullopt;
        }
        return ns;
    }
    int64_t view_d = static_cast<int64_t>(new_shape.size()) - 1;
    int64_t chunk_base = old_strides.back();
    int64_t tensor_numel = 1, view_numel = 1;
    for (size_t td = old_shape.size(); td-- > 0;) {
        tensor_numel *= old_shape[td];
        bool ends = td == 0;
        if (!ends && old_shape[td - 1] != 1) {
            int64_t prod = 0;
            bool ok = !__builtin_mul_overflow(tensor_numel, chunk_base, &prod);
            ends = !(ok && old_strides[td - 1] == prod);
        }
        if (ends) {
            while (view_d >= 0 && (view_numel < tensor_numel || new_shape[view_d] == 1)) {
                if (__builtin_mul_overflow(view_numel, chunk_base, &ns[view_d])) return std::nullopt;
                view_numel *= new_shape[view_d];
                --view_d;
            }
            if (view_numel != tensor_numel) return std::nullopt;
            if (td > 0) {
                chunk_base = old_strides[td - 1];
                tensor_numel = 1;
                view_numel = 1;
            }
        }
    }
    if (view_d != -1) return std::nullopt;
    return ns;
}

std::optional<std::vector<MergedDim>> merge_dims(const Shape &shape, const std::vector<const Strides *> &strides) {
    for (int64_t n : shape) {
        if (n == 0) return std::nullopt;
    }
    std::vector<MergedDim> dims;
    const size_t N = strides.size();
    for (size_t i = 0; i < shape.size(); ++i) {
        int64_t size = shape[i];
        if (size == 1) continue;
        std::vector<int64_t> st(N);
        for (size_t k = 0; k < N; ++k) st[k] = (*strides[k])[i];
        if (!dims.empty()) {
            MergedDim &outer = dims.back();
            bool joins = true;
            for (size_t k = 0; joins && k < N; ++k) {
                int64_t prod = 0;
                joins = !__builtin_mul_overflow(st[k], size, &prod) && prod == outer.strides[k];
            }
            if (joins) {
                outer.size *= size;
                outer.strides = st;
                continue;
            }
        }
        dims.push_back(MergedDim{size, st});
    }
    return dims;
}

// ---- Layout / TensorData -----------------------------------------------------------------------------------

std::string Device::str() const { return kind == K::Cpu ? "cpu" : "rocm:" + std::to_string(index); }

Layout Layout::contiguous(Shape shape) {
    Layout l;
    l.strides = contiguous_strides(shape);
    l.shape = std::move(shape);
    l.offset = 0;
    return l;
}

int64_t Layout::num_elements() const {
    int64_t n = 1;
    for (int64_t s : shape) n *= s;
    return n;
}

Layout Layout::expand_to(const Shape &target) const {
    size_t n = target.size(), m = shape.size();
    if (m > n) throw Error("cannot broadcast shape " + shape_str(shape) + " to " + shape_str(target));
    Strides st(n, 0);
    for (size_t i = 0; i < m; ++i) {
        int64_t src = shape[i], dst = target[n - m + i];
        if (src == dst) {
            st[n - m + i] = strides[i];
        } else if (src != 1) {
            std::ostringstream msg;
            msg << "The expanded size of the tensor (" << dst << ") must match the existing size (" << src
                << ") at non-singleton dimension " << n - m + i << ". Target sizes: " << shape_str(target)
                << ". Tensor sizes: " << shape_str(shape);
            throw Error(msg.str());
        }
    }
    return Layout{target, st, offset};
}

Layout Layout::select(size_t dim, int64_t index) const {
    Layout l = *this;
    l.offset += index * strides[dim];
    l.shape.erase(l.shape.begin() + static_cast<long>(dim));
    l.strides.erase(l.strides.begin() + static_cast<long>(dim));
    return l;
}

TensorData TensorData::expand_to(const Shape &shape) const { return TensorData{storage, layout.expand_to(shape), dtype}; }

// ---- views (ref: src/tensor/view.rs) ---------------------------------------------------------------------

Tensor Tensor::reshape(const std::vector<int64_t> &spec) const {
    const Layout &l = d_.layout;
    Shape shape = infer_size(spec, l.num_elements());
    if (auto st = compute_view_strides(l.shape, l.strides, shape)) {
        return Tensor(TensorData{d_.storage, Layout{shape, *st, l.offset}, d_.dtype});
    }
    Tensor c = contiguous();
    return Tensor(TensorData{c.d_.storage, Layout::contiguous(shape), d_.dtype});
}

Tensor Tensor::permute(const std::vector<int64_t> &dims) const {
    const Layout &l = d_.layout;
    size_t n = l.shape.size();
    if (dims.size() != n) {
        throw Error("permute(): number of dimensions in the tensor input does not match the length of the desired "
                    "ordering of dimensions i.e. input.dim() = " +
                    std::to_string(n) + " is not equal to len(dims) = " + std::to_string(dims.size()));
    }
    std::vector<bool> seen(n, false);
    Layout out{Shape(n), Strides(n), l.offset};
    for (size_t i = 0; i < n; ++i) {
        size_t d = normalize_dim(dims[i], n);
        if (seen[d]) throw Error("permute(): duplicate dims are not allowed.");
        seen[d] = true;
        out.shape[i] = l.shape[d];
        out.strides[i] = l.strides[d];
    }
    return Tensor(TensorData{d_.storage, out, d_.dtype});
}

Tensor Tensor::transpose(int64_t dim0, int64_t dim1) const {
    Layout l = d_.layout;
    size_t n = l.shape.size();
    size_t a = normalize_dim(dim0, n), b = normalize_dim(dim1, n);
    if (n == 0) return *this;
    std::swap(l.shape[a], l.shape[b]);
    std::swap(l.strides[a], l.strides[b]);
    return Tensor(TensorData{d_.storage, l, d_.dtype});
}

Tensor Tensor::expand(const std::vector<int64_t> &spec) const {
    const Layout &l = d_.layout;
    if (spec.size() < l.shape.size()) {
        throw Error("expand: the number of sizes provided (" + std::to_string(spec.size()) +
                    ") must be greater or equal to the number of dimensions in the tensor (" +
                    std::to_string(l.shape.size()) + ")");
    }
    Shape target(spec.size());
    size_t lead = spec.size() - l.shape.size();
    for (size_t i = 0; i < spec.size(); ++i) {
        if (spec[i] == -1) {
            if (i < lead) throw Error("expand: -1 is not allowed in a leading, non-existing dimension " + std::to_string(i));
            target[i] = l.shape[i - lead];
        } else if (spec[i] < 0) {
            throw Error("invalid shape dimension " + std::to_string(spec[i]));
        } else {
            target[i] = spec[i];
        }
    }
    return Tensor(TensorData{d_.storage, l.expand_to(target), d_.dtype});
}

Tensor Tensor::unsqueeze(int64_t dim) const {
    Layout l = d_.layout;
    size_t n = l.shape.size();
    int64_t range = static_cast<int64_t>(n) + 1;
    if (dim < -range || dim >= range) throw Error("Dimension out of range for unsqueeze: " + std::to_string(dim));
    size_t d = static_cast<size_t>(dim < 0 ? dim + range : dim);
    int64_t stride = 1;
    if (d < n && __builtin_mul_overflow(l.shape[d], l.strides[d], &stride)) stride = 1;
    l.shape.insert(l.shape.begin() + static_cast<long>(d), 1);
    l.strides.insert(l.strides.begin() + static_cast<long>(d), stride);
    return Tensor(TensorData{d_.storage, l, d_.dtype});
}

// ref: src/tensor/view.rs (view_layout): a reshape that must not copy.
Tensor Tensor::view(const std::vector<int64_t> &spec) const {
    const Layout &l = d_.layout;
    Shape shape = infer_size(spec, l.num_elements());
    auto st = compute_view_strides(l.shape, l.strides, shape);
    if (!st) {
        throw Error("view size is not compatible with input tensor's size and stride (at least one dimension spans "
                    "across two contiguous subspaces). Use .reshape(...) instead.");
    }
    return Tensor(TensorData{d_.storage, Layout{shape, *st, l.offset}, d_.dtype});
}

Tensor Tensor::expand_as(const Tensor &other) const {
    return expand(std::vector<int64_t>(other.shape().begin(), other.shape().end()));
}

namespace {
Layout without_dims(const Layout &l, const std::vector<bool> &remove) {
    Layout out{{}, {}, l.offset};
    for (size_t d = 0; d < l.shape.size(); ++d) {
        if (remove[d]) continue;
        out.shape.push_back(l.shape[d]);
        out.strides.push_back(l.strides[d]);
    }
    return out;
}
}  // namespace

// Removes all dimensions of size 1.
Tensor Tensor::squeeze() const {
    const Layout &l = d_.layout;
    std::vector<bool> remove(l.shape.size());
    for (size_t d = 0; d < l.shape.size(); ++d) remove[d] = l.shape[d] == 1;
    return Tensor(TensorData{d_.storage, without_dims(l, remove), d_.dtype});
}

// Removes the given dimensions where they have size 1; an empty list removes none.
Tensor Tensor::squeeze_dim(const std::vector<int64_t> &dims) const {
    const Layout &l = d_.layout;
    std::vector<bool> remove(l.shape.size(), false);
    if (!dims.empty()) {
        std::vector<bool> mask = dims_mask(dims, l.shape.size());
        for (size_t d = 0; d < l.shape.size(); ++d) remove[d] = mask[d] && l.shape[d] == 1;
    }
    return Tensor(TensorData{d_.storage, without_dims(l, remove), d_.dtype});
}

// All windows of `size` elements, `step` apart, along `dim`, as a new last dimension.
Tensor Tensor::unfold(int64_t dim, int64_t size, int64_t step) const {
    const Layout &l = d_.layout;
    const size_t nd = l.shape.size();
    const size_t d = normalize_dim(dim, nd);
    const int64_t max = nd == 0 ? 1 : l.shape[d];
    if (size < 0 || size > max) {
        throw Error("maximum size for tensor at dimension " + std::to_string(d) + " is " + std::to_string(max) +
                    " but size is " + std::to_string(size));
    }
    if (step <= 0) throw Error("step is " + std::to_string(step) + " but must be > 0");
    Layout out = l;
    out.shape.push_back(size);
    out.strides.push_back(nd == 0 ? 1 : l.strides[d]);
    if (nd > 0) {
        out.shape[d] = (l.shape[d] - size) / step + 1;
        // With a single window the stride is never used, and a huge step may not fit.
        int64_t stride;
        out.strides[d] = __builtin_mul_overflow(l.strides[d], step, &stride) ? l.strides[d] : stride;
    }
    return Tensor(TensorData{d_.storage, out, d_.dtype});
}

// A view with an explicit shape, strides and storage offset (in elements); it must lie inside the storage
// (ref: src/tensor/mod.rs:199-218).
Tensor Tensor::as_strided(const Shape &size, const Strides &stride, int64_t storage_offset) const {
    if (size.size() != stride.size()) throw Error("mismatch in length of strides and shape");
    bool empty = false, fits = storage_offset >= 0;
    int64_t end = storage_offset;
    for (size_t d = 0; d < size.size() && fits; ++d) {
        if (size[d] < 0 || stride[d] < 0) throw Error("as_strided: sizes and strides must not be negative");
        if (size[d] == 0) empty = true;
        int64_t reach;
        if (size[d] > 0) fits = !__builtin_mul_overflow(size[d] - 1, stride[d], &reach) && !__builtin_add_overflow(end, reach, &end);
    }
    const int64_t item = static_cast<int64_t>(size_in_bytes(d_.dtype));
    int64_t needed = 0;
    if (!empty && fits) fits = !__builtin_add_overflow(end, int64_t{1}, &end) && !__builtin_mul_overflow(end, item, &needed);
    if (empty) needed = 0;
    const int64_t have = static_cast<int64_t>(d_.storage->nbytes());
    if (!fits || needed > have) {
        throw Error("setStorage: sizes " + shape_str(size) + ", strides " + shape_str(stride) + ", storage offset " +
                    std::to_string(storage_offset) + ", and itemsize " + std::to_string(item) + " requiring a storage size of " +
                    (fits ? std::to_string(needed) : std::string("more than usize::MAX")) +
                    " are out of bounds for storage of size " + std::to_string(have));
    }
    return Tensor(TensorData{d_.storage, Layout{size, stride, storage_offset}, d_.dtype});
}

Tensor Tensor::narrow(int64_t dim, int64_t start, int64_t length) const {
    Layout l = d_.layout;
    if (l.shape.empty()) throw Error("narrow() cannot be applied to a 0-dim tensor.");
    size_t d = normalize_dim(dim, l.shape.size());
    int64_t size = l.shape[d];
    if (start < -size || start > size) {
        throw Error("start out of range (expected to be in range of [" + std::to_string(-size) + ", " +
                    std::to_string(size) + "], but got " + std::to_string(start) + ")");
    }
    if (start < 0) start += size;
    if (length < 0 || start + length > size) {
        throw Error("start (" + std::to_string(start) + ") + length (" + std::to_string(length) +
                    ") exceeds dimension size (" + std::to_string(size) + ").");
    }
    l.offset += start * l.strides[d];
    l.shape[d] = length;
    return Tensor(TensorData{d_.storage, l, d_.dtype});
}

// ref: src/tensor/view.rs:32-58, 317-333: a Python-style slice start:end:step; bounds may be negative and are
// clamped into 0..=size.
Tensor Tensor::slice(int64_t dim, std::optional<int64_t> start, std::optional<int64_t> end, int64_t step) const {
    Layout l = d_.layout;
    if (l.shape.empty()) throw Error("slice() cannot be applied to a 0-dim tensor.");
    if (step <= 0) throw Error("slice step must be positive");
    const size_t d = normalize_dim(dim, l.shape.size());
    const int64_t size = l.shape[d];
    auto clamp = [&](int64_t v) {
        if (v < 0) v += size;
        return v < 0 ? int64_t{0} : (v > size ? size : v);
    };
    const int64_t from = clamp(start.value_or(0)), to = clamp(end.value_or(size));
    const int64_t len = to > from ? (to - from - 1) / step + 1 : 0;
    l.offset += from * l.strides[d];
    l.shape[d] = len;
    l.strides[d] *= step;
    return Tensor(TensorData{d_.storage, l, d_.dtype});
}

Tensor Tensor::select(int64_t dim, int64_t index) const {
    const Layout &l = d_.layout;
    if (l.shape.empty()) throw Error("select() cannot be applied to a 0-dim tensor.");
    size_t d = normalize_dim(dim, l.shape.size());
    int64_t size = l.shape[d];
    if (index < -size || index >= size) {
        throw Error("select(): index " + std::to_string(index) + " out of range for tensor of size " +
                    shape_str(l.shape) + " at dimension " + std::to_string(d));
    }
    if (index < 0) index += size;
    return Tensor(TensorData{d_.storage, l.select(d, index), d_.dtype});
}

Tensor Tensor::flatten(int64_t start_dim, int64_t end_dim) const {
    const Shape &s = d_.layout.shape;
    if (s.empty()) return reshape({1});
    size_t a = normalize_dim(start_dim, s.size()), b = normalize_dim(end_dim, s.size());
    if (a > b) throw Error("flatten() has invalid args: start_dim cannot come after end_dim");
    std::vector<int64_t> spec(s.begin(), s.begin() + static_cast<long>(a));
    int64_t merged = 1;
    for (size_t i = a; i <= b; ++i) merged *= s[i];
    spec.push_back(merged);
    spec.insert(spec.end(), s.begin() + static_cast<long>(b) + 1, s.end());
    return reshape(spec);
}

}  // namespace homura
