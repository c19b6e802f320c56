// Storage, the device dispatch of every kernel, and the ROCm host side that turns tensors into
// hmr_tensor_desc's and calls the C ABI. See homura.hpp for the map to the reference's files.
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <map>
#include <set>
#include <mutex>
#include <utility>
#include <vector>

#include "homura.hpp"
#include "homura_rocm.h"
#include "homura_rocm_ext.h"

namespace homura {

namespace {

// ---- the C ABI: status -> Error (ref: src/backend/rocm/mod.rs:55-75) ------------------------------

void expect(hmr_status s) {
    if (s == HMR_OK) return;
    std::string message = hmr_last_error();
    if (s == HMR_OUT_OF_MEMORY) throw Error("ROCm out of memory: " + message);
    throw Error(message);
}

// ---- contexts: one per device, created on first use (ref: src/backend/rocm/context.rs:137-210) ----

struct DeviceState {
    hmr_context_t ctx = nullptr;
    std::recursive_mutex exec;  // makes one op's kernel submissions atomic
    std::mutex alloc;
    std::set<std::pair<size_t, uintptr_t>> cache;  // freed blocks by size, then address; reused in stream order
};

std::mutex g_registry;
std::map<int, std::unique_ptr<DeviceState>> g_devices;

DeviceState &device_state(int index) {
    std::lock_guard<std::mutex> lock(g_registry);
    auto it = g_devices.find(index);
    if (it != g_devices.end()) return *it->second;
    auto st = std::make_unique<DeviceState>();
    expect(hmr_context_create(index, &st->ctx));
    return *(g_devices[index] = std::move(st));
}

// Runs `f(ctx)` inside the device's execution lock.
template <class F>
void exec(const TensorData &on, F f) {
    DeviceState &st = device_state(on.device().index);
    std::lock_guard<std::recursive_mutex> lock(st.exec);
    f(st.ctx);
}

// ---- a minimal caching allocator over hmr_malloc (ref: src/backend/caching.rs:1-13) ---------------
// Every kernel of a device runs on its one stream, so a freed block may be handed out again at once:
// work already queued on it finishes before anything queued later touches it.

size_t round_block(size_t nbytes) {
    const size_t q = nbytes < (1u << 20) ? 512 : (2u << 20);
    return (nbytes + q - 1) / q * q;
}

void *device_alloc(int index, size_t block) {
    DeviceState &st = device_state(index);
    {
        std::lock_guard<std::mutex> lock(st.alloc);
        // Of the cached blocks of this size the one at the lowest address, as the reference's best fit picks
        // (ref: src/backend/caching.rs:5-6): a loop that frees its result and asks again gets the same block.
        auto it = st.cache.lower_bound({block, 0});
        if (it != st.cache.end() && it->first == block) {
            void *p = reinterpret_cast<void *>(it->second);
            st.cache.erase(it);
            return p;
        }
    }
    void *p = nullptr;
    hmr_status s = hmr_malloc(index, block, &p);
    if (s == HMR_OUT_OF_MEMORY) {
        // Release the cache and try once more, as the reference's allocator does.
        {
            std::lock_guard<std::recursive_mutex> run(st.exec);
            expect(hmr_context_synchronize(st.ctx));
            std::lock_guard<std::mutex> lock(st.alloc);
            for (auto &kv : st.cache) expect(hmr_free(index, reinterpret_cast<void *>(kv.second)));
            st.cache.clear();
        }
        s = hmr_malloc(index, block, &p);
    }
    expect(s);
    return p;
}

void device_release(int index, size_t block, void *p) {
    DeviceState &st = device_state(index);
    std::lock_guard<std::mutex> lock(st.alloc);
    st.cache.emplace(block, reinterpret_cast<uintptr_t>(p));
}

const hcb_backend *g_cpu = nullptr;

const hcb_backend &cpu_backend(const char *kernel) {
    if (!g_cpu) {
        throw Error(std::string(kernel) + ": no CPU backend is registered; this library only runs kernels on ROCm "
                                          "tensors");
    }
    return *g_cpu;
}

void cpu_check(int rc) {
    if (rc != 0) throw Error(g_cpu->last_error());
}

hcb_tensor cpu_desc(const TensorData &t) {
    return hcb_tensor{t.storage->ptr(),          t.layout.offset,       static_cast<int32_t>(t.dtype),
                      static_cast<int32_t>(t.layout.shape.size()), t.layout.shape.data(), t.layout.strides.data()};
}

hcb_scalar cpu_scalar(Scalar s) {
    hcb_scalar c{};
    c.kind = s.kind == Scalar::K::Bool ? HCB_SCALAR_BOOL : (s.kind == Scalar::K::Int ? HCB_SCALAR_INT : HCB_SCALAR_FLOAT);
    c.i = s.i;
    c.f = s.f;
    return c;
}

void check_shape(const TensorData &out, const TensorData &in) {
    if (out.layout.shape != in.layout.shape) throw Error("kernel operands must have the same shape");
}

// ---- descriptions (ref: src/backend/rocm/copy.rs:59-119) ----------------------------------------------

constexpr size_t kMaxDims = HMR_MAX_DIMS;

hmr_tensor_desc desc_with_dims(const char *kernel, const TensorData &t, int64_t offset,
                               const std::vector<MergedDim> &dims, size_t operand) {
    if (dims.size() > kMaxDims) {
        throw Error(std::string(kernel) + " on ROCm supports at most " + std::to_string(kMaxDims) +
                    " dimensions that can't be merged, got " + std::to_string(dims.size()));
    }
    hmr_tensor_desc d;
    std::memset(&d, 0, sizeof d);
    d.data = t.storage->ptr();
    d.offset = offset;
    d.dtype = static_cast<int32_t>(t.dtype);
    d.ndim = static_cast<int32_t>(dims.size());
    for (size_t j = 0; j < dims.size(); ++j) {
        d.sizes[j] = dims[j].size;
        d.strides[j] = dims[j].strides[operand];
    }
    return d;
}

// The descriptions of operands of one shape, merged together; false when they have no elements.
bool descs(const char *kernel, const std::vector<const TensorData *> &ops, std::vector<hmr_tensor_desc> &out) {
    std::vector<const Strides *> strides;
    for (const TensorData *t : ops) strides.push_back(&t->layout.strides);
    auto dims = merge_dims(ops[0]->layout.shape, strides);
    if (!dims) return false;
    out.clear();
    for (size_t k = 0; k < ops.size(); ++k) out.push_back(desc_with_dims(kernel, *ops[k], ops[k]->layout.offset, *dims, k));
    return true;
}

Strides walk_strides(const Layout &l) {
    return l.num_elements() == 0 ? Strides(l.strides.size(), 0) : l.strides;
}

// ref: src/backend/rocm/reduce.rs:32-103
struct Reduction {
    std::vector<MergedDim> dims;  // merged kept dims: strides[0] of the outputs, [1] of the source
    hmr_tensor_desc kept, red;
};

bool describe(const char *kernel, const TensorData &src, const std::vector<bool> &mask, Reduction &r) {
    const Layout &l = src.layout;
    Strides strides = walk_strides(l);
    Shape kept_shape, red_shape;
    Strides kept_strides, red_strides;
    for (size_t i = 0; i < l.shape.size(); ++i) {
        if (mask[i]) {
            red_shape.push_back(l.shape[i]);
            red_strides.push_back(strides[i]);
        } else {
            kept_shape.push_back(l.shape[i]);
            kept_strides.push_back(strides[i]);
        }
    }
    Strides out_strides = contiguous_strides(kept_shape);
    auto dims = merge_dims(kept_shape, {&out_strides, &kept_strides});
    if (!dims) return false;
    r.dims = *dims;
    std::vector<MergedDim> red_dims;
    if (auto rd = merge_dims(red_shape, {&red_strides})) red_dims = *rd;
    else red_dims = {MergedDim{0, {0}}};  // nothing to fold
    std::vector<MergedDim> src_dims;
    for (const MergedDim &d : r.dims) src_dims.push_back(MergedDim{d.size, {d.strides[1]}});
    r.kept = desc_with_dims(kernel, src, l.offset, src_dims, 0);
    r.red = desc_with_dims(kernel, src, 0, red_dims, 0);
    return true;
}

hmr_tensor_desc output_desc(const char *kernel, const Reduction &r, const TensorData &out) {
    if (!out.layout.is_contiguous()) throw Error(std::string("internal error: ") + kernel + " into a strided tensor");
    std::vector<MergedDim> dims;
    for (const MergedDim &d : r.dims) dims.push_back(MergedDim{d.size, {d.strides[0]}});
    return desc_with_dims(kernel, out, out.layout.offset, dims, 0);
}

// A workspace of `bytes` bytes on `device`, allocated before the execution lock is taken.
std::shared_ptr<Storage> workspace(int64_t bytes, Device device) {
    if (bytes <= 0) return nullptr;
    return std::make_shared<Storage>(device, static_cast<size_t>(bytes));
}

// ref: src/backend/rocm/reduce.rs:222-263
bool lines(const char *kernel, const TensorData &out, const TensorData &src, size_t dim, hmr_tensor_desc &o,
           hmr_tensor_desc &s, int64_t &n, int64_t &so, int64_t &si) {
    const Layout &ls = src.layout, &lo = out.layout;
    check_shape(out, src);
    if (ls.num_elements() == 0) return false;
    Shape other_shape;
    Strides other_out, other_src;
    for (size_t d = 0; d < ls.shape.size(); ++d) {
        if (d == dim) continue;
        other_shape.push_back(ls.shape[d]);
        other_out.push_back(lo.strides[d]);
        other_src.push_back(ls.strides[d]);
    }
    if (ls.shape.empty()) {
        n = 1;
        so = si = 0;
    } else {
        n = ls.shape[dim];
        so = lo.strides[dim];
        si = ls.strides[dim];
    }
    auto dims = merge_dims(other_shape, {&other_out, &other_src});
    if (!dims) return false;
    o = desc_with_dims(kernel, out, lo.offset, *dims, 0);
    s = desc_with_dims(kernel, src, ls.offset, *dims, 1);
    return true;
}

}  // namespace

// ---- Storage ---------------------------------------------------------------------------------------------

Storage::Storage(Device device, size_t nbytes) : device_(device), nbytes_(nbytes) {
    if (device.kind == Device::K::Cpu) {
        block_ = (nbytes + 63) / 64 * 64 + 64;
        ptr_ = std::aligned_alloc(64, block_);
        if (!ptr_) throw Error("host allocation failed");
    } else {
        block_ = round_block(nbytes == 0 ? 1 : nbytes);
        ptr_ = device_alloc(device.index, block_);
    }
}

Storage::~Storage() {
    if (!ptr_) return;
    if (device_.kind == Device::K::Cpu) std::free(ptr_);
    else device_release(device_.index, block_, ptr_);
}

void register_cpu_backend(const hcb_backend *table) { g_cpu = table; }

void empty_cache() {
    // Lock order everywhere is exec -> registry (an op allocates its outputs, and so looks its device up,
    // inside the execution lock), so the registry lock is dropped before any execution lock is taken.
    // Device states live until the process ends: the pointers stay valid.
    std::vector<std::pair<int, DeviceState *>> devices;
    {
        std::lock_guard<std::mutex> lock(g_registry);
        for (auto &kv : g_devices) devices.emplace_back(kv.first, kv.second.get());
    }
    for (auto &[index, st] : devices) {
        std::lock_guard<std::recursive_mutex> run(st->exec);
        expect(hmr_context_synchronize(st->ctx));
        std::lock_guard<std::mutex> a(st->alloc);
        for (auto &b : st->cache) expect(hmr_free(index, reinterpret_cast<void *>(b.second)));
        st->cache.clear();
    }
}

void synchronize(Device device) {
    if (device.kind != Device::K::Rocm) return;
    DeviceState &st = device_state(device.index);
    std::lock_guard<std::recursive_mutex> run(st.exec);
    expect(hmr_context_synchronize(st.ctx));
}

void *stream_handle(Device device) {
    if (device.kind != Device::K::Rocm) throw Error("stream_handle: not a ROCm device");
    void *s = nullptr;
    expect(hmr_ext_stream(device_state(device.index).ctx, &s));
    return s;
}

// ---- dispatch ------------------------------------------------------------------------------------------------

namespace backend {

namespace {
bool on_cpu(const TensorData &t) { return t.device().kind == Device::K::Cpu; }
}  // namespace

void copy(const TensorData &dst, const TensorData &src_in) {
    if (dst.device() != src_in.device()) throw Error("internal error: copy between devices");
    TensorData src = src_in.expand_to(dst.layout.shape);
    if (on_cpu(dst)) {
        hcb_tensor d = cpu_desc(dst), s = cpu_desc(src);
        cpu_check(cpu_backend("copy").copy(&d, &s));
        return;
    }
    std::vector<hmr_tensor_desc> ds;
    if (!descs("copy", {&dst, &src}, ds)) return;
    auto flat = [](const hmr_tensor_desc &x) { return x.ndim == 0 || (x.ndim == 1 && x.strides[0] == 1); };
    exec(dst, [&](hmr_context_t ctx) {
        if (dst.dtype == src.dtype && flat(ds[0]) && flat(ds[1])) {
            size_t size = size_in_bytes(dst.dtype);
            expect(hmr_copy_device(ctx, static_cast<char *>(ds[0].data) + ds[0].offset * size,
                                   static_cast<const char *>(ds[1].data) + ds[1].offset * size,
                                   static_cast<uint64_t>(dst.layout.num_elements()) * size));
        } else {
            expect(hmr_copy(ctx, &ds[0], &ds[1]));
        }
    });
}

void fill(const TensorData &dst, Scalar value) {
    if (on_cpu(dst)) {
        hcb_tensor d = cpu_desc(dst);
        cpu_check(cpu_backend("fill").fill(&d, cpu_scalar(value)));
        return;
    }
    std::vector<hmr_tensor_desc> ds;
    if (!descs("fill", {&dst}, ds)) return;
    uint64_t bits = scalar_bits(value, dst.dtype);
    exec(dst, [&](hmr_context_t ctx) { expect(hmr_fill(ctx, &ds[0], bits)); });
}

void unary(UnaryOp op, const TensorData &out, const TensorData &src) {
    check_shape(out, src);
    if (on_cpu(out)) {
        hcb_tensor o = cpu_desc(out), s = cpu_desc(src);
        cpu_check(cpu_backend("unary").unary(static_cast<int32_t>(op), &o, &s));
        return;
    }
    std::vector<hmr_tensor_desc> ds;
    if (!descs("unary", {&out, &src}, ds)) return;
    exec(out, [&](hmr_context_t ctx) { expect(hmr_unary(ctx, static_cast<int32_t>(op), &ds[0], &ds[1])); });
}

void binary(BinaryOp op, const TensorData &out, const TensorData &a, const TensorData &b) {
    check_shape(out, a);
    check_shape(out, b);
    if (on_cpu(out)) {
        hcb_tensor o = cpu_desc(out), x = cpu_desc(a), y = cpu_desc(b);
        cpu_check(cpu_backend("binary").binary(static_cast<int32_t>(op), &o, &x, &y));
        return;
    }
    std::vector<hmr_tensor_desc> ds;
    if (!descs("binary", {&out, &a, &b}, ds)) return;
    exec(out, [&](hmr_context_t ctx) { expect(hmr_binary(ctx, static_cast<int32_t>(op), &ds[0], &ds[1], &ds[2])); });
}

void binary_constant(BinaryOp op, const TensorData &out, const TensorData &a, Scalar value, bool constant_first) {
    check_shape(out, a);
    if (on_cpu(out)) {
        hcb_tensor o = cpu_desc(out), x = cpu_desc(a);
        cpu_check(cpu_backend("binary_constant")
                      .binary_constant(static_cast<int32_t>(op), &o, &x, cpu_scalar(value), constant_first));
        return;
    }
    uint64_t bits = scalar_bits(value, a.dtype);
    std::vector<hmr_tensor_desc> ds;
    if (!descs("binary_constant", {&out, &a}, ds)) return;
    exec(out, [&](hmr_context_t ctx) {
        expect(hmr_binary_constant(ctx, static_cast<int32_t>(op), &ds[0], &ds[1], bits, constant_first));
    });
}

void binary_scalar(BinaryOp op, const TensorData &out, const TensorData &a, double s, bool scalar_first) {
    check_shape(out, a);
    if (on_cpu(out)) {
        hcb_tensor o = cpu_desc(out), x = cpu_desc(a);
        cpu_check(cpu_backend("binary_scalar").binary_scalar(static_cast<int32_t>(op), &o, &x, s, scalar_first));
        return;
    }
    std::vector<hmr_tensor_desc> ds;
    if (!descs("binary_scalar", {&out, &a}, ds)) return;
    exec(out, [&](hmr_context_t ctx) {
        expect(hmr_binary_scalar(ctx, static_cast<int32_t>(op), &ds[0], &ds[1], s, scalar_first));
    });
}

void where_(const TensorData &out, const TensorData &cond, const TensorData &x, const TensorData &y) {
    check_shape(out, cond);
    check_shape(out, x);
    check_shape(out, y);
    if (on_cpu(out)) {
        hcb_tensor o = cpu_desc(out), c = cpu_desc(cond), a = cpu_desc(x), b = cpu_desc(y);
        cpu_check(cpu_backend("where_").where_(&o, &c, &a, &b));
        return;
    }
    std::vector<hmr_tensor_desc> ds;
    if (!descs("where_", {&out, &cond, &x, &y}, ds)) return;
    exec(out, [&](hmr_context_t ctx) { expect(hmr_where(ctx, &ds[0], &ds[1], &ds[2], &ds[3])); });
}

void where_constant(const TensorData &out, const TensorData &cond, Branch x, Branch y) {
    check_shape(out, cond);
    if (x.tensor && y.tensor) return where_(out, cond, *x.tensor, *y.tensor);
    if (on_cpu(out)) {
        hcb_tensor o = cpu_desc(out), c = cpu_desc(cond), a{}, b{};
        if (x.tensor) a = cpu_desc(*x.tensor);
        if (y.tensor) b = cpu_desc(*y.tensor);
        cpu_check(cpu_backend("where_constant")
                      .where_constant(&o, &c, x.tensor ? &a : nullptr, cpu_scalar(x.constant), y.tensor ? &b : nullptr,
                                      cpu_scalar(y.constant)));
        return;
    }
    uint64_t xb = x.tensor ? 0 : scalar_bits(x.constant, out.dtype);
    uint64_t yb = y.tensor ? 0 : scalar_bits(y.constant, out.dtype);
    std::vector<const TensorData *> ops = {&out, &cond};
    if (x.tensor) {
        check_shape(out, *x.tensor);
        ops.push_back(x.tensor);
    }
    if (y.tensor) {
        check_shape(out, *y.tensor);
        ops.push_back(y.tensor);
    }
    std::vector<hmr_tensor_desc> ds;
    if (!descs("where_constant", ops, ds)) return;
    const hmr_tensor_desc *xd = x.tensor ? &ds[2] : nullptr;
    const hmr_tensor_desc *yd = y.tensor ? &ds[2] : nullptr;
    exec(out, [&](hmr_context_t ctx) { expect(hmr_where_constant(ctx, &ds[0], &ds[1], xd, xb, yd, yb)); });
}

void reduce(ReduceOp op, const TensorData &out, const TensorData &src, const std::vector<bool> &mask) {
    if (on_cpu(out)) {
        hcb_tensor o = cpu_desc(out), s = cpu_desc(src);
        std::vector<uint8_t> m(mask.begin(), mask.end());
        cpu_check(cpu_backend("reduce").reduce(static_cast<int32_t>(op), &o, &s, m.data()));
        return;
    }
    Reduction r;
    if (!describe("reduce", src, mask, r)) return;
    hmr_tensor_desc o = output_desc("reduce", r, out);
    int64_t bytes = 0;
    expect(hmr_reduce_workspace(&r.kept, &r.red, 0, &bytes));
    auto ws = workspace(bytes, src.device());
    exec(out, [&](hmr_context_t ctx) {
        expect(hmr_reduce(ctx, static_cast<int32_t>(op), &o, &r.kept, &r.red, ws ? ws->ptr() : nullptr, bytes));
    });
}

void var(const TensorData &out, const TensorData &src, const std::vector<bool> &mask, double correction,
         bool take_sqrt) {
    if (on_cpu(out)) {
        hcb_tensor o = cpu_desc(out), s = cpu_desc(src);
        std::vector<uint8_t> m(mask.begin(), mask.end());
        cpu_check(cpu_backend("var").var(&o, &s, m.data(), correction, take_sqrt));
        return;
    }
    Reduction r;
    if (!describe("var", src, mask, r)) return;
    hmr_tensor_desc o = output_desc("var", r, out);
    int64_t bytes = 0;
    expect(hmr_reduce_workspace(&r.kept, &r.red, 1, &bytes));
    auto ws = workspace(bytes, src.device());
    exec(out, [&](hmr_context_t ctx) {
        expect(hmr_var(ctx, &o, &r.kept, &r.red, correction, take_sqrt, ws ? ws->ptr() : nullptr, bytes));
    });
}

void arg_reduce(const TensorData *values, const TensorData &indices, const TensorData &src, size_t dim,
                bool is_max) {
    if (on_cpu(indices)) {
        hcb_tensor v{}, i = cpu_desc(indices), s = cpu_desc(src);
        if (values) v = cpu_desc(*values);
        cpu_check(cpu_backend("arg_reduce").arg_reduce(values ? &v : nullptr, &i, &s, static_cast<int32_t>(dim), is_max));
        return;
    }
    size_t nd = src.layout.shape.size();
    std::vector<bool> mask(nd, false);
    if (nd > 0) {
        mask[dim] = true;
        if (src.layout.shape[dim] <= 0) throw Error("cannot compute the arg reduction of an empty dimension");
    }
    Reduction r;
    if (!describe("arg_reduce", src, mask, r)) return;
    hmr_tensor_desc i = output_desc("arg_reduce", r, indices);
    hmr_tensor_desc v{};
    if (values) v = output_desc("arg_reduce", r, *values);
    int64_t bytes = 0;
    expect(hmr_reduce_workspace(&r.kept, &r.red, 0, &bytes));
    auto ws = workspace(bytes, src.device());
    exec(indices, [&](hmr_context_t ctx) {
        expect(hmr_arg_reduce(ctx, values ? &v : nullptr, &i, &r.kept, &r.red, is_max, ws ? ws->ptr() : nullptr, bytes));
    });
}

void softmax(const TensorData &out, const TensorData &src, size_t dim, bool log) {
    if (on_cpu(out)) {
        hcb_tensor o = cpu_desc(out), s = cpu_desc(src);
        cpu_check(cpu_backend("softmax").softmax(&o, &s, static_cast<int32_t>(dim), log));
        return;
    }
    hmr_tensor_desc o, s;
    int64_t n = 0, so = 0, si = 0;
    if (!lines("softmax", out, src, dim, o, s, n, so, si)) return;
    int64_t bytes = 0;
    expect(hmr_softmax_workspace(&s, n, si, &bytes));
    auto ws = workspace(bytes, src.device());
    exec(out, [&](hmr_context_t ctx) {
        expect(hmr_softmax(ctx, &o, &s, n, so, si, log, ws ? ws->ptr() : nullptr, bytes));
    });
}

// ref: src/backend/rocm/reduce.rs:304-319
void exclusive_cumprod(const TensorData &out, const TensorData &src, size_t dim, bool reverse) {
    if (!out.layout.is_contiguous() || out.dtype != src.dtype) throw Error("exclusive_cumprod writes a contiguous tensor of the source's dtype");
    if (on_cpu(out)) {
        check_shape(out, src);
        hcb_tensor o = cpu_desc(out), s = cpu_desc(src);
        cpu_check(cpu_backend("exclusive_cumprod").exclusive_cumprod(&o, &s, static_cast<int32_t>(dim), reverse));
        return;
    }
    if (!is_floating_point(src.dtype)) throw Error(std::string("expected a floating point dtype, got ") + name_of(src.dtype));
    hmr_tensor_desc o, s;
    int64_t n, so, si;
    if (!lines("exclusive_cumprod", out, src, dim, o, s, n, so, si)) return;
    exec(out, [&](hmr_context_t ctx) { expect(hmr_exclusive_cumprod(ctx, &o, &s, n, so, si, reverse ? 1 : 0)); });
}

// ref: src/backend/rocm/elementwise.rs:155-215: the coefficient travels in the computation type.
void fused(const Fused &op, const TensorData &out, const TensorData &a, const TensorData &b, const TensorData *c) {
    check_shape(out, a);
    check_shape(out, b);
    if (c) check_shape(out, *c);
    if (on_cpu(out)) {
        hcb_tensor o = cpu_desc(out), x = cpu_desc(a), y = cpu_desc(b), z{};
        if (c) z = cpu_desc(*c);
        cpu_check(cpu_backend("fused").fused(static_cast<int32_t>(op.kind), op.scalar, &o, &x, &y, c ? &z : nullptr));
        return;
    }
    if (!is_floating_point(out.dtype)) throw Error(std::string("expected a floating point dtype, got ") + name_of(out.dtype));
    // As `C::of` and `T::down(..).up()` of the reference, for C = f32 (F16, BF16, F32) or f64.
    const bool wide = out.dtype == DType::F64;
    auto of = [&](double v) { return wide ? v : static_cast<double>(static_cast<float>(v)); };
    double coefficient = 0.0;
    bool small = false;
    switch (op.kind) {
        case Fused::ScaledAdd:
            coefficient = round_through(op.scalar, out.dtype);  // alpha rounded to the dtype first
            break;
        case Fused::Lerp: {
            double w = of(op.scalar);
            small = std::fabs(w) < 0.5;
            coefficient = small ? w : of(w - 1.0);
            break;
        }
        default: coefficient = of(op.scalar); break;
    }
    std::vector<hmr_tensor_desc> ds;
    std::vector<const TensorData *> ops = {&out, &a, &b};
    if (c) ops.push_back(c);
    if (!descs("fused", ops, ds)) return;
    exec(out, [&](hmr_context_t ctx) {
        expect(hmr_fused(ctx, static_cast<int32_t>(op.kind), &ds[0], &ds[1], &ds[2], c ? &ds[3] : nullptr, coefficient,
                         small ? 1 : 0));
    });
}

// ref: src/backend/rocm/elementwise.rs:323-346: batch dimensions merged, the two matrix dimensions kept.
void triangle(const TensorData &out, const TensorData &src, int64_t diagonal, bool upper) {
    const Layout &ls = src.layout, &lo = out.layout;
    const size_t nd = ls.shape.size();
    if (nd < 2 || ls.shape != lo.shape) throw Error("triangle: operands must have the same shape of two or more dimensions");
    if (on_cpu(out)) {
        hcb_tensor o = cpu_desc(out), s = cpu_desc(src);
        cpu_check(cpu_backend("triangle").triangle(&o, &s, diagonal, upper));
        return;
    }
    if (ls.num_elements() == 0) return;
    Shape batch(ls.shape.begin(), ls.shape.end() - 2);
    Strides bo(lo.strides.begin(), lo.strides.end() - 2), bs(ls.strides.begin(), ls.strides.end() - 2);
    auto merged = merge_dims(batch, {&bo, &bs});
    std::vector<MergedDim> dims = merged ? *merged : std::vector<MergedDim>{};
    for (size_t d = nd - 2; d < nd; ++d) dims.push_back(MergedDim{ls.shape[d], {lo.strides[d], ls.strides[d]}});
    hmr_tensor_desc o = desc_with_dims("triangle", out, lo.offset, dims, 0);
    hmr_tensor_desc s = desc_with_dims("triangle", src, ls.offset, dims, 1);
    exec(out, [&](hmr_context_t ctx) { expect(hmr_triangle(ctx, &o, &s, diagonal, upper ? 1 : 0)); });
}

// ref: src/backend/rocm/elementwise.rs:348-386: the source is read through negative strides from the
// last element of each reversed dimension.
void flip(const TensorData &out, const TensorData &src, const std::vector<bool> &mask) {
    const Layout &l = src.layout;
    if (!out.layout.is_contiguous() || out.layout.shape != l.shape) throw Error("flip writes a contiguous tensor of the source's shape");
    if (on_cpu(out)) {
        hcb_tensor o = cpu_desc(out), s = cpu_desc(src);
        std::vector<uint8_t> m(mask.begin(), mask.end());
        cpu_check(cpu_backend("flip").flip(&o, &s, m.data()));
        return;
    }
    if (l.num_elements() == 0) return;
    int64_t src_offset = l.offset;
    std::vector<MergedDim> dims;
    Strides out_strides = contiguous_strides(l.shape);
    for (size_t d = 0; d < l.shape.size(); ++d) {
        const int64_t size = l.shape[d];
        if (size == 1) continue;
        int64_t st = l.strides[d];
        if (mask[d]) {
            src_offset += (size - 1) * st;
            st = -st;
        }
        const int64_t pair[2] = {out_strides[d], st};
        // Neighbours merge when they are contiguous with each other in both operands, which with signed
        // strides also requires both to be reversed or neither.
        if (!dims.empty()) {
            MergedDim &outer = dims.back();
            bool joins = true;
            for (int k = 0; k < 2; ++k) {
                int64_t prod = 0;
                joins = joins && !__builtin_mul_overflow(pair[k], size, &prod) && prod == outer.strides[k];
            }
            if (joins) {
                outer.size *= size;
                outer.strides = {pair[0], pair[1]};
                continue;
            }
        }
        dims.push_back(MergedDim{size, {pair[0], pair[1]}});
    }
    hmr_tensor_desc o = desc_with_dims("flip", out, out.layout.offset, dims, 0);
    hmr_tensor_desc s = desc_with_dims("flip", src, src_offset, dims, 1);
    exec(out, [&](hmr_context_t ctx) { expect(hmr_flip(ctx, &o, &s)); });
}

// ref: src/backend/rocm/elementwise.rs:218-264: all four operands described with the output's two
// dimensions, v1 broadcast along the columns and v2 along the rows.
void addr(const TensorData &out, const TensorData &v1, const TensorData &v2, const TensorData &input, Scalar alpha,
          Scalar beta) {
    const Layout &lo = out.layout, &l1 = v1.layout, &l2 = v2.layout, &lc = input.layout;
    if (l1.shape.size() != 1 || l2.shape.size() != 1 || lo.shape != Shape{l1.shape[0], l2.shape[0]} || lc.shape != lo.shape) {
        throw Error("addr: the operands must be [n, m], [n], [m] and a view of [n, m]");
    }
    if (on_cpu(out)) {
        hcb_tensor o = cpu_desc(out), a = cpu_desc(v1), b = cpu_desc(v2), c = cpu_desc(input);
        cpu_check(cpu_backend("addr").addr(&o, &a, &b, &c, cpu_scalar(alpha), cpu_scalar(beta)));
        return;
    }
    if (lo.num_elements() == 0) return;
    const bool reads = beta.to_f64() != 0.0;
    std::vector<MergedDim> dims = {MergedDim{lo.shape[0], {lo.strides[0], l1.strides[0], 0, lc.strides[0]}},
                                   MergedDim{lo.shape[1], {lo.strides[1], 0, l2.strides[0], lc.strides[1]}}};
    hmr_tensor_desc d_out = desc_with_dims("addr", out, lo.offset, dims, 0), d1 = desc_with_dims("addr", v1, l1.offset, dims, 1),
                    d2 = desc_with_dims("addr", v2, l2.offset, dims, 2), d_in = desc_with_dims("addr", input, lc.offset, dims, 3);
    const bool floating = is_floating_point(out.dtype);
    exec(out, [&](hmr_context_t ctx) {
        expect(hmr_addr(ctx, &d_out, &d1, &d2, reads ? &d_in : nullptr, floating ? alpha.to_f64() : 0.0,
                        floating ? beta.to_f64() : 0.0, floating ? 0 : alpha.to_i64(), floating ? 0 : beta.to_i64()));
    });
}

// ---- indexing (ref: src/backend/rocm/index.rs) -----------------------------------------------------------------

namespace {

// The strides of an operand walked over a shape it shares with the others of a call (but along `dim`).
struct Walked {
    const TensorData *data;
    Strides strides;
    int64_t offset;
};

// The descriptions of `operands` over `shape`, with the dimensions before `dim` and those after it merged as
// the CPU merges them and `dim` kept in between; `at` is its position among them
// (ref: src/backend/rocm/index.rs:62-88). `shape` has elements.
std::vector<hmr_tensor_desc> around(const char *kernel, const std::vector<Walked> &operands, const Shape &shape, size_t dim,
                                    int &at) {
    auto part = [&](size_t from, size_t to) {
        Shape sub(shape.begin() + from, shape.begin() + to);
        std::vector<Strides> cut;
        for (const Walked &w : operands) cut.emplace_back(w.strides.begin() + from, w.strides.begin() + to);
        std::vector<const Strides *> ptrs;
        for (const Strides &c : cut) ptrs.push_back(&c);
        auto merged = merge_dims(sub, ptrs);
        return merged ? *merged : std::vector<MergedDim>{};
    };
    std::vector<MergedDim> dims = part(0, dim);
    at = static_cast<int>(dims.size());
    MergedDim middle{shape[dim], {}};
    for (const Walked &w : operands) middle.strides.push_back(w.strides[dim]);
    dims.push_back(middle);
    for (const MergedDim &d : part(dim + 1, shape.size())) dims.push_back(d);
    std::vector<hmr_tensor_desc> out;
    for (size_t k = 0; k < operands.size(); ++k) out.push_back(desc_with_dims(kernel, *operands[k].data, operands[k].offset, dims, k));
    return out;
}

Walked walked(const TensorData &t) { return Walked{&t, walk_strides(t.layout), t.layout.offset}; }

// The description of `data` with its own dimensions merged (ref: index.rs:36-45); false without elements.
bool own_desc(const char *kernel, const TensorData &data, hmr_tensor_desc &d) {
    std::vector<hmr_tensor_desc> ds;
    if (!descs(kernel, {&data}, ds)) return false;
    d = ds[0];
    return true;
}

}  // namespace

// ref: src/backend/mod.rs:375-378
std::string out_of_bounds(int64_t value, size_t dim, int64_t size) {
    return "index " + std::to_string(value) + " is out of bounds for dimension " + std::to_string(dim) + " with size " +
           std::to_string(size);
}

namespace {

// Inside the execution lock of `on`'s device: checks the positions of `index` against a dimension `dim` of
// `size` on the device, reads the verdict back (a synchronization) and, if every position is in range, queues
// `then`: the check and the kernel see the same index data (ref: index.rs:118-215).
template <class F>
void run_checked(const char *kernel, const TensorData &on, const TensorData &index, size_t dim, int64_t size, Bounds bounds,
                 F then) {
    hmr_tensor_desc check{};
    const bool checks = bounds != Bounds::Valid && bounds != Bounds::ValidWrap && own_desc(kernel, index, check);
    std::shared_ptr<Storage> slots = checks ? workspace(16, on.device()) : nullptr;
    exec(on, [&](hmr_context_t ctx) {
        if (checks) {
            const int64_t low = bounds == Bounds::AllowNegative ? -size : 0;
            uint64_t words[2] = {0, 0};
            expect(hmr_index_check(ctx, &check, low, size, 0, 0, static_cast<uint64_t *>(slots->ptr())));
            expect(hmr_copy_to_host(ctx, words, slots->ptr(), sizeof words));
            if (words[0] != ~uint64_t{0}) throw Error(out_of_bounds(static_cast<int64_t>(words[1]), dim, size));
        }
        then(ctx);
    });
}

}  // namespace

void index_select(const TensorData &out, const TensorData &src, size_t dim, const TensorData &index, Bounds bounds) {
    if (on_cpu(out)) {
        hcb_tensor o = cpu_desc(out), s = cpu_desc(src), i = cpu_desc(index);
        const Bounds known = bounds == Bounds::ValidWrap ? Bounds::AllowNegative : bounds;  // the CPU kernel checks again
        cpu_check(cpu_backend("index_select").index_select(&o, &s, static_cast<int32_t>(dim), &i, static_cast<int32_t>(known)));
        return;
    }
    const int64_t size = src.layout.shape[dim];
    const Shape &shape = out.layout.shape;
    std::vector<hmr_tensor_desc> d;
    int at = 0;
    const bool work = out.layout.num_elements() > 0;
    if (work) {
        // The index walked along `dim` of out, its other strides 0.
        Strides along(shape.size(), 0);
        const Strides own = walk_strides(index.layout);
        along[dim] = own.empty() ? 0 : own[0];
        d = around("index_select", {walked(out), walked(src), Walked{&index, along, index.layout.offset}}, shape, dim, at);
        d[1].sizes[at] = size;
    }
    run_checked("index_select", out, index, dim, size, bounds, [&](hmr_context_t ctx) {
        if (!work) return;
        hmr_tensor_desc i = d[2];  // the 1-D index: its walk along `dim`
        i.ndim = 1;
        i.sizes[0] = d[2].sizes[at];
        i.strides[0] = d[2].strides[at];
        expect(hmr_index_select(ctx, &d[0], &d[1], &i, at, bounds == Bounds::AllowNegative || bounds == Bounds::ValidWrap ? 1 : 0));
    });
}

void gather(const TensorData &out, const TensorData &src, size_t dim, const TensorData &index) {
    if (on_cpu(out)) {
        hcb_tensor o = cpu_desc(out), s = cpu_desc(src), i = cpu_desc(index);
        cpu_check(cpu_backend("gather").gather(&o, &s, static_cast<int32_t>(dim), &i));
        return;
    }
    const int64_t size = src.layout.shape[dim];
    std::vector<hmr_tensor_desc> d;
    int at = 0;
    const bool work = out.layout.num_elements() > 0;
    if (work) {
        d = around("gather", {walked(out), walked(src), walked(index)}, out.layout.shape, dim, at);
        d[1].sizes[at] = size;  // the source's own length along `dim`, as for index_select
    }
    run_checked("gather", out, index, dim, size, Bounds::NonNegative, [&](hmr_context_t ctx) {
        if (work) expect(hmr_gather(ctx, &d[0], &d[1], &d[2], at));
    });
}

void index_add(const TensorData &out, size_t dim, const TensorData &index, const TensorData &src, Bounds bounds) {
    if (on_cpu(out)) {
        hcb_tensor o = cpu_desc(out), s = cpu_desc(src), i = cpu_desc(index);
        cpu_check(cpu_backend("index_add").index_add(&o, static_cast<int32_t>(dim), &i, &s, static_cast<int32_t>(bounds)));
        return;
    }
    if (bounds == Bounds::AllowNegative) throw Error("internal error: index_add on ROCm takes positions counted from the start");
    const int64_t size = out.layout.shape[dim], m = index.layout.num_elements();
    const bool work = src.layout.num_elements() > 0;
    std::vector<hmr_tensor_desc> d;
    hmr_tensor_desc idx{};
    int at = 0;
    int64_t bytes = 0;
    if (work) {
        d = around("index_add", {walked(out), walked(src)}, out.layout.shape, dim, at);
        d[1].sizes[at] = m;
        own_desc("index_add", index, idx);
        expect(hmr_index_add_workspace(m, size, &bytes));
    }
    std::shared_ptr<Storage> ws = workspace(bytes, out.device());
    run_checked("index_add", out, index, dim, size, bounds, [&](hmr_context_t ctx) {
        if (work) expect(hmr_index_add(ctx, &d[0], &d[1], &idx, at, ws ? ws->ptr() : nullptr, bytes));
    });
}

void scatter_add(const TensorData &out, size_t dim, const TensorData &index, const TensorData &src) {
    if (on_cpu(out)) {
        hcb_tensor o = cpu_desc(out), s = cpu_desc(src), i = cpu_desc(index);
        cpu_check(cpu_backend("scatter_add").scatter_add(&o, static_cast<int32_t>(dim), &i, &s));
        return;
    }
    const int64_t size = out.layout.shape[dim], n = index.layout.num_elements();
    std::vector<hmr_tensor_desc> d;
    int at = 0;
    int64_t bytes = 0;
    if (n > 0) {
        d = around("scatter_add", {walked(index), walked(out), walked(src)}, index.layout.shape, dim, at);
        d[1].sizes[at] = size;
        expect(hmr_scatter_add_workspace(n, &bytes));
    }
    std::shared_ptr<Storage> ws = workspace(bytes, out.device());
    run_checked("scatter_add", out, index, dim, size, Bounds::NonNegative, [&](hmr_context_t ctx) {
        if (n > 0) expect(hmr_scatter_add(ctx, &d[1], &d[2], &d[0], at, ws ? ws->ptr() : nullptr, bytes));
    });
}

// ref: src/backend/rocm/index.rs:299-336
void index_overwrite(const TensorData &out, size_t dim, const TensorData &index, const TensorData &src) {
    if (on_cpu(out)) {
        hcb_tensor o = cpu_desc(out), s = cpu_desc(src), i = cpu_desc(index);
        cpu_check(cpu_backend("index_overwrite").index_overwrite(&o, static_cast<int32_t>(dim), &i, &s));
        return;
    }
    if (src.layout.num_elements() == 0) return;
    if (!index.layout.is_contiguous() || index.dtype != DType::I64) {
        throw Error("internal error: index_overwrite with positions that aren't contiguous I64");
    }
    const int64_t size = out.layout.shape[dim], m = index.layout.num_elements();
    int at = 0;
    std::vector<hmr_tensor_desc> d = around("index_overwrite", {walked(src), walked(out)}, src.layout.shape, dim, at);
    d[1].sizes[at] = size;
    // One dimension even for a single position, as the kernel expects.
    const std::vector<MergedDim> flat{MergedDim{m, {1}}};
    const hmr_tensor_desc positions = desc_with_dims("index_overwrite", index, index.layout.offset, flat, 0);
    int64_t bytes = 0;
    expect(hmr_index_overwrite_workspace(size, &bytes));
    std::shared_ptr<Storage> ws = workspace(bytes, out.device());
    exec(out, [&](hmr_context_t ctx) {
        expect(hmr_index_overwrite(ctx, &d[1], &d[0], &positions, at, ws ? ws->ptr() : nullptr, bytes));
    });
}

// ref: src/backend/rocm/index.rs:560-612: the count, its read-back and the coordinates in one critical section,
// so that both passes see the same mask.
namespace {

// The mask as the device kernels take it: every dimension unmerged, the kernel reports coordinates along each.
hmr_tensor_desc mask_desc(const TensorData &mask) {
    std::vector<MergedDim> dims;
    const Strides strides = walk_strides(mask.layout);
    for (size_t d = 0; d < mask.layout.shape.size(); ++d) dims.push_back(MergedDim{mask.layout.shape[d], {strides[d]}});
    return desc_with_dims("mask_coordinates", mask, mask.layout.offset, dims, 0);
}

}  // namespace

MaskCount mask_count(const TensorData &mask) {
    MaskCount counted;
    counted.mask = mask;
    const int64_t n = mask.layout.num_elements();
    if (on_cpu(mask)) {
        hcb_tensor m = cpu_desc(mask);
        cpu_check(cpu_backend("mask_coordinates").mask_coordinates(&m, nullptr, &counted.count));
        return counted;
    }
    if (n == 0) return counted;
    const hmr_tensor_desc desc = mask_desc(mask);
    int64_t total_word = 0;
    expect(hmr_mask_workspace(n, &counted.workspace_bytes, &total_word));
    counted.workspace = workspace(counted.workspace_bytes, mask.device());
    exec(mask, [&](hmr_context_t ctx) {
        expect(hmr_mask_count(ctx, &desc, counted.workspace->ptr(), counted.workspace_bytes));
        uint64_t count = 0;
        expect(hmr_copy_to_host(ctx, &count, static_cast<const uint64_t *>(counted.workspace->ptr()) + total_word, sizeof count));
        counted.count = static_cast<int64_t>(count);
    });
    return counted;
}

std::vector<TensorData> mask_coordinates(const MaskCount &counted) {
    const TensorData &mask = counted.mask;
    const size_t nd = mask.layout.shape.size();
    const Device device = mask.device();
    Tensor coords = Tensor::uninit_on(Shape{static_cast<int64_t>(nd), counted.count}, DType::I64, device);
    if (on_cpu(mask)) {
        hcb_tensor m = cpu_desc(mask);
        hcb_tensor o = cpu_desc(coords.data());
        int64_t count = counted.count;
        cpu_check(cpu_backend("mask_coordinates").mask_coordinates(&m, &o, &count));
    } else if (counted.count > 0) {
        const hmr_tensor_desc desc = mask_desc(mask);
        const TensorData &out = coords.data();
        const std::vector<MergedDim> rows{MergedDim{static_cast<int64_t>(nd), {counted.count}}, MergedDim{counted.count, {1}}};
        const hmr_tensor_desc o = desc_with_dims("mask_coordinates", out, out.layout.offset, rows, 0);
        exec(mask, [&](hmr_context_t ctx) {
            expect(hmr_mask_coordinates(ctx, &desc, counted.workspace->ptr(), counted.workspace_bytes, &o));
        });
    }
    std::vector<TensorData> rows;
    for (size_t d = 0; d < nd; ++d) rows.push_back(coords.select(0, static_cast<int64_t>(d)).data());
    return rows;
}

std::vector<TensorData> mask_coordinates(const TensorData &mask) { return mask_coordinates(mask_count(mask)); }

// ref: src/backend/rocm/index.rs:614-668: the indices are checked and, without a position out of range, `out`
// written, in one critical section.
std::optional<std::pair<size_t, int64_t>> index_positions(const TensorData *out, const std::vector<TensorData> &coords,
                                                          const std::vector<int64_t> &sizes) {
    const TensorData *first = out ? out : (coords.empty() ? nullptr : &coords[0]);
    if (first == nullptr) return std::nullopt;
    if (on_cpu(*first)) {
        std::vector<hcb_tensor> descs_;
        for (const TensorData &c : coords) descs_.push_back(cpu_desc(c));
        std::vector<const hcb_tensor *> ptrs;
        for (const hcb_tensor &c : descs_) ptrs.push_back(&c);
        hcb_tensor o{};
        if (out) o = cpu_desc(*out);
        int32_t bad = -1;
        int64_t value = 0;
        cpu_check(cpu_backend("index_positions")
                      .index_positions(out ? &o : nullptr, static_cast<int32_t>(coords.size()), ptrs.data(), sizes.data(), &bad, &value));
        if (bad >= 0) return std::make_pair(static_cast<size_t>(bad), value);
        return std::nullopt;
    }
    // The checks: one per index with elements.
    std::vector<hmr_tensor_desc> checks(coords.size());
    std::vector<bool> has(coords.size(), false);
    for (size_t k = 0; k < coords.size(); ++k) has[k] = own_desc("index_positions", coords[k], checks[k]);
    // The positions: one pass per index over the broadcast shape.
    Strides strides(sizes.size(), 1);
    for (size_t k = sizes.size(); k-- > 1;) strides[k - 1] = strides[k] * sizes[k];
    struct Pass {
        hmr_tensor_desc out, coord;
    };
    std::vector<Pass> passes;
    std::vector<TensorData> expanded;
    if (out && out->layout.num_elements() > 0) {
        for (const TensorData &c : coords) expanded.push_back(c.expand_to(out->layout.shape));
        for (const TensorData &c : expanded) {
            std::vector<hmr_tensor_desc> d;
            if (!descs("index_positions", {out, &c}, d)) throw Error("internal error: index_positions over an empty shape");
            passes.push_back(Pass{d[0], d[1]});
        }
    }
    std::shared_ptr<Storage> slots = workspace(static_cast<int64_t>(16 * (coords.empty() ? 1 : coords.size())), first->device());
    std::optional<std::pair<size_t, int64_t>> bad;
    exec(*first, [&](hmr_context_t ctx) {
        std::vector<uint64_t> words(2 * coords.size(), 0);
        bool any = false;
        for (size_t k = 0; k < coords.size(); ++k) {
            if (!has[k]) continue;
            any = true;
            expect(hmr_index_check(ctx, &checks[k], -sizes[k], sizes[k], 0, 0, static_cast<uint64_t *>(slots->ptr()) + 2 * k));
        }
        if (any) expect(hmr_copy_to_host(ctx, words.data(), slots->ptr(), words.size() * sizeof(uint64_t)));
        for (size_t k = 0; k < coords.size(); ++k) {
            if (has[k] && words[2 * k] != ~uint64_t{0}) {
                bad = std::make_pair(k, static_cast<int64_t>(words[2 * k + 1]));
                return;
            }
        }
        for (size_t k = 0; k < passes.size(); ++k) {
            expect(hmr_index_positions(ctx, &passes[k].out, &passes[k].coord, sizes[k], strides[k], k == 0 ? 1 : 0));
        }
    });
    return bad;
}

namespace {
// ref: src/backend/rocm/random.rs:11-19
bool flat_desc(const char *kernel, const TensorData &out, hmr_tensor_desc &d) {
    if (!out.layout.is_contiguous()) throw Error(std::string("internal error: ") + kernel + " into a strided tensor");
    std::vector<hmr_tensor_desc> ds;
    if (!descs(kernel, {&out}, ds)) return false;
    d = ds[0];
    return true;
}
}  // namespace

void random_uniform(const TensorData &out, uint64_t seed, uint64_t offset, double from, double to) {
    if (on_cpu(out)) {
        hcb_tensor o = cpu_desc(out);
        cpu_check(cpu_backend("uniform").random_uniform(&o, seed, offset, from, to));
        return;
    }
    hmr_tensor_desc d;
    if (!flat_desc("uniform", out, d)) return;
    exec(out, [&](hmr_context_t ctx) { expect(hmr_random_uniform(ctx, &d, seed, offset, from, to)); });
}

void random_normal(const TensorData &out, uint64_t seed, uint64_t offset, double mean, double std) {
    if (on_cpu(out)) {
        hcb_tensor o = cpu_desc(out);
        cpu_check(cpu_backend("normal").random_normal(&o, seed, offset, mean, std));
        return;
    }
    hmr_tensor_desc d;
    if (!flat_desc("normal", out, d)) return;
    exec(out, [&](hmr_context_t ctx) { expect(hmr_random_normal(ctx, &d, seed, offset, mean, std)); });
}

std::optional<uint64_t> random_int_batch(const TensorData &out, uint64_t seed, uint64_t offset, uint64_t blocks, int64_t low,
                                         uint64_t range, uint64_t threshold, const TensorData *workspace) {
    if (on_cpu(out)) {
        hcb_tensor o = cpu_desc(out);
        uint64_t accepted = 0;
        cpu_check(cpu_backend("randint").random_int(&o, seed, offset, blocks, low, range, threshold, &accepted));
        return accepted;
    }
    hmr_tensor_desc d;
    if (!flat_desc("randint", out, d)) return std::nullopt;
    const uint64_t tiles = (blocks + HMR_RANDOM_INT_TILE - 1) / HMR_RANDOM_INT_TILE;
    void *ws = nullptr;
    if (threshold != 0) {
        if (!workspace || workspace->layout.offset != 0 || static_cast<uint64_t>(workspace->layout.num_elements()) <= 2 * tiles) {
            throw Error("internal error: the workspace of randint");
        }
        ws = workspace->storage->ptr();
    }
    exec(out, [&](hmr_context_t ctx) { expect(hmr_random_int(ctx, &d, seed, offset, blocks, low, range, threshold, ws)); });
    if (threshold == 0) return std::nullopt;
    // The batch's count is the workspace's last word: read it back (waits for the device).
    int64_t count = 0;
    DeviceState &st = device_state(out.device().index);
    std::lock_guard<std::recursive_mutex> lock(st.exec);
    expect(hmr_copy_to_host(st.ctx, &count, static_cast<const char *>(ws) + 2 * tiles * sizeof(int64_t), sizeof count));
    return static_cast<uint64_t>(count);
}

void upload(const TensorData &dst, const TensorData &src) {
    if (!src.layout.is_contiguous() || !dst.layout.is_contiguous() || !on_cpu(src) || on_cpu(dst)) {
        throw Error("internal error: upload needs a contiguous CPU source and a contiguous ROCm destination");
    }
    size_t size = size_in_bytes(dst.dtype);
    size_t nbytes = static_cast<size_t>(src.layout.num_elements()) * size;
    if (nbytes == 0) return;
    exec(dst, [&](hmr_context_t ctx) {
        expect(hmr_copy_from_host(ctx, static_cast<char *>(dst.storage->ptr()) + dst.layout.offset * size,
                                  static_cast<const char *>(src.storage->ptr()) + src.layout.offset * size, nbytes));
    });
}

void download(const TensorData &dst, const TensorData &src) {
    if (!src.layout.is_contiguous() || !dst.layout.is_contiguous() || on_cpu(src) || !on_cpu(dst)) {
        throw Error("internal error: download needs a contiguous ROCm source and a contiguous CPU destination");
    }
    size_t size = size_in_bytes(dst.dtype);
    size_t nbytes = static_cast<size_t>(src.layout.num_elements()) * size;
    if (nbytes == 0) return;
    exec(src, [&](hmr_context_t ctx) {
        expect(hmr_copy_to_host(ctx, static_cast<char *>(dst.storage->ptr()) + dst.layout.offset * size,
                                static_cast<const char *>(src.storage->ptr()) + src.layout.offset * size, nbytes));
    });
}

}  // namespace backend

// ---- plan hooks ------------------------------------------------------------------------------------------------

ReducePlanInfo rocm_reduce_plan(const Tensor &src, const std::vector<int64_t> &dims) {
    std::vector<bool> mask = dims_mask(dims, src.num_dims());
    Reduction r;
    if (!describe("test", src.data(), mask, r)) throw Error("reduction without outputs");
    ReducePlanInfo p{};
    expect(hmr_test_reduce_plan(&r.kept, &r.red, &p.group, &p.splits, &p.chunk));
    return p;
}

SoftmaxPlanInfo rocm_softmax_plan(const Tensor &src, int64_t dim) {
    size_t d = normalize_dim(dim, src.num_dims());
    hmr_tensor_desc o, s;
    int64_t n = 0, so = 0, si = 0;
    if (!lines("test", src.data(), src.data(), d, o, s, n, so, si)) throw Error("softmax without elements");
    int32_t split = 0, group = 0, cache = 0;
    expect(hmr_test_softmax_plan(&s, n, si, &split, &group, &cache));
    return SoftmaxPlanInfo{split != 0, group, cache};
}

}  // namespace homura
