// homura.hpp -- the host side of homura's tensor elementwise / broadcast / reduction path, in
// C++ (the reference's host side is Rust; no Rust toolchain exists where this is built).
//
// It mirrors, name for name, the part of the reference that sits between user code and the C ABI:
//   dtype rules      promote_types, ResultType, can_cast, Scalar      ref: src/dtype.rs:279-535
//   shape algebra    broadcast_shapes, contiguous_strides, dims_mask,
//                    compute_view_strides, infer_size                 ref: src/shape.rs:520-742
//   Layout / views   expand_to, permute, transpose, narrow, select... ref: src/tensor/mod.rs:83-170,
//                                                                          src/tensor/view.rs
//   ops front end    binary_op, where_/select, unary_op, reduce_op,
//                    arg_op, var_op, softmax_op, cast_data            ref: src/ops/{binary,unary,reduce,composite,mod}.rs
//   dispatch         backend::<kernel> by device                      ref: src/backend/mod.rs:298-534
//   ROCm host        merge_dims, descs, workspaces, exec lock, status
//                    -> error                                         ref: src/backend/rocm/{copy,elementwise,reduce,context,mod}.rs
// Where the reference panics, this code throws homura::Error with the reference's message.
// Autograd, in-place ops and the Meta device are outside this path and absent.
#pragma once

#include <cstdint>
#include <memory>
#include <optional>
#include <stdexcept>
#include <string>
#include <variant>
#include <vector>

#include "cpu_backend.h"

namespace homura {

struct Error : std::runtime_error {
    using std::runtime_error::runtime_error;
};

// ---- dtype ------------------------------------------------------------------------------------------

enum class DType : int32_t { Bool = 0, U8, I8, I16, I32, I64, F16, BF16, F32, F64 };
enum class Kind { Bool, Int, Float };

Kind kind_of(DType d);
inline bool is_floating_point(DType d) { return kind_of(d) == Kind::Float; }
inline bool is_integral(DType d) { return kind_of(d) == Kind::Int; }
size_t size_in_bytes(DType d);
const char *name_of(DType d);

DType default_dtype();
void set_default_dtype(DType d);  // floating point dtypes only

struct Scalar {
    enum class K { Bool, Int, Float } kind;
    int64_t i = 0;
    double f = 0.0;
    static Scalar of_bool(bool v) { return Scalar{K::Bool, v ? 1 : 0, 0.0}; }
    static Scalar of_int(int64_t v) { return Scalar{K::Int, v, 0.0}; }
    static Scalar of_float(double v) { return Scalar{K::Float, 0, v}; }
    double to_f64() const;
    int64_t to_i64() const;
    bool to_bool() const;
    DType dtype() const;  // default float dtype / I64 / Bool
    // The value as a scalar of `dtype` if it fits (fill_, masked_fill): ref src/dtype.rs:334-374.
    std::optional<Scalar> checked_to(DType dtype) const;
    std::string str() const;
};

DType promote_types(DType a, DType b);
bool can_cast(DType from, DType to);

class ResultType {
  public:
    ResultType &tensor(DType dtype, size_t num_dims);
    ResultType &scalar(Scalar s);
    DType result() const;

  private:
    std::optional<DType> dim_, zero_dim_, scalar_;
};

// `value` converted to `dtype` as the CPU's fill converts it, little-endian in the low bytes
// (ref: src/backend/rocm/copy.rs:253-270).
double float_max(DType d);                              // the largest finite value of a float dtype
void int_range(DType d, int64_t &lo, int64_t &hi);      // of an integer or bool dtype
uint64_t scalar_bits(Scalar value, DType dtype);
// `value` taken to a floating point dtype's computation type (f32, or f64 for F64), rounded to the dtype,
// and read back.
double round_through(double value, DType dtype);

// ---- shapes -------------------------------------------------------------------------------------------

using Shape = std::vector<int64_t>;
using Strides = std::vector<int64_t>;

std::string shape_str(const Shape &s);
size_t normalize_dim(int64_t dim, size_t num_dims);
std::vector<bool> dims_mask(const std::vector<int64_t> &dims, size_t num_dims);
Strides contiguous_strides(const Shape &shape);
bool is_contiguous(const Shape &shape, const Strides &strides);
bool is_expandable_to(const Shape &shape, const Shape &desired);
Shape broadcast_shapes(const Shape &a, const Shape &b);
Shape infer_size(const std::vector<int64_t> &spec, int64_t num_elements);
std::optional<Strides> compute_view_strides(const Shape &old_shape, const Strides &old_strides, const Shape &new_shape);

// One merged dimension: its size and its stride in each operand (ref: src/backend/rocm/copy.rs:28-57).
struct MergedDim {
    int64_t size;
    std::vector<int64_t> strides;
};
// nullopt for an empty shape.
std::optional<std::vector<MergedDim>> merge_dims(const Shape &shape, const std::vector<const Strides *> &strides);

// ---- devices, storage, layout -----------------------------------------------------------------------

struct Device {
    enum class K { Cpu, Rocm } kind = K::Cpu;
    int index = 0;
    static Device cpu() { return Device{K::Cpu, 0}; }
    static Device rocm(int i) { return Device{K::Rocm, i}; }
    bool operator==(const Device &o) const { return kind == o.kind && index == o.index; }
    bool operator!=(const Device &o) const { return !(*this == o); }
    std::string str() const;
};

class Storage {
  public:
    Storage(Device device, size_t nbytes);  // uninitialised; throws Error / OutOfMemory
    ~Storage();
    Storage(const Storage &) = delete;
    Storage &operator=(const Storage &) = delete;
    Device device() const { return device_; }
    void *ptr() const { return ptr_; }
    size_t nbytes() const { return nbytes_; }

  private:
    Device device_;
    void *ptr_ = nullptr;
    size_t nbytes_ = 0;
    size_t block_ = 0;
};

struct Layout {
    Shape shape;
    Strides strides;
    int64_t offset = 0;
    static Layout contiguous(Shape shape);
    int64_t num_elements() const;
    bool is_contiguous() const { return homura::is_contiguous(shape, strides); }
    Layout expand_to(const Shape &target) const;  // ref: src/tensor/mod.rs:139-170
    Layout select(size_t dim, int64_t index) const;
};

struct TensorData {
    std::shared_ptr<Storage> storage;
    Layout layout;
    DType dtype = DType::F32;
    Device device() const { return storage->device(); }
    TensorData expand_to(const Shape &shape) const;
};

// Registers the kernels that run on Device::Cpu tensors (see cpu_backend.h). nullptr unregisters.
void register_cpu_backend(const hcb_backend *table);
// Returns device memory cached by the allocator to the driver.
void empty_cache();
// Waits for everything queued on the device's stream.
void synchronize(Device device);
// Whether a half tensor combined with an F32 tensor is widened inside the binary kernel (default)
// or, as the reference does, by a separate cast kernel first. Both give the same bits.
void set_fused_promotion(bool on);
// The hipStream_t of the device's context (for harnesses that record their own events).
void *stream_handle(Device device);

// ---- Tensor ---------------------------------------------------------------------------------------------

class Tensor;
using Operand = std::variant<Tensor, Scalar>;

enum class UnaryOp : int32_t {
    Neg = 0, Abs, Sign, Relu, Exp, Log, Sqrt, Rsqrt, Reciprocal, Sin, Cos, Erf, Tanh, Sigmoid, LogSigmoid,
    Silu, Gelu, GeluTanh, LogicalNot
};
enum class BinaryOp : int32_t {
    Add = 0, Sub, Mul, Div, Pow, Maximum, Minimum, Greater, GreaterEqual, Less, LessEqual, Equal, NotEqual,
    LogicalAnd, LogicalOr, BitwiseAnd
};
enum class ReduceOp : int32_t { Sum = 0, Prod, Mean, Max, Min, All, Any };
enum class GeluApproximate { None, Tanh };

struct ValuesAndIndices;

class Tensor {
  public:
    Tensor() = default;
    explicit Tensor(TensorData d) : d_(std::move(d)) {}

    // Creation. `bytes` holds num_elements * size_in_bytes(dtype) bytes in row-major order.
    static Tensor from_bytes(const void *bytes, DType dtype, const Shape &shape, Device device = Device::cpu());
    static Tensor uninit_on(const Shape &shape, DType dtype, Device device);
    static Tensor full(const Shape &shape, Scalar value, DType dtype, Device device);

    const TensorData &data() const { return d_; }
    const Shape &shape() const { return d_.layout.shape; }
    const Strides &stride() const { return d_.layout.strides; }
    int64_t storage_offset() const { return d_.layout.offset; }
    DType dtype() const { return d_.dtype; }
    Device device() const { return d_.device(); }
    size_t num_dims() const { return d_.layout.shape.size(); }
    int64_t num_elements() const { return d_.layout.num_elements(); }
    bool is_contiguous() const { return d_.layout.is_contiguous(); }

    // The elements in row-major order (moves to the host; waits for the device).
    std::vector<uint8_t> to_bytes() const;

    Tensor to(DType dtype) const;
    Tensor to(Device device) const;
    Tensor contiguous() const;

    // Views (ref: src/tensor/view.rs).
    Tensor reshape(const std::vector<int64_t> &spec) const;
    Tensor permute(const std::vector<int64_t> &dims) const;
    Tensor transpose(int64_t dim0, int64_t dim1) const;
    Tensor expand(const std::vector<int64_t> &spec) const;
    Tensor unsqueeze(int64_t dim) const;
    Tensor narrow(int64_t dim, int64_t start, int64_t length) const;
    Tensor select(int64_t dim, int64_t index) const;
    Tensor slice(int64_t dim, std::optional<int64_t> start, std::optional<int64_t> end, int64_t step) const;
    Tensor flatten(int64_t start_dim, int64_t end_dim) const;
    // ref: src/tensor/view.rs (view, expand_as, squeeze, squeeze_dim, unfold, as_strided)
    Tensor view(const std::vector<int64_t> &spec) const;
    Tensor expand_as(const Tensor &other) const;
    Tensor squeeze() const;
    Tensor squeeze_dim(const std::vector<int64_t> &dims) const;
    Tensor unfold(int64_t dim, int64_t size, int64_t step) const;
    Tensor as_strided(const Shape &size, const Strides &stride, int64_t storage_offset) const;

    // Unary (ref: src/ops/unary.rs).
    Tensor unary(UnaryOp op) const;
    Tensor neg() const { return unary(UnaryOp::Neg); }
    Tensor abs() const { return unary(UnaryOp::Abs); }
    Tensor sign() const { return unary(UnaryOp::Sign); }
    Tensor relu() const { return unary(UnaryOp::Relu); }
    Tensor exp() const { return unary(UnaryOp::Exp); }
    Tensor log() const { return unary(UnaryOp::Log); }
    Tensor sqrt() const { return unary(UnaryOp::Sqrt); }
    Tensor rsqrt() const { return unary(UnaryOp::Rsqrt); }
    Tensor reciprocal() const { return unary(UnaryOp::Reciprocal); }
    Tensor sin() const { return unary(UnaryOp::Sin); }
    Tensor cos() const { return unary(UnaryOp::Cos); }
    Tensor erf() const { return unary(UnaryOp::Erf); }
    Tensor tanh() const { return unary(UnaryOp::Tanh); }
    Tensor sigmoid() const { return unary(UnaryOp::Sigmoid); }
    Tensor log_sigmoid() const { return unary(UnaryOp::LogSigmoid); }
    Tensor silu() const { return unary(UnaryOp::Silu); }
    Tensor gelu(GeluApproximate a = GeluApproximate::None) const {
        return unary(a == GeluApproximate::None ? UnaryOp::Gelu : UnaryOp::GeluTanh);
    }
    Tensor logical_not() const { return unary(UnaryOp::LogicalNot); }

    // Binary with broadcasting and type promotion (ref: src/ops/binary.rs).
    Tensor binary(BinaryOp op, const Operand &other) const;
    Tensor add(const Operand &o) const { return binary(BinaryOp::Add, o); }
    Tensor sub(const Operand &o) const { return binary(BinaryOp::Sub, o); }
    Tensor mul(const Operand &o) const { return binary(BinaryOp::Mul, o); }
    Tensor div(const Operand &o) const { return binary(BinaryOp::Div, o); }
    Tensor pow(const Operand &o) const { return binary(BinaryOp::Pow, o); }
    Tensor maximum(const Operand &o) const { return binary(BinaryOp::Maximum, o); }
    Tensor minimum(const Operand &o) const { return binary(BinaryOp::Minimum, o); }
    Tensor greater(const Operand &o) const { return binary(BinaryOp::Greater, o); }
    Tensor greater_equal(const Operand &o) const { return binary(BinaryOp::GreaterEqual, o); }
    Tensor less(const Operand &o) const { return binary(BinaryOp::Less, o); }
    Tensor less_equal(const Operand &o) const { return binary(BinaryOp::LessEqual, o); }
    Tensor equal(const Operand &o) const { return binary(BinaryOp::Equal, o); }
    Tensor not_equal(const Operand &o) const { return binary(BinaryOp::NotEqual, o); }
    Tensor logical_and(const Operand &o) const { return binary(BinaryOp::LogicalAnd, o); }
    Tensor logical_or(const Operand &o) const { return binary(BinaryOp::LogicalOr, o); }
    Tensor bitwise_and(const Operand &o) const { return binary(BinaryOp::BitwiseAnd, o); }  // extension
    Tensor clamp(const Operand &min, const Operand &max) const { return maximum(min).minimum(max); }
    Tensor clamp_min(const Operand &min) const { return maximum(min); }
    Tensor clamp_max(const Operand &max) const { return minimum(max); }
    Tensor masked_fill(const Tensor &mask, const Operand &value) const;

    // In-place operations: the result of the out-of-place operation is checked against `self` (same shape, a
    // dtype that can be cast to its own, elements that are distinct memory locations) and copied into it
    // (ref: src/ops/binary.rs:225-242, 340-366, 419-429, 479-515, src/ops/mod.rs:308-392).
    const Tensor &binary_(BinaryOp op, const Operand &other) const;
    const Tensor &add_(const Operand &o) const { return binary_(BinaryOp::Add, o); }
    const Tensor &sub_(const Operand &o) const { return binary_(BinaryOp::Sub, o); }
    const Tensor &mul_(const Operand &o) const { return binary_(BinaryOp::Mul, o); }
    const Tensor &div_(const Operand &o) const { return binary_(BinaryOp::Div, o); }
    const Tensor &pow_(const Operand &o) const { return binary_(BinaryOp::Pow, o); }
    const Tensor &clamp_(const Operand &min, const Operand &max) const;
    const Tensor &masked_fill_(const Tensor &mask, const Operand &value) const;
    // Copies `src` into self, broadcasting it and converting its dtype; `src` may be on another device and may
    // overlap self (ref: src/ops/binary.rs:504-515, 594-641).
    const Tensor &copy_(const Tensor &src) const;
    const Tensor &fill_(Scalar value) const;  // ref: src/ops/binary.rs:532-560, 606-622
    const Tensor &zero_() const { return fill_(Scalar::of_int(0)); }

    // Reductions (ref: src/ops/reduce.rs).
    Tensor sum() const;
    Tensor sum_dim(const std::vector<int64_t> &dims, bool keepdim) const;
    Tensor sum_to_size(const Shape &size) const;
    Tensor mean() const;
    Tensor mean_dim(const std::vector<int64_t> &dims, bool keepdim) const;
    Tensor prod() const;
    Tensor prod_dim(int64_t dim, bool keepdim) const;
    Tensor max() const;
    Tensor min() const;
    ValuesAndIndices max_dim(int64_t dim, bool keepdim) const;
    ValuesAndIndices min_dim(int64_t dim, bool keepdim) const;
    Tensor argmax() const;
    Tensor argmin() const;
    Tensor argmax_dim(int64_t dim, bool keepdim) const;
    Tensor argmin_dim(int64_t dim, bool keepdim) const;
    Tensor var(int64_t correction) const;
    Tensor var_dim(const std::vector<int64_t> &dims, int64_t correction, bool keepdim) const;
    Tensor std(int64_t correction) const;
    Tensor std_dim(const std::vector<int64_t> &dims, int64_t correction, bool keepdim) const;
    Tensor all() const;
    Tensor any() const;
    Tensor all_dim(const std::vector<int64_t> &dims, bool keepdim) const;
    Tensor any_dim(const std::vector<int64_t> &dims, bool keepdim) const;

    // ref: src/ops/composite.rs:10-27
    Tensor softmax(int64_t dim) const;
    Tensor log_softmax(int64_t dim) const;
    // Gathering and scattering (ref: src/tensor/index.rs:712-755, src/ops/scatter.rs:42-234).
    Tensor index_select(int64_t dim, const Tensor &index) const;
    Tensor gather(int64_t dim, const Tensor &index) const;
    Tensor index_add(int64_t dim, const Tensor &index, const Tensor &source) const;
    Tensor scatter_add(int64_t dim, const Tensor &index, const Tensor &src) const;
    // Advanced indexing with one optional index tensor (I32 / I64 positions or a bool mask) per leading
    // dimension; nullopt keeps the dimension (ref: src/ops/advanced_index.rs:403-440).
    Tensor index_tensors(const std::vector<std::optional<Tensor>> &indices) const;
    Tensor index_put_tensors(const std::vector<std::optional<Tensor>> &indices, const Tensor &values, bool accumulate) const;
    // ref: src/ops/shape_ops.rs:182-263
    Tensor triu(int64_t diagonal) const;
    Tensor tril(int64_t diagonal) const;
    Tensor flip(const std::vector<int64_t> &dims) const;
    // ref: src/ops/composite.rs:450-508 (compositions of the ops above, as the reference's are)
    Tensor addcmul(const Tensor &tensor1, const Tensor &tensor2, Scalar value) const;
    Tensor addcdiv(const Tensor &tensor1, const Tensor &tensor2, Scalar value) const;
    Tensor lerp(const Tensor &end, const Operand &weight) const;
    // ref: src/ops/composite.rs (addcmul_, addcdiv_, lerp_)
    const Tensor &addcmul_(const Tensor &tensor1, const Tensor &tensor2, Scalar value) const;
    const Tensor &addcdiv_(const Tensor &tensor1, const Tensor &tensor2, Scalar value) const;
    const Tensor &lerp_(const Tensor &end, const Operand &weight) const;
    // beta * self + alpha * outer(vec1, vec2), one kernel (ref: src/ops/composite.rs:346-384).
    Tensor addr(const Tensor &vec1, const Tensor &vec2, Scalar beta, Scalar alpha) const;

  private:
    TensorData d_;
};

struct ValuesAndIndices {
    Tensor values;
    Tensor indices;
};

// op(lhs, rhs); at least one operand is a tensor (ref: src/ops/binary.rs:68-143).
Tensor binary_op(BinaryOp op, const Operand &lhs, const Operand &rhs);
// torch.where (ref: src/ops/binary.rs:152-176).
Tensor where_(const Tensor &condition, const Operand &x, const Operand &y);
// For each element of the floating point `x`, the product of the elements before it along `dim` (after it
// when `reverse`), multiplied in order: what the gradient of `prod` uses for inputs with zeros
// (ref: src/ops/reduce.rs:158-170).
Tensor exclusive_cumprod(const Tensor &x, size_t dim, bool reverse);
// The input gradients of the reductions and of softmax for an output gradient `g`, composed from the ops above as
// the reference's backward nodes compose them outside grad mode (ref: src/autograd/formulas/reduce.rs:160-470,
// softmax.rs:43-84). `dims` empty = all elements (the full reductions); otherwise the reduced dimensions and
// whether they were kept.
namespace grad {
Tensor sum(const Tensor &g, const Shape &self_shape, const std::vector<int64_t> &dims, bool keepdim);
Tensor mean(const Tensor &g, const Shape &self_shape, const std::vector<int64_t> &dims, bool keepdim);
Tensor sum_to_size(const Tensor &g, const Shape &self_shape);
Tensor prod(const Tensor &g, const Tensor &x, const Tensor &result, std::optional<int64_t> dim, bool keepdim);
Tensor extremum(const Tensor &g, const Tensor &x, const Tensor &result);  // x.max() / x.min()
// x.max_dim / x.min_dim (values): g scattered to the positions the saved indices name.
Tensor extremum_dim(const Tensor &g, const Tensor &indices, const Shape &self_shape, int64_t dim, bool keepdim);
Tensor var_std(const Tensor &g, const Tensor &x, const std::optional<Tensor> &std_result, const std::vector<int64_t> &dims,
               int64_t correction, bool keepdim);
Tensor softmax(const Tensor &g, const Tensor &y, int64_t dim, bool log);
}  // namespace grad

// Random sampling from the process-wide Philox4x32-10 generator, shared by all devices: a GPU computes the
// CPU's uniform samples and integers bit for bit, also when calls on the two alternate
// (ref: src/ops/random.rs). `uniform` and `normal` are what `uniform_` / `normal_` fill a tensor with.
void manual_seed(uint64_t seed);
Tensor rand(const Shape &shape, DType dtype, Device device);
Tensor randn(const Shape &shape, DType dtype, Device device);
Tensor randint(int64_t low, int64_t high, const Shape &shape, DType dtype, Device device);
Tensor uniform(const Shape &shape, double from, double to, DType dtype, Device device);
Tensor normal(const Shape &shape, double mean, double std, DType dtype, Device device);

// The optimizers' single-rounding steps (ref: src/optim/mod.rs:569-616): new tensors from tensors of one
// shape, floating point dtype and device. A finite scalar beyond the range of the type it is converted
// to (the dtype for alpha, the computation type otherwise) is an error.
namespace optim {
Tensor scaled_add(const Tensor &a, const Tensor &b, double alpha);                // a + alpha * b
Tensor lerp(const Tensor &a, const Tensor &b, double weight);                     // lerp(a, b, weight)
Tensor addcmul(const Tensor &a, const Tensor &b, const Tensor &c, double value);  // a + value * b * c
Tensor addcdiv(const Tensor &a, const Tensor &b, const Tensor &c, double value);  // a + value * b / c

// One parameter's update, as the loop bodies of Sgd::step (ref: src/optim/sgd.rs:152-191) and of Adam's
// and AdamW's (ref: src/optim/adam.rs:123-171) compute it. Tensors here are values, so where the reference
// updates the parameter and its state in place these return the new parameter and replace the state's
// tensors; the bits are the same. Every coefficient is checked before anything is computed.
struct SgdOptions {
    double lr = 0.0, momentum = 0.0, dampening = 0.0, weight_decay = 0.0;
    bool nesterov = false, maximize = false;
};
struct AdamOptions {
    double lr = 1e-3, beta1 = 0.9, beta2 = 0.999, eps = 1e-8, weight_decay = 0.0;
    bool amsgrad = false, maximize = false;
};
struct AdamState {
    double step;  // counted in f32 like the reference's default-dtype step tensor
    Tensor exp_avg, exp_avg_sq;
    std::optional<Tensor> max_exp_avg_sq;
};
Tensor sgd_step(const Tensor &p, const Tensor &grad, std::optional<Tensor> &momentum_buffer, const SgdOptions &o);
Tensor adam_step(const Tensor &p, const Tensor &grad, std::optional<AdamState> &state, const AdamOptions &o,
                 bool decoupled_weight_decay);
}  // namespace optim

// ---- backend dispatch (ref: src/backend/mod.rs:298-534) ---------------------------------------------

// How the positions of an index tensor are checked (ref: src/backend/mod.rs:360-373).
// ValidWrap: checked already to lie in -size..size; negative positions count from the end.
enum class Bounds { Valid = 0, NonNegative = 1, AllowNegative = 2, ValidWrap = 3 };

// The optimizers' fused steps (ref: src/backend/cpu/mod.rs:509-530).
struct Fused {
    enum Kind { ScaledAdd = 0, Lerp = 1, Addcmul = 2, Addcdiv = 3 } kind;
    double scalar;  // alpha, weight or value
};

namespace backend {
struct Branch {
    const TensorData *tensor = nullptr;  // else the constant
    Scalar constant{};
};
void copy(const TensorData &dst, const TensorData &src);
void fill(const TensorData &dst, Scalar value);
void unary(UnaryOp op, const TensorData &out, const TensorData &src);
void binary(BinaryOp op, const TensorData &out, const TensorData &a, const TensorData &b);
void binary_constant(BinaryOp op, const TensorData &out, const TensorData &a, Scalar value, bool constant_first);
void binary_scalar(BinaryOp op, const TensorData &out, const TensorData &a, double s, bool scalar_first);
void where_(const TensorData &out, const TensorData &cond, const TensorData &x, const TensorData &y);
void where_constant(const TensorData &out, const TensorData &cond, Branch x, Branch y);
void reduce(ReduceOp op, const TensorData &out, const TensorData &src, const std::vector<bool> &mask);
void var(const TensorData &out, const TensorData &src, const std::vector<bool> &mask, double correction,
         bool take_sqrt);
void arg_reduce(const TensorData *values, const TensorData &indices, const TensorData &src, size_t dim,
                bool is_max);
void softmax(const TensorData &out, const TensorData &src, size_t dim, bool log);
void exclusive_cumprod(const TensorData &out, const TensorData &src, size_t dim, bool reverse);
// Indexing (ref: src/backend/mod.rs:375-430). `index` is I32 or I64; a position out of range is an Error with
// the CPU's message. index_add and scatter_add add into `out`, a new contiguous tensor.
std::string out_of_bounds(int64_t value, size_t dim, int64_t size);
void index_select(const TensorData &out, const TensorData &src, size_t dim, const TensorData &index, Bounds bounds);
void gather(const TensorData &out, const TensorData &src, size_t dim, const TensorData &index);
void index_add(const TensorData &out, size_t dim, const TensorData &index, const TensorData &src, Bounds bounds);
void scatter_add(const TensorData &out, size_t dim, const TensorData &index, const TensorData &src);
// Copies slice i of src along dim into slice index[i] of out, the last of repeated positions winning; `index`
// holds valid positions (contiguous I64) (ref: src/backend/mod.rs:391-396).
void index_overwrite(const TensorData &out, size_t dim, const TensorData &index, const TensorData &src);
// The coordinates of the true elements of a bool tensor in row-major order: one I64 vector per dimension, on
// the mask's device (ref: src/backend/mod.rs:398-403).
std::vector<TensorData> mask_coordinates(const TensorData &mask);
// The same in two steps, for a caller that needs the number of true elements first and the coordinates later or
// not at all: the count, with what the second step needs kept beside it.
struct MaskCount {
    TensorData mask;
    int64_t count = 0;
    std::shared_ptr<Storage> workspace;  // the device's per-tile offsets
    int64_t workspace_bytes = 0;
};
MaskCount mask_count(const TensorData &mask);
std::vector<TensorData> mask_coordinates(const MaskCount &counted);
// The positions of advanced indexing: checks each index, in order, to lie in -size..size for its size in `sizes`
// and returns the first value out of range as (k, value). Without one, and with `out` (I64, the shape the indices
// broadcast to), writes the row-major position in the subspace of `sizes` of every element, negative coordinates
// counting from the end (ref: src/backend/mod.rs:425-447).
std::optional<std::pair<size_t, int64_t>> index_positions(const TensorData *out, const std::vector<TensorData> &coords,
                                                          const std::vector<int64_t> &sizes);
void fused(const Fused &op, const TensorData &out, const TensorData &a, const TensorData &b, const TensorData *c);
void triangle(const TensorData &out, const TensorData &src, int64_t diagonal, bool upper);
void flip(const TensorData &out, const TensorData &src, const std::vector<bool> &mask);
// out [n, m] = beta * input + alpha * outer(v1 [n], v2 [m]); input is a view of [n, m], alpha and beta
// values of the dtype (ref: src/backend/mod.rs:562-587).
void addr(const TensorData &out, const TensorData &v1, const TensorData &v2, const TensorData &input, Scalar alpha,
          Scalar beta);
// Samples of the Philox blocks from `offset` on under `seed` into a contiguous tensor
// (ref: src/backend/rocm/random.rs:30-118). random_int_batch is one batch of the integer rejection sampling
// into the I64 `out`; it returns how many words it accepted (not read back, and `out` filled, when
// `threshold` is 0 on a ROCm device: then every word is accepted).
void random_uniform(const TensorData &out, uint64_t seed, uint64_t offset, double from, double to);
void random_normal(const TensorData &out, uint64_t seed, uint64_t offset, double mean, double std);
std::optional<uint64_t> random_int_batch(const TensorData &out, uint64_t seed, uint64_t offset, uint64_t blocks, int64_t low,
                                         uint64_t range, uint64_t threshold, const TensorData *workspace);
// Host <-> device and device <-> host transfers of contiguous data of one dtype.
void upload(const TensorData &dst, const TensorData &src);
void download(const TensorData &dst, const TensorData &src);
}  // namespace backend

// The plan the library reports for a reduction / softmax of `src` (test hook).
struct ReducePlanInfo {
    int64_t group, splits, chunk;
};
ReducePlanInfo rocm_reduce_plan(const Tensor &src, const std::vector<int64_t> &dims);
struct SoftmaxPlanInfo {
    bool split;
    int32_t group, cache;
};
SoftmaxPlanInfo rocm_softmax_plan(const Tensor &src, int64_t dim);

}  // namespace homura
