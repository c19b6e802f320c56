// Input gradients of the reductions and of softmax, as compositions of the forward ops
// (ref: src/autograd/formulas/reduce.rs, softmax.rs). Nothing here touches a device directly: every step is
// an op of the path, so a gradient runs wherever its operands live.
#include <cmath>
#include <cstring>
#include <limits>

#include "homura.hpp"

namespace homura {
namespace grad {

namespace {

std::vector<int64_t> as_spec(const Shape &shape) { return std::vector<int64_t>(shape.begin(), shape.end()); }

// The shape the gradient of a reduction over `dims` is reshaped to before it is broadcast back: the reduced
// dimensions put back as 1s (ref: reduce.rs:12-27). Nothing to do when they were kept.
Tensor unreduce(const Tensor &g, const Shape &self_shape, const std::vector<int64_t> &dims, bool keepdim) {
    if (keepdim || dims.empty()) return g;
    std::vector<bool> mask = dims_mask(dims, self_shape.size());
    std::vector<int64_t> kept;
    for (size_t d = 0; d < self_shape.size(); ++d) kept.push_back(mask[d] ? 1 : self_shape[d]);
    return g.reshape(kept);
}

int64_t reduced_count(const Shape &shape, const std::vector<int64_t> &dims) {
    int64_t n = 1;
    if (dims.empty()) {
        for (int64_t s : shape) n *= s;
        return n;
    }
    std::vector<bool> mask = dims_mask(dims, shape.size());
    for (size_t d = 0; d < shape.size(); ++d) n *= mask[d] ? shape[d] : 1;
    return n;
}

int64_t count_of(const Tensor &flags) {
    std::vector<uint8_t> bytes = flags.sum().to_bytes();  // an I64 scalar; waits for the device
    int64_t n = 0;
    std::memcpy(&n, bytes.data(), sizeof n);
    return n;
}

}  // namespace

// ref: reduce.rs:160-207
Tensor sum(const Tensor &g, const Shape &self_shape, const std::vector<int64_t> &dims, bool keepdim) {
    return unreduce(g, self_shape, dims, keepdim).expand(as_spec(self_shape));
}

Tensor sum_to_size(const Tensor &g, const Shape &self_shape) { return g.expand(as_spec(self_shape)); }

// ref: reduce.rs:209-229
Tensor mean(const Tensor &g, const Shape &self_shape, const std::vector<int64_t> &dims, bool keepdim) {
    return sum(g, self_shape, dims, keepdim).div(Scalar::of_int(reduced_count(self_shape, dims)));
}

// ref: reduce.rs:258-329: without zeros g * (result / x); with zeros g times the product of the other elements
// of the slice, which is exclusive_cumprod forwards times backwards; a whole product with several zeros is zero.
Tensor prod(const Tensor &g_in, const Tensor &x, const Tensor &result_in, std::optional<int64_t> dim, bool keepdim) {
    if (x.num_dims() == 0) return g_in;
    Tensor g = g_in, result = result_in;
    size_t d = 0;
    if (dim) {
        d = normalize_dim(*dim, x.num_dims());
        g = unreduce(g, x.shape(), {static_cast<int64_t>(d)}, keepdim);
        result = unreduce(result, x.shape(), {static_cast<int64_t>(d)}, keepdim);
    }
    const int64_t zeros = count_of(x.equal(Scalar::of_float(0.0)));
    if (zeros == 0) return g.mul(result.div(x));
    if (!dim && zeros > 1) return Tensor::full(x.shape(), Scalar::of_int(0), x.dtype(), x.device());
    Tensor flat = dim ? x : x.reshape({-1});
    if (flat.shape()[d] == 1) return g.reshape(as_spec(x.shape()));
    Tensor others = exclusive_cumprod(flat, d, false).mul(exclusive_cumprod(flat, d, true));
    return g.mul(others).reshape(as_spec(x.shape()));
}

// ref: reduce.rs:331-351: g divided evenly among the positions that hold the result, selected rather than
// multiplied, so that the others get zeros also for an infinite or NaN g; a NaN result is shared by every NaN.
Tensor extremum(const Tensor &g, const Tensor &x, const Tensor &result) {
    Tensor both_nan = x.not_equal(x).logical_and(result.not_equal(result));
    Tensor mask = x.equal(result).logical_or(both_nan);
    Tensor share = g.div(mask.sum());
    return Tensor::full(x.shape(), Scalar::of_int(0), g.dtype(), g.device()).masked_fill(mask, share);
}

// ref: reduce.rs:353-380
Tensor extremum_dim(const Tensor &g_in, const Tensor &indices_in, const Shape &self_shape, int64_t dim, bool keepdim) {
    const size_t d = normalize_dim(dim, self_shape.size());
    Tensor g = unreduce(g_in, self_shape, {static_cast<int64_t>(d)}, keepdim);
    Tensor indices = unreduce(indices_in, self_shape, {static_cast<int64_t>(d)}, keepdim);
    Tensor zeros = Tensor::full(self_shape, Scalar::of_int(0), g.dtype(), g.device());
    return zeros.scatter_add(static_cast<int64_t>(d), indices, g);
}

// ref: reduce.rs:382-424
Tensor var_std(const Tensor &g_in, const Tensor &x, const std::optional<Tensor> &std_result, const std::vector<int64_t> &dims_in,
               int64_t correction_in, bool keepdim) {
    Tensor g = g_in;
    if (std_result) {
        g = g.div(std_result->mul(Scalar::of_float(2.0))).masked_fill(std_result->equal(Scalar::of_float(0.0)), Scalar::of_float(0.0));
    }
    const double correction = static_cast<double>(correction_in);
    const bool all = dims_in.empty() || x.num_dims() == 0;
    if (all) {
        Tensor mean = x.mean();
        const double dof = static_cast<double>(x.num_elements()) - correction;
        if (dof <= 0.0) {
            Tensor infinite = Tensor::full(x.shape(), Scalar::of_float(std::numeric_limits<double>::infinity()), x.dtype(), x.device())
                                  .masked_fill(x.equal(mean), Scalar::of_float(std::numeric_limits<double>::quiet_NaN()));
            return g.mul(infinite);
        }
        return g.mul(Scalar::of_float(2.0 / dof)).mul(x.sub(mean));
    }
    g = unreduce(g, x.shape(), dims_in, keepdim);
    Tensor mean = x.mean_dim(dims_in, true);
    const double scale = 2.0 / (static_cast<double>(reduced_count(x.shape(), dims_in)) - correction);
    return g.mul(Scalar::of_float(scale)).mul(x.sub(mean));
}

// ref: softmax.rs:43-84: softmax y * (g - sum(g * y)), log-softmax g - exp(y) * sum(g), the sums along `dim`;
// half precision goes through f32 and is rounded once.
Tensor softmax(const Tensor &g_in, const Tensor &y_in, int64_t dim, bool log) {
    const DType dtype = y_in.dtype();
    const bool half = dtype == DType::F16 || dtype == DType::BF16;
    Tensor g = half ? g_in.to(DType::F32) : g_in, y = half ? y_in.to(DType::F32) : y_in;
    Tensor grad = log ? g.sub(y.exp().mul(g.sum_dim({dim}, true))) : y.mul(g.sub(g.mul(y).sum_dim({dim}, true)));
    return grad.to(dtype);
}

}  // namespace grad
}  // namespace homura
