// Python binding of the host layer (module homura_amd._host), used by the parity tests and by
// bench.py. It only forwards: every rule lives in the C++ host layer, every kernel behind the C ABI.
#include <pybind11/numpy.h>
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include "homura.hpp"

namespace py = pybind11;
using namespace homura;

namespace {

Operand to_operand(const py::handle &h) {
    if (py::isinstance<Tensor>(h)) return Operand(h.cast<Tensor>());
    if (py::isinstance<py::bool_>(h)) return Operand(Scalar::of_bool(h.cast<bool>()));
    if (py::isinstance<py::int_>(h)) return Operand(Scalar::of_int(h.cast<int64_t>()));
    if (py::isinstance<py::float_>(h)) return Operand(Scalar::of_float(h.cast<double>()));
    throw py::type_error("expected a Tensor, bool, int or float operand");
}

Device parse_device(const std::string &s) {
    if (s == "cpu") return Device::cpu();
    if (s.rfind("rocm:", 0) == 0) return Device::rocm(std::stoi(s.substr(5)));
    if (s == "rocm") return Device::rocm(0);
    throw Error("unknown device '" + s + "'");
}

std::vector<int64_t> to_dims(const py::handle &h) {
    if (py::isinstance<py::int_>(h)) return {h.cast<int64_t>()};
    return h.cast<std::vector<int64_t>>();
}

}  // namespace

PYBIND11_MODULE(_host, m) {
    m.doc() = "homura host layer (C++) over libhomura_rocm.so";
    py::register_exception<Error>(m, "HomuraError");

    py::enum_<DType>(m, "DType")
        .value("Bool", DType::Bool).value("U8", DType::U8).value("I8", DType::I8).value("I16", DType::I16)
        .value("I32", DType::I32).value("I64", DType::I64).value("F16", DType::F16).value("BF16", DType::BF16)
        .value("F32", DType::F32).value("F64", DType::F64);

    m.def("promote_types", &promote_types);
    m.def("can_cast", &can_cast);
    m.def("default_dtype", &default_dtype);
    m.def("set_default_dtype", &set_default_dtype);
    m.def("result_type", [](const std::vector<std::pair<DType, int>> &tensors, const py::list &scalars) {
        ResultType rt;
        for (auto &t : tensors) rt.tensor(t.first, static_cast<size_t>(t.second));
        for (auto s : scalars) rt.scalar(std::get<Scalar>(to_operand(s)));
        return rt.result();
    });
    m.def("scalar_bits", [](const py::handle &v, DType d) { return scalar_bits(std::get<Scalar>(to_operand(v)), d); });
    m.def("broadcast_shapes", &broadcast_shapes);
    m.def("contiguous_strides", &contiguous_strides);
    m.def("is_contiguous", [](const Shape &s, const Strides &st) { return is_contiguous(s, st); });
    m.def("dims_mask", &dims_mask);
    m.def("compute_view_strides", &compute_view_strides);
    m.def("merge_dims", [](const Shape &shape, const std::vector<Strides> &strides) -> py::object {
        std::vector<const Strides *> ps;
        for (auto &s : strides) ps.push_back(&s);
        auto r = merge_dims(shape, ps);
        if (!r) return py::none();
        py::list out;
        for (auto &d : *r) out.append(py::make_tuple(d.size, d.strides));
        return out;
    });
    m.def("register_cpu_backend", [](uintptr_t table) { register_cpu_backend(reinterpret_cast<const hcb_backend *>(table)); },
          "Registers the hcb_backend table at this address for kernels on CPU tensors (0 unregisters).");
    m.def("empty_cache", &empty_cache, py::call_guard<py::gil_scoped_release>());
    m.def("set_fused_promotion", &set_fused_promotion);
    m.def("synchronize", [](const std::string &d) {
        py::gil_scoped_release release;
        synchronize(parse_device(d));
    });
    m.def("stream_handle", [](const std::string &d) { return reinterpret_cast<uintptr_t>(stream_handle(parse_device(d))); });
    m.def("where_", [](const Tensor &c, const py::handle &x, const py::handle &y) {
        return where_(c, to_operand(x), to_operand(y));
    });
    m.def("full", [](const Shape &shape, const py::handle &v, DType d, const std::string &dev) {
        return Tensor::full(shape, std::get<Scalar>(to_operand(v)), d, parse_device(dev));
    });
    // The optimizers' single-rounding steps (ref: src/optim/mod.rs:569-592).
    m.def("scaled_add", &optim::scaled_add);
    m.def("lerp_step", &optim::lerp);
    m.def("addcmul_step", &optim::addcmul);
    m.def("addcdiv_step", &optim::addcdiv);
    // One parameter's optimizer update; the state goes in and comes out as tensors (None before the first step).
    m.def("sgd_step",
          [](const Tensor &p, const Tensor &grad, std::optional<Tensor> buffer, double lr, double momentum, double dampening,
             double weight_decay, bool nesterov, bool maximize) {
              optim::SgdOptions o{lr, momentum, dampening, weight_decay, nesterov, maximize};
              Tensor out = optim::sgd_step(p, grad, buffer, o);
              return py::make_tuple(out, buffer);
          },
          py::arg("p"), py::arg("grad"), py::arg("momentum_buffer"), py::arg("lr"), py::arg("momentum") = 0.0,
          py::arg("dampening") = 0.0, py::arg("weight_decay") = 0.0, py::arg("nesterov") = false,
          py::arg("maximize") = false);
    m.def("adam_step",
          [](const Tensor &p, const Tensor &grad, const py::object &state, double lr, double beta1, double beta2, double eps,
             double weight_decay, bool amsgrad, bool maximize, bool decoupled) {
              std::optional<optim::AdamState> st;
              if (!state.is_none()) {
                  py::tuple t = state.cast<py::tuple>();
                  st = optim::AdamState{t[0].cast<double>(), t[1].cast<Tensor>(), t[2].cast<Tensor>(),
                                        t[3].is_none() ? std::nullopt : std::optional<Tensor>(t[3].cast<Tensor>())};
              }
              optim::AdamOptions o{lr, beta1, beta2, eps, weight_decay, amsgrad, maximize};
              Tensor out = optim::adam_step(p, grad, st, o, decoupled);
              return py::make_tuple(out, py::make_tuple(st->step, st->exp_avg, st->exp_avg_sq, st->max_exp_avg_sq));
          },
          py::arg("p"), py::arg("grad"), py::arg("state"), py::arg("lr"), py::arg("beta1") = 0.9, py::arg("beta2") = 0.999,
          py::arg("eps") = 1e-8, py::arg("weight_decay") = 0.0, py::arg("amsgrad") = false, py::arg("maximize") = false,
          py::arg("decoupled_weight_decay") = false);
    m.def("grad_sum", &grad::sum);
    m.def("grad_mean", &grad::mean);
    m.def("grad_sum_to_size", &grad::sum_to_size);
    m.def("grad_prod", &grad::prod);
    m.def("grad_extremum", &grad::extremum);
    m.def("grad_extremum_dim", &grad::extremum_dim);
    m.def("grad_var_std", &grad::var_std);
    m.def("grad_softmax", &grad::softmax);
    m.def("manual_seed", &manual_seed);
    m.def("rand", [](const Shape &shape, DType d, const std::string &dev) { return rand(shape, d, parse_device(dev)); },
          py::arg("shape"), py::arg("dtype") = DType::F32, py::arg("device") = "cpu");
    m.def("randn", [](const Shape &shape, DType d, const std::string &dev) { return randn(shape, d, parse_device(dev)); },
          py::arg("shape"), py::arg("dtype") = DType::F32, py::arg("device") = "cpu");
    m.def("randint", [](int64_t low, int64_t high, const Shape &shape, DType d, const std::string &dev) {
        return randint(low, high, shape, d, parse_device(dev));
    }, py::arg("low"), py::arg("high"), py::arg("shape"), py::arg("dtype") = DType::I64, py::arg("device") = "cpu");
    m.def("uniform", [](const Shape &shape, double from, double to, DType d, const std::string &dev) {
        return uniform(shape, from, to, d, parse_device(dev));
    }, py::arg("shape"), py::arg("from_"), py::arg("to"), py::arg("dtype") = DType::F32, py::arg("device") = "cpu");
    m.def("normal", [](const Shape &shape, double mean, double std, DType d, const std::string &dev) {
        return normal(shape, mean, std, d, parse_device(dev));
    }, py::arg("shape"), py::arg("mean"), py::arg("std"), py::arg("dtype") = DType::F32, py::arg("device") = "cpu");
    m.def("exclusive_cumprod", &exclusive_cumprod, py::arg("x"), py::arg("dim"), py::arg("reverse") = false);
    m.def("reduce_plan", [](const Tensor &t, const std::vector<int64_t> &dims) {
        auto p = rocm_reduce_plan(t, dims);
        return py::make_tuple(p.group, p.splits, p.chunk);
    });
    m.def("softmax_plan", [](const Tensor &t, int64_t dim) {
        auto p = rocm_softmax_plan(t, dim);
        return py::make_tuple(p.split, p.group, p.cache);
    });

    py::class_<Tensor> T(m, "Tensor");
    T.def_static("from_bytes",
                 [](const py::buffer &b, DType dtype, const Shape &shape, const std::string &device) {
                     py::buffer_info info = b.request();
                     int64_t n = 1;
                     for (int64_t s : shape) n *= s;
                     size_t need = static_cast<size_t>(n) * size_in_bytes(dtype);
                     size_t have = static_cast<size_t>(info.size) * static_cast<size_t>(info.itemsize);
                     if (have != need) throw Error("from_bytes: buffer has " + std::to_string(have) + " bytes, shape needs " + std::to_string(need));
                     return Tensor::from_bytes(info.ptr, dtype, shape, parse_device(device));
                 },
                 py::arg("buffer"), py::arg("dtype"), py::arg("shape"), py::arg("device") = "cpu");
    T.def("to_bytes", [](const Tensor &t) {
        std::vector<uint8_t> v;
        {
            py::gil_scoped_release release;
            v = t.to_bytes();
        }
        return py::bytes(reinterpret_cast<const char *>(v.data()), v.size());
    });
    T.def_property_readonly("shape", [](const Tensor &t) { return t.shape(); });
    T.def_property_readonly("strides", [](const Tensor &t) { return t.stride(); });
    T.def_property_readonly("offset", [](const Tensor &t) { return t.storage_offset(); });
    T.def_property_readonly("dtype", [](const Tensor &t) { return t.dtype(); });
    T.def_property_readonly("device", [](const Tensor &t) { return t.device().str(); });
    T.def_property_readonly("data_ptr", [](const Tensor &t) {
        return reinterpret_cast<uintptr_t>(t.data().storage->ptr()) +
               static_cast<uintptr_t>(t.storage_offset()) * size_in_bytes(t.dtype());
    });
    T.def("is_contiguous", &Tensor::is_contiguous);
    T.def("num_elements", &Tensor::num_elements);
    T.def("to", [](const Tensor &t, const py::handle &target) {
        if (py::isinstance<DType>(target)) return t.to(target.cast<DType>());
        return t.to(parse_device(target.cast<std::string>()));
    });
    T.def("contiguous", &Tensor::contiguous);
    T.def("reshape", &Tensor::reshape);
    T.def("permute", &Tensor::permute);
    T.def("transpose", &Tensor::transpose);
    T.def("expand", &Tensor::expand);
    T.def("unsqueeze", &Tensor::unsqueeze);
    T.def("narrow", &Tensor::narrow);
    T.def("select", &Tensor::select);
    T.def("flatten", &Tensor::flatten);

    const std::pair<const char *, UnaryOp> unary_ops[] = {
        {"neg", UnaryOp::Neg}, {"abs", UnaryOp::Abs}, {"sign", UnaryOp::Sign}, {"relu", UnaryOp::Relu},
        {"exp", UnaryOp::Exp}, {"log", UnaryOp::Log}, {"sqrt", UnaryOp::Sqrt}, {"rsqrt", UnaryOp::Rsqrt},
        {"reciprocal", UnaryOp::Reciprocal}, {"sin", UnaryOp::Sin}, {"cos", UnaryOp::Cos}, {"erf", UnaryOp::Erf},
        {"tanh", UnaryOp::Tanh}, {"sigmoid", UnaryOp::Sigmoid}, {"log_sigmoid", UnaryOp::LogSigmoid},
        {"silu", UnaryOp::Silu}, {"gelu", UnaryOp::Gelu}, {"gelu_tanh", UnaryOp::GeluTanh},
        {"logical_not", UnaryOp::LogicalNot}};
    for (auto &u : unary_ops) {
        UnaryOp op = u.second;
        T.def(u.first, [op](const Tensor &t) { return t.unary(op); });
    }
    const std::pair<const char *, BinaryOp> binary_ops[] = {
        {"add", BinaryOp::Add}, {"sub", BinaryOp::Sub}, {"mul", BinaryOp::Mul}, {"div", BinaryOp::Div},
        {"pow", BinaryOp::Pow}, {"maximum", BinaryOp::Maximum}, {"minimum", BinaryOp::Minimum},
        {"greater", BinaryOp::Greater}, {"greater_equal", BinaryOp::GreaterEqual}, {"less", BinaryOp::Less},
        {"less_equal", BinaryOp::LessEqual}, {"equal", BinaryOp::Equal}, {"not_equal", BinaryOp::NotEqual},
        {"logical_and", BinaryOp::LogicalAnd}, {"logical_or", BinaryOp::LogicalOr},
        {"bitwise_and", BinaryOp::BitwiseAnd}};
    for (auto &b : binary_ops) {
        BinaryOp op = b.second;
        T.def(b.first, [op](const Tensor &t, const py::handle &o) { return t.binary(op, to_operand(o)); });
        // r<op>: the scalar (or tensor) on the left, `2.0 / x`.
        T.def((std::string("r") + b.first).c_str(),
              [op](const Tensor &t, const py::handle &o) { return binary_op(op, to_operand(o), Operand(t)); });
    }
    T.def("clamp", [](const Tensor &t, const py::handle &lo, const py::handle &hi) {
        return t.clamp(to_operand(lo), to_operand(hi));
    });
    T.def("clamp_min", [](const Tensor &t, const py::handle &lo) { return t.clamp_min(to_operand(lo)); });
    T.def("clamp_max", [](const Tensor &t, const py::handle &hi) { return t.clamp_max(to_operand(hi)); });
    T.def("masked_fill", [](const Tensor &t, const Tensor &mask, const py::handle &v) {
        return t.masked_fill(mask, to_operand(v));
    });
    // In-place operations return the tensor they wrote.
    const std::pair<const char *, BinaryOp> in_place_ops[] = {{"add_", BinaryOp::Add}, {"sub_", BinaryOp::Sub},
                                                              {"mul_", BinaryOp::Mul}, {"div_", BinaryOp::Div},
                                                              {"pow_", BinaryOp::Pow}};
    for (auto &b : in_place_ops) {
        BinaryOp op = b.second;
        T.def(b.first, [op](const Tensor &t, const py::handle &o) { return t.binary_(op, to_operand(o)); });
    }
    T.def("clamp_", [](const Tensor &t, const py::handle &lo, const py::handle &hi) {
        return t.clamp_(to_operand(lo), to_operand(hi));
    });
    T.def("masked_fill_", [](const Tensor &t, const Tensor &mask, const py::handle &v) {
        return t.masked_fill_(mask, to_operand(v));
    });
    T.def("copy_", [](const Tensor &t, const Tensor &src) { return t.copy_(src); });
    T.def("addcmul_", [](const Tensor &t, const Tensor &a, const Tensor &b, const py::handle &v) {
        return t.addcmul_(a, b, std::get<Scalar>(to_operand(v)));
    });
    T.def("addcdiv_", [](const Tensor &t, const Tensor &a, const Tensor &b, const py::handle &v) {
        return t.addcdiv_(a, b, std::get<Scalar>(to_operand(v)));
    });
    T.def("lerp_", [](const Tensor &t, const Tensor &end, const py::handle &w) { return t.lerp_(end, to_operand(w)); });
    T.def("fill_", [](const Tensor &t, const py::handle &v) { return t.fill_(std::get<Scalar>(to_operand(v))); });
    T.def("zero_", [](const Tensor &t) { return t.zero_(); });

    T.def("sum", &Tensor::sum);
    T.def("sum_dim", [](const Tensor &t, const py::handle &d, bool k) { return t.sum_dim(to_dims(d), k); });
    T.def("sum_to_size", &Tensor::sum_to_size);
    T.def("mean", &Tensor::mean);
    T.def("mean_dim", [](const Tensor &t, const py::handle &d, bool k) { return t.mean_dim(to_dims(d), k); });
    T.def("prod", &Tensor::prod);
    T.def("prod_dim", &Tensor::prod_dim);
    T.def("max", &Tensor::max);
    T.def("min", &Tensor::min);
    T.def("max_dim", [](const Tensor &t, int64_t d, bool k) {
        auto r = t.max_dim(d, k);
        return py::make_tuple(r.values, r.indices);
    });
    T.def("min_dim", [](const Tensor &t, int64_t d, bool k) {
        auto r = t.min_dim(d, k);
        return py::make_tuple(r.values, r.indices);
    });
    T.def("argmax", &Tensor::argmax);
    T.def("argmin", &Tensor::argmin);
    T.def("argmax_dim", &Tensor::argmax_dim);
    T.def("argmin_dim", &Tensor::argmin_dim);
    T.def("var", &Tensor::var);
    T.def("var_dim", [](const Tensor &t, const py::handle &d, int64_t c, bool k) { return t.var_dim(to_dims(d), c, k); });
    T.def("std", &Tensor::std);
    T.def("std_dim", [](const Tensor &t, const py::handle &d, int64_t c, bool k) { return t.std_dim(to_dims(d), c, k); });
    T.def("all", &Tensor::all);
    T.def("any", &Tensor::any);
    T.def("all_dim", [](const Tensor &t, const py::handle &d, bool k) { return t.all_dim(to_dims(d), k); });
    T.def("any_dim", [](const Tensor &t, const py::handle &d, bool k) { return t.any_dim(to_dims(d), k); });
    T.def("softmax", &Tensor::softmax);
    T.def("log_softmax", &Tensor::log_softmax);
    T.def("index_select", &Tensor::index_select);
    T.def("gather", &Tensor::gather);
    T.def("index_add", &Tensor::index_add);
    T.def("scatter_add", &Tensor::scatter_add);
    T.def("view", &Tensor::view);
    T.def("expand_as", &Tensor::expand_as);
    T.def("squeeze", &Tensor::squeeze);
    T.def("squeeze_dim", [](const Tensor &t, const py::handle &d) { return t.squeeze_dim(to_dims(d)); });
    T.def("unfold", &Tensor::unfold);
    T.def("as_strided", &Tensor::as_strided);
    T.def("slice", &Tensor::slice, py::arg("dim"), py::arg("start") = py::none(), py::arg("end") = py::none(), py::arg("step") = 1);
    T.def("index_tensors", &Tensor::index_tensors, py::call_guard<py::gil_scoped_release>());
    T.def("index_put_tensors", &Tensor::index_put_tensors);
    T.def("mask_coordinates", [](const Tensor &mask) {
        std::vector<Tensor> out;
        for (const homura::TensorData &d : homura::backend::mask_coordinates(mask.data())) out.emplace_back(d);
        return out;
    }, py::call_guard<py::gil_scoped_release>());
    T.def("triu", &Tensor::triu, py::arg("diagonal") = 0);
    T.def("tril", &Tensor::tril, py::arg("diagonal") = 0);
    T.def("flip", &Tensor::flip);
    T.def("addcmul", [](const Tensor &t, const Tensor &t1, const Tensor &t2, const py::handle &value) {
        return t.addcmul(t1, t2, std::get<Scalar>(to_operand(value)));
    });
    T.def("addcdiv", [](const Tensor &t, const Tensor &t1, const Tensor &t2, const py::handle &value) {
        return t.addcdiv(t1, t2, std::get<Scalar>(to_operand(value)));
    });
    T.def("addr", [](const Tensor &t, const Tensor &v1, const Tensor &v2, const py::handle &beta, const py::handle &alpha) {
        return t.addr(v1, v2, std::get<Scalar>(to_operand(beta)), std::get<Scalar>(to_operand(alpha)));
    }, py::arg("vec1"), py::arg("vec2"), py::arg("beta") = 1, py::arg("alpha") = 1);
    T.def("lerp", [](const Tensor &t, const Tensor &end, const py::handle &weight) { return t.lerp(end, to_operand(weight)); });
}
