// Python module "tiramisu": the Tiramisu front-end from Python, bound to this build's library
// and its HIP back-end.  Class, function and overload names follow the reference's pybind11
// bindings (python_bindings/src/Py*.cpp, summarised in python_bindings/tiramisu.pyi), so programs
// written against them (python_bindings/tutorials/*.py) keep their text; on top of that the GPU
// memory tags of buffers are exposed, which GPU programs need and the reference leaves unbound
// (python_bindings/src/PyBuffer.cpp:8-24).  Objects that a function keeps pointers to
// (computations, buffers, functions) are never deleted from Python.
#include <pybind11/operators.h>
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include <tiramisu/tiramisu.h>

namespace py = pybind11;
using namespace tiramisu;

namespace {

template <typename T> using kept = std::unique_ptr<T, py::nodelete>;

void define_types(py::module &m) {
    py::enum_<primitive_t>(m, "primitive_t")
        .value("p_uint8", p_uint8).value("p_uint16", p_uint16).value("p_uint32", p_uint32).value("p_uint64", p_uint64)
        .value("p_int8", p_int8).value("p_int16", p_int16).value("p_int32", p_int32).value("p_int64", p_int64)
        .value("p_float32", p_float32).value("p_float64", p_float64).value("p_boolean", p_boolean)
        .value("p_bfloat16", p_bfloat16).value("p_none", p_none)
        .export_values();
    py::enum_<rank_t>(m, "rank_t").value("r_sender", rank_t::r_sender).value("r_receiver", rank_t::r_receiver).export_values();
    py::enum_<argument_t>(m, "argument_t")
        .value("a_input", a_input).value("a_output", a_output).value("a_temporary", a_temporary).export_values();
    py::enum_<expr_t>(m, "expr_t")
        .value("e_val", e_val).value("e_var", e_var).value("e_sync", e_sync).value("e_op", e_op).value("e_none", e_none).export_values();
    py::enum_<hardware_architecture_t>(m, "hardware_architecture_t")
        .value("arch_cpu", hardware_architecture_t::arch_cpu)
        .value("arch_nvidia_gpu", hardware_architecture_t::arch_nvidia_gpu)
        .value("arch_amd_gpu", hardware_architecture_t::arch_amd_gpu)
        .export_values();
    py::enum_<op_t>(m, "op_t")
        .value("o_minus", o_minus).value("o_floor", o_floor).value("o_sin", o_sin).value("o_cos", o_cos).value("o_tan", o_tan)
        .value("o_asin", o_asin).value("o_acos", o_acos).value("o_atan", o_atan).value("o_sinh", o_sinh).value("o_cosh", o_cosh)
        .value("o_tanh", o_tanh).value("o_abs", o_abs).value("o_sqrt", o_sqrt).value("o_expo", o_expo).value("o_log", o_log)
        .value("o_ceil", o_ceil).value("o_round", o_round).value("o_trunc", o_trunc).value("o_allocate", o_allocate).value("o_free", o_free)
        .value("o_cast", o_cast).value("o_add", o_add).value("o_sub", o_sub).value("o_mul", o_mul).value("o_div", o_div).value("o_mod", o_mod)
        .value("o_logical_and", o_logical_and).value("o_logical_or", o_logical_or).value("o_logical_not", o_logical_not)
        .value("o_eq", o_eq).value("o_ne", o_ne).value("o_le", o_le).value("o_lt", o_lt).value("o_ge", o_ge).value("o_gt", o_gt)
        .value("o_max", o_max).value("o_min", o_min).value("o_right_shift", o_right_shift).value("o_left_shift", o_left_shift)
        .value("o_memcpy", o_memcpy).value("o_select", o_select).value("o_cond", o_cond).value("o_lerp", o_lerp)
        .value("o_call", o_call).value("o_access", o_access).value("o_buffer", o_buffer).value("o_none", o_none)
        .export_values();
}

void define_expr(py::module &m) {
    auto e = py::class_<expr>(m, "expr")
        .def(py::init<>())
        .def(py::init<primitive_t>())
        .def(py::init([](int64_t v) { return (v >= INT32_MIN && v <= INT32_MAX) ? expr((int32_t)v) : expr(v); }))
        .def(py::init([](double v) { return expr((float)v); }))   // Python floats become fp32 values, as expr(1.5f) in C++ programs
        .def(py::init<const expr &>())
        .def(py::init<op_t, primitive_t, expr>())
        .def(py::init<op_t, expr>())
        .def(py::init<op_t, std::string>())
        .def(py::init<op_t, expr, expr>())
        .def(py::init<op_t, expr, expr, expr>())
        .def(py::init<op_t, std::string, std::vector<expr>, primitive_t>())
        .def("cast", [](const expr &x, primitive_t t) { return cast(t, x); })
        .def("is_equal", &expr::is_equal)
        .def("set_name", &expr::set_name)
        .def("get_name", [](const expr &x) { return x.get_name(); })
        .def("get_data_type", &expr::get_data_type)
        .def("get_int_val", &expr::get_int_val)
        .def("get_double_val", &expr::get_double_val)
        .def("logical_not", [](const expr &x) { return !x; })
        .def("dump", [](const expr &x) { py::print(x.to_str()); })
        .def("__repr__", [](const expr &x) { return x.to_str(); })
        .def("__neg__", [](const expr &x) { return -x; })
        .def("__truediv__", [](const expr &a, const expr &b) { return a / b; })
        .def("__rtruediv__", [](const expr &a, const expr &b) { return b / a; })
        .def("__floordiv__", [](const expr &a, const expr &b) { return a / b; })
        .def("__mod__", [](const expr &a, const expr &b) { return a % b; })
        .def("__rmod__", [](const expr &a, const expr &b) { return b % a; })
        .def("__rshift__", [](const expr &a, const expr &b) { return a >> b; })
        .def("__lshift__", [](const expr &a, const expr &b) { return a << b; })
        .def("__and__", [](const expr &a, const expr &b) { return a && b; })
        .def("__or__", [](const expr &a, const expr &b) { return a || b; })
        .def(py::self + py::self).def(py::self - py::self).def(py::self * py::self)
        .def("__radd__", [](const expr &a, const expr &b) { return b + a; })
        .def("__rsub__", [](const expr &a, const expr &b) { return b - a; })
        .def("__rmul__", [](const expr &a, const expr &b) { return b * a; })
        .def("__eq__", [](const expr &a, const expr &b) { return a == b; })
        .def("__ne__", [](const expr &a, const expr &b) { return a != b; })
        .def("__lt__", [](const expr &a, const expr &b) { return a < b; })
        .def("__le__", [](const expr &a, const expr &b) { return a <= b; })
        .def("__gt__", [](const expr &a, const expr &b) { return a > b; })
        .def("__ge__", [](const expr &a, const expr &b) { return a >= b; });
    e.attr("__hash__") = py::none();
    e.def("get_uint8_value", [](const expr &x) { return (uint8_t)x.get_int_val(); })
        .def("get_int8_value", [](const expr &x) { return (int8_t)x.get_int_val(); })
        .def("get_uint16_value", [](const expr &x) { return (uint16_t)x.get_int_val(); })
        .def("get_int16_value", [](const expr &x) { return (int16_t)x.get_int_val(); })
        .def("get_uint32_value", [](const expr &x) { return (uint32_t)x.get_int_val(); })
        .def("get_int32_value", [](const expr &x) { return (int32_t)x.get_int_val(); })
        .def("get_uint64_value", [](const expr &x) { return (uint64_t)x.get_int_val(); })
        .def("get_int64_value", [](const expr &x) { return (int64_t)x.get_int_val(); })
        .def("get_float32_value", [](const expr &x) { return (float)x.get_double_val(); })
        .def("get_float64_value", [](const expr &x) { return x.get_double_val(); });

    py::class_<var, expr>(m, "var")
        .def(py::init<primitive_t, std::string>())
        .def(py::init<std::string>())
        .def(py::init<std::string, expr, expr>())
        .def(py::init<>())
        .def("get_name", [](const var &v) { return v.get_name(); })
        .def("get_lower", &var::get_lower)
        .def("get_upper", &var::get_upper)
        .def("dump", [](const var &v) { py::print(v.to_str()); });
    py::class_<tiramisu::sync, expr>(m, "sync").def(py::init<>());

    py::implicitly_convertible<int64_t, expr>();
    py::implicitly_convertible<double, expr>();

    m.def("memcpy", [](const buffer &from, const buffer &to) { return tiramisu::memcpy(from, to); });
    m.def("allocate", [](const buffer &b) { return allocate(b); });
    m.def("cuda_stream_synchronize", [] { return cuda_stream_synchronize(); });
    m.def("hip_stream_synchronize", [] { return cuda_stream_synchronize(); });
    m.def("cast", [](primitive_t t, const expr &x) { return cast(t, x); });
}

void define_buffer(py::module &m) {
    py::class_<buffer, kept<buffer>>(m, "buffer")
        .def(py::init([](std::string name, std::vector<expr> sizes, primitive_t t, argument_t a) { return new buffer(name, sizes, t, a); }))
        .def("get_name", &buffer::get_name)
        .def("dump", &buffer::dump)
        .def("allocate_at", [](buffer &b, computation &c, var level) { return b.allocate_at(c, level); }, py::return_value_policy::reference)
        .def("tag_gpu_global", &buffer::tag_gpu_global)
        .def("tag_gpu_shared", &buffer::tag_gpu_shared)
        .def("tag_gpu_local", &buffer::tag_gpu_local)
        .def("tag_gpu_register", &buffer::tag_gpu_register)
        .def("tag_gpu_constant", &buffer::tag_gpu_constant);
}

expr access(computation &c, const std::vector<expr> &index) {
    return expr(o_access, c.get_name(), index, c.get_data_type());
}

void define_computation(py::module &m) {
    py::class_<computation, kept<computation>>(m, "computation")
        .def(py::init([](std::string name, std::vector<var> iters, expr e) { return new computation(name, iters, e); }))
        .def(py::init([](std::string name, std::vector<var> iters, primitive_t t) { return new computation(name, iters, t); }))
        .def(py::init([](std::vector<var> iters, primitive_t t) { return new computation(iters, t); }))
        .def("__getitem__", [](computation &c, std::vector<expr> index) { return access(c, index); })
        .def("__getitem__", [](computation &c, expr index) { return access(c, {index}); })
        .def("__call__", [](computation &c, py::args index) {
            std::vector<expr> idx;
            for (auto a : index) idx.push_back(a.cast<expr>());
            return access(c, idx);
        })
        .def("get_name", &computation::get_name)
        .def("parallelize", &computation::parallelize)
        .def("vectorize", py::overload_cast<var, int>(&computation::vectorize))
        .def("unroll", py::overload_cast<var, int>(&computation::unroll))
        .def("interchange", py::overload_cast<var, var>(&computation::interchange))
        .def("store_in", py::overload_cast<buffer *>(&computation::store_in))
        .def("store_in", py::overload_cast<buffer *, std::vector<expr>>(&computation::store_in))
        .def("tile", py::overload_cast<var, var, int, int>(&computation::tile))
        .def("tile", py::overload_cast<var, var, int, int, var, var, var, var>(&computation::tile))
        .def("tile", py::overload_cast<var, var, var, int, int, int>(&computation::tile))
        .def("tile", py::overload_cast<var, var, var, int, int, int, var, var, var, var, var, var>(&computation::tile))
        .def("after", py::overload_cast<computation &, var>(&computation::after))
        .def("after", py::overload_cast<computation &, int>(&computation::after))
        .def("set_expression", &computation::set_expression)
        .def("gpu_tile", py::overload_cast<var, var, int, int>(&computation::gpu_tile))
        .def("gpu_tile", py::overload_cast<var, var, int, int, var, var, var, var>(&computation::gpu_tile))
        .def("gpu_tile", py::overload_cast<var, var, var, int, int, int>(&computation::gpu_tile))
        .def("gpu_tile", py::overload_cast<var, var, var, int, int, int, var, var, var, var, var, var>(&computation::gpu_tile))
        .def("then", py::overload_cast<computation &, var>(&computation::then), py::return_value_policy::reference)
        .def("then", py::overload_cast<computation &, int>(&computation::then), py::return_value_policy::reference)
        .def("split", py::overload_cast<var, int>(&computation::split))
        .def("split", py::overload_cast<var, int, var, var>(&computation::split))
        .def("split", py::overload_cast<int, int>(&computation::split))
        .def("cache_shared", &computation::cache_shared, py::return_value_policy::reference)
        .def("get_buffer", &computation::get_buffer, py::return_value_policy::reference)
        .def("after_low_level", py::overload_cast<computation &, int>(&computation::after_low_level))
        .def("dump", &computation::dump);

    py::class_<input, computation, kept<input>>(m, "input")
        .def(py::init([](std::string name, std::vector<var> iters, primitive_t t) { return new input(name, iters, t); }))
        .def(py::init([](std::vector<var> iters, primitive_t t) { return new input(iters, t); }))
        .def(py::init([](std::string name, std::vector<std::string> dims, std::vector<expr> sizes, primitive_t t) {
            return new input(name, dims, sizes, t);
        }));

    py::class_<constant, computation, kept<constant>>(m, "constant")
        .def(py::init([](std::string name, const expr &e) { return new constant(name, e); }))
        .def(py::init([](std::string name, const expr &e, primitive_t t, bool function_wide, computation *with, int level) {
            return new constant(name, e, t, function_wide, with, level, global::get_implicit_function());
        }))
        .def("__add__", [](constant &c, const expr &o) { return (expr)c + o; })
        .def("__radd__", [](constant &c, const expr &o) { return o + (expr)c; })
        .def("__sub__", [](constant &c, const expr &o) { return (expr)c - o; })
        .def("__rsub__", [](constant &c, const expr &o) { return o - (expr)c; })
        .def("__mul__", [](constant &c, const expr &o) { return (expr)c * o; })
        .def("__rmul__", [](constant &c, const expr &o) { return o * (expr)c; });
    // a constant where an expression is expected (loop bounds: var("i", 0, N)), as constant::operator expr() gives in C++
    py::reinterpret_borrow<py::class_<expr>>(m.attr("expr")).def(py::init([](constant &c) { return (expr)c; }));
    py::implicitly_convertible<constant, expr>();
}

void define_function(py::module &m) {
    py::class_<function, kept<function>>(m, "function")
        .def(py::init([](std::string name) { return new function(name); }))
        .def("get_name", &function::get_name)
        .def("dump", &function::dump)
        .def("dump_halide_stmt", &function::dump_halide_stmt)
        .def("gen_c_code", &function::gen_c_code)
        .def("codegen", [](function &f, const std::vector<buffer *> &args, const std::string &obj, bool gpu, bool) { f.codegen(args, obj, gpu); });
    m.def("init", [](std::string name) { tiramisu::init(name); });
    m.def("get_implicit_function", [] { return global::get_implicit_function(); }, py::return_value_policy::reference);
    m.def("codegen", [](const std::vector<buffer *> &args, const std::string &obj, bool gpu, bool) { tiramisu::codegen(args, obj, gpu); },
          py::arg("arguments"), py::arg("obj_filename"), py::arg("gen_cuda_stmt") = false, py::arg("gen_python") = false);
    m.def("codegen", [](const std::vector<buffer *> &args, const std::string &obj, hardware_architecture_t arch, bool) { tiramisu::codegen(args, obj, arch); },
          py::arg("arguments"), py::arg("obj_filename"), py::arg("gen_architecture_flag"), py::arg("gen_python") = false);
}

}  // namespace

PYBIND11_MODULE(tiramisu, m) {
    m.doc() = "Tiramisu front-end with the HIP (gfx950) back-end";
    define_types(m);
    define_expr(m);
    define_buffer(m);
    define_computation(m);
    define_function(m);
}
