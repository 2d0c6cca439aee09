// pybind11 module tt_buda_amd._C: DataFormat at the top level and the backend_api submodule with
// the names, argument order, GIL policy and pickling of pybuda._C
// (pybuda/csrc/pybuda_bindings.cpp:54-101, pybuda/csrc/backend_api/backend_api.cpp:321-329,
// 384-591, 622-625, 666-725).
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include <iostream>
#include <sstream>

#include "backend.hpp"

namespace py = pybind11;
using namespace tt;

namespace {

// Keeps the Python tensor behind a descriptor alive; dropped under the GIL wherever the last copy
// of the descriptor dies.
std::shared_ptr<void> keep_alive(py::object obj)
{
    auto *held = new py::object(std::move(obj));
    return std::shared_ptr<void>(held, [](void *p) {
        py::gil_scoped_acquire gil;
        delete static_cast<py::object *>(p);
    });
}

void bind_data_format(py::module &m)
{
    py::enum_<DataFormat> e(m, "DataFormat");
    for (const auto &f : detail::kFormats) e.value(f.name, f.df);
    e.export_values();
    e.def("to_json", [](DataFormat df) {
        std::stringstream ss;
        ss << df;
        return ss.str();
    });
    e.def_static("from_json", [](const std::string &name) { return data_format_from_name(name); });

    py::enum_<MathFidelity>(m, "MathFidelity")
        .value("LoFi", MathFidelity::LoFi)
        .value("HiFi2", MathFidelity::HiFi2)
        .value("HiFi3", MathFidelity::HiFi3)
        .value("HiFi4", MathFidelity::HiFi4)
        .value("Invalid", MathFidelity::Invalid)
        .export_values()
        .def("to_json",
             [](MathFidelity f) {
                 std::stringstream ss;
                 ss << f;
                 return ss.str();
             })
        .def_static("from_json", [](const std::string &name) {
            for (MathFidelity f : {MathFidelity::LoFi, MathFidelity::HiFi2, MathFidelity::HiFi3, MathFidelity::HiFi4,
                                   MathFidelity::Invalid}) {
                std::stringstream ss;
                ss << f;
                if (ss.str() == name) return f;
            }
            throw std::out_of_range("Unknown math fidelity: " + name);
        });

    m.def("data_format_byte_size", &data_format_byte_size, py::arg("df"), py::arg("elements") = 1);
    m.def("tile_size_bytes", &balancer::tile_size_bytes, py::arg("data_format"), py::arg("include_header_padding") = true);
    m.def("is_b_data_format", &is_b_data_format);
    m.def("is_a_data_format", &is_a_data_format);
    m.def("is_integer_data_format", &is_integer_data_format);
    m.def("to_a_data_format", &to_a_data_format);
    m.def("to_b_data_format", &to_b_data_format);
    m.def("get_precision_bits", &get_precision_bits);
    m.def("preserve_lower_precision_cast", &preserve_lower_precision_cast);
}

void bind_backend(py::module &m)
{
    py::enum_<DEVICE_STATUS_CODE>(m, "BackendStatusCode")
        .value("Success", DEVICE_STATUS_CODE::Success)
        .value("RuntimeError", DEVICE_STATUS_CODE::RuntimeError)
        .value("TimeoutError", DEVICE_STATUS_CODE::TimeoutError);

    py::enum_<IO_TYPE>(m, "IOType")
        .value("Queue", IO_TYPE::Queue)
        .value("RandomAccess", IO_TYPE::RandomAccess)
        .value("Invalid", IO_TYPE::Invalid);

    py::enum_<IO_LAYOUT>(m, "IOLayout")
        .value("Tilized", IO_LAYOUT::Tilized)
        .value("Flat", IO_LAYOUT::Flat)
        .value("Invalid", IO_LAYOUT::Invalid);

    py::enum_<DEVICE>(m, "BackendType").value("Hip", DEVICE::Hip).value("NoBackend", DEVICE::Invalid);
    py::enum_<ARCH>(m, "BackendDevice").value("MI355X", ARCH::MI355X).value("Invalid", ARCH::Invalid);
    py::enum_<DEVICE_MODE>(m, "DeviceMode")
        .value("CompileAndRun", DEVICE_MODE::CompileAndRun)
        .value("CompileOnly", DEVICE_MODE::CompileOnly)
        .value("RunOnly", DEVICE_MODE::RunOnly);

    // Same constructor arguments and setters as the reference's BackendConfig (backend_api.cpp:243-281); the descriptor
    // paths are kept and not read (there is no SoC or cluster description to load).
    py::class_<tt_backend_config>(m, "BackendConfig")
        .def(py::init([](DEVICE backend_type, ARCH backend_device, DEVICE_MODE device_mode, int opt_level, const std::string &output_dir,
                         const std::string &soc_descriptor_path, const std::string &cluster_descriptor_path) {
                 tt_backend_config cfg;
                 cfg.type = backend_type;
                 cfg.arch = backend_device;
                 cfg.mode = device_mode;
                 cfg.output_dir = output_dir;
                 cfg.soc_descriptor_path = soc_descriptor_path;
                 cfg.cluster_descriptor_path = cluster_descriptor_path;
                 const char *env_opt_level = std::getenv("TT_BACKEND_OPT_LEVEL");
                 cfg.optimization_level = env_opt_level ? std::atoi(env_opt_level) : opt_level;
                 return cfg;
             }),
             py::arg("backend_type") = DEVICE::Hip, py::arg("backend_device") = ARCH::MI355X,
             py::arg("device_mode") = DEVICE_MODE::CompileAndRun, py::arg("opt_level") = 0, py::arg("output_dir") = "",
             py::arg("soc_descriptor_path") = "", py::arg("cluster_descriptor_path") = "")
        .def("set_golden_ignore_df_precision",
             [](tt_backend_config &self, bool ignore_data_format_precision) { self.ignore_data_format_precision = ignore_data_format_precision; })
        .def("set_performance_trace_args", [](tt_backend_config &self, std::string args) { self.perf_desc_args = args; })
        .def("set_runtime_args", [](tt_backend_config &self, std::string args) { self.runtime_args = args; })
        .def_readonly("ignore_data_format_precision", &tt_backend_config::ignore_data_format_precision)
        .def_readonly("optimization_level", &tt_backend_config::optimization_level)
        .def_readonly("output_dir", &tt_backend_config::output_dir)
        .def_readonly("perf_desc_args", &tt_backend_config::perf_desc_args)
        .def_readonly("runtime_args", &tt_backend_config::runtime_args);

    py::class_<Stride>(m, "StrideDescriptor")
        .def(py::init<>())
        .def_readwrite("xy_offsets", &Stride::xy_offsets)
        .def_readwrite("stride", &Stride::stride)
        .def(py::pickle([](const Stride &s) { return py::make_tuple(s.xy_offsets, s.stride); },
                        [](py::tuple t) {
                            if (t.size() != 2) throw std::runtime_error("Invalid state for tt::Stride");
                            Stride s;
                            s.xy_offsets = t[0].cast<std::vector<std::pair<int, int>>>();
                            s.stride = t[1].cast<int>();
                            return s;
                        }));

    py::class_<tt_dram_io_desc>(m, "DramIODesc")
        .def(py::init<>())
        .def_property_readonly("name", [](tt_dram_io_desc &d) { return d.queue_name; })
        .def_property_readonly("data_format", [](tt_dram_io_desc &d) { return d.bufq_target_format; })
        .def_readwrite("bufq_grid_dim_r", &tt_dram_io_desc::bufq_grid_dim_r)
        .def_readwrite("bufq_grid_dim_c", &tt_dram_io_desc::bufq_grid_dim_c)
        .def_readwrite("ublock_rt", &tt_dram_io_desc::ublock_rt)
        .def_readwrite("ublock_ct", &tt_dram_io_desc::ublock_ct)
        .def_readwrite("mblock_m", &tt_dram_io_desc::mblock_m)
        .def_readwrite("mblock_n", &tt_dram_io_desc::mblock_n)
        .def_readwrite("tile_height", &tt_dram_io_desc::tile_height)
        .def_readwrite("tile_width", &tt_dram_io_desc::tile_width)
        .def_readwrite("t", &tt_dram_io_desc::t)
        .def_readwrite("hstack_factor", &tt_dram_io_desc::hstack_factor)
        .def_readwrite("vstack_factor", &tt_dram_io_desc::vstack_factor)
        .def_readwrite("stack_row_major", &tt_dram_io_desc::stack_row_major)
        .def_readwrite("s_descriptor", &tt_dram_io_desc::s_descriptor)
        .def_readwrite("input_count", &tt_dram_io_desc::input_count)
        .def_readwrite("netlist_path", &tt_dram_io_desc::netlist_path)
        .def_readwrite("bufq_target_format", &tt_dram_io_desc::bufq_target_format)
        .def_readwrite("bufq_num_slots", &tt_dram_io_desc::bufq_num_slots)
        .def_readwrite("io_type", &tt_dram_io_desc::io_type)
        .def_readwrite("layout", &tt_dram_io_desc::layout)
        .def_property(
            "ublock_order", [](const tt_dram_io_desc &d) { return std::string(d.ublock_order ? "c" : "r"); },
            [](tt_dram_io_desc &d, const std::string &o) {
                if (o != "r" && o != "c") throw std::runtime_error("ublock_order is 'r' or 'c'");
                d.ublock_order = o == "c";
            })
        .def_property(
            "tile_header", [](const tt_dram_io_desc &d) { return d.tile_header != 0; },
            [](tt_dram_io_desc &d, bool h) { d.tile_header = h; })
        .def_readonly("bufq_start_addr_channel", &tt_dram_io_desc::bufq_start_addr_channel)
        .def_readonly("bufq_entry_size", &tt_dram_io_desc::bufq_entry_size)
        .def(py::pickle(
            [](const tt_dram_io_desc &p) {
                return py::make_tuple(p.netlist_path, p.queue_name, p.bufq_grid_dim_r, p.bufq_grid_dim_c, p.bufq_num_slots,
                                      p.ublock_rt, p.ublock_ct, p.mblock_m, p.mblock_n, p.tile_height, p.tile_width, p.t,
                                      p.input_count, p.hstack_factor, p.vstack_factor, p.stack_row_major, p.bufq_target_format,
                                      p.bufq_start_addr_channel, p.bufq_entry_size, p.io_type, p.s_descriptor, p.backend_type,
                                      p.layout, p.ublock_order, p.tile_header);
            },
            [](py::tuple t) {  // the reference's 23 fields, then the two this build keeps in the descriptor
                if (t.size() != 23 && t.size() != 25) throw std::runtime_error("tt::tt_dram_io_desc: Invalid state!");
                tt_dram_io_desc p;
                p.netlist_path = t[0].cast<std::string>();
                p.queue_name = t[1].cast<std::string>();
                p.bufq_grid_dim_r = t[2].cast<std::uint32_t>();
                p.bufq_grid_dim_c = t[3].cast<std::uint32_t>();
                p.bufq_num_slots = t[4].cast<std::uint32_t>();
                p.ublock_rt = t[5].cast<std::uint32_t>();
                p.ublock_ct = t[6].cast<std::uint32_t>();
                p.mblock_m = t[7].cast<std::uint32_t>();
                p.mblock_n = t[8].cast<std::uint32_t>();
                p.tile_height = t[9].cast<std::uint32_t>();
                p.tile_width = t[10].cast<std::uint32_t>();
                p.t = t[11].cast<std::uint32_t>();
                p.input_count = t[12].cast<std::uint32_t>();
                p.hstack_factor = t[13].cast<std::uint32_t>();
                p.vstack_factor = t[14].cast<std::uint32_t>();
                p.stack_row_major = t[15].cast<std::uint32_t>();
                p.bufq_target_format = t[16].cast<DataFormat>();
                p.bufq_start_addr_channel = t[17].cast<std::vector<std::pair<std::uint32_t, std::uint16_t>>>();
                p.bufq_entry_size = t[18].cast<std::uint32_t>();
                p.io_type = t[19].cast<IO_TYPE>();
                p.s_descriptor = t[20].cast<Stride>();
                p.backend_type = t[21].cast<DEVICE>();
                p.layout = t[22].cast<IO_LAYOUT>();
                if (t.size() == 25) {
                    p.ublock_order = t[23].cast<std::uint32_t>();
                    p.tile_header = t[24].cast<std::uint32_t>();
                }
                return p;
            }));

    py::class_<tt_PytorchTensorDesc>(m, "PytorchTensorDesc", py::buffer_protocol())
        .def(py::init<>())
        .def(py::init([](py::object pytorch_tensor, std::uint32_t itemsize, DataFormat format, std::uint32_t dim,
                         std::array<std::uint32_t, 4> shape, std::array<std::uint32_t, 4> strides) {
            const auto ptr = pytorch_tensor.attr("data_ptr")().cast<std::uint64_t>();
            return tt_PytorchTensorDesc((const void *)ptr, itemsize, format, shape, strides, dim,
                                        keep_alive(std::move(pytorch_tensor)));
        }))
        .def(py::init([](std::uint64_t buffer, std::uint32_t itemsize, DataFormat format, std::uint32_t dim,
                         std::array<std::uint32_t, 4> shape, std::array<std::uint32_t, 4> strides) {
            return tt_PytorchTensorDesc((const void *)buffer, itemsize, format, shape, strides, dim);
        }))
        .def_readwrite("itemsize", &tt_PytorchTensorDesc::itemsize)
        .def_readwrite("format", &tt_PytorchTensorDesc::format)
        .def_readwrite("shape", &tt_PytorchTensorDesc::shape)
        .def_readwrite("strides", &tt_PytorchTensorDesc::strides)
        .def_readwrite("dim", &tt_PytorchTensorDesc::dim)
        .def_property_readonly("ptr", [](const tt_PytorchTensorDesc &d) { return (std::uint64_t)d.ptr; })
        .def("print",
             [](tt_PytorchTensorDesc &d) {
                 std::cout << "Descriptor: ptr=" << (std::uint64_t)d.ptr << ", itemsize=" << d.itemsize
                           << ", format =" << (int)d.format << ", dim =" << d.dim << ", shape =" << d.shape[0] << ","
                           << d.shape[1] << "," << d.shape[2] << "," << d.shape[3] << ", strides =" << d.strides[0] << ","
                           << d.strides[1] << "," << d.strides[2] << "," << d.strides[3] << std::endl;
             })
        // 4-D buffer whose format string is always `float`, as in the reference: the consumer
        // (torch.frombuffer) reinterprets the bytes with its own dtype.
        .def_buffer([](tt_PytorchTensorDesc &d) -> py::buffer_info {
            return py::buffer_info(const_cast<void *>(d.ptr), d.itemsize, py::format_descriptor<float>::format(), 4,
                                   d.shape, d.strides);
        })
        .def(py::pickle(
            [](const tt_PytorchTensorDesc &t) {
                return py::make_tuple(reinterpret_cast<std::uintptr_t>(t.ptr), t.itemsize, t.format, t.shape, t.strides, t.dim);
            },
            [](py::tuple t) {
                if (t.size() != 6) throw std::runtime_error("tt::tt_PytorchTensorDesc: Invalid state!");
                tt_PytorchTensorDesc p;
                p.ptr = reinterpret_cast<const void *>(t[0].cast<std::uintptr_t>());
                p.itemsize = t[1].cast<std::uint32_t>();
                p.format = t[2].cast<DataFormat>();
                p.shape = t[3].cast<std::array<std::uint32_t, 4>>();
                p.strides = t[4].cast<std::array<std::uint32_t, 4>>();
                p.dim = t[5].cast<std::uint32_t>();
                return p;
            }));

    py::class_<tt_TilizedTensorDesc>(m, "TilizedTensorDesc")
        .def(py::init<>())
        .def_readwrite("num_buffers", &tt_TilizedTensorDesc::num_buffers)
        .def_readwrite("buf_size_bytes", &tt_TilizedTensorDesc::buf_size_bytes)
        .def_readwrite("format", &tt_TilizedTensorDesc::format)
        .def_property_readonly("ptr", [](const tt_TilizedTensorDesc &d) { return (std::uint64_t)d.ptr; })
        .def("print",
             [](tt_TilizedTensorDesc &d) {
                 std::cout << "Descriptor: ptr=" << (std::uint64_t)d.ptr << ", num_buffers=" << d.num_buffers
                           << ", buf_size_bytes=" << (int)d.buf_size_bytes << ", format =" << d.format;
             })
        // the pointer is not part of the state: a reloaded descriptor is filled by debinarize_tensor
        .def(py::pickle([](const tt_TilizedTensorDesc &t) { return py::make_tuple(t.num_buffers, t.buf_size_bytes, t.format); },
                        [](py::tuple t) {
                            if (t.size() != 3) throw std::runtime_error("tt::tt_TilizedTensorDesc: Invalid state!");
                            return tt_TilizedTensorDesc(nullptr, t[0].cast<std::uint32_t>(), t[1].cast<std::uint32_t>(),
                                                        t[2].cast<DataFormat>());
                        }));

    py::class_<tt_backend, std::shared_ptr<tt_backend>>(m, "BackendApi")
        .def(py::init(&tt_backend::create), py::arg("device") = 0, py::arg("config") = tt_backend_config())
        .def("get_config", &tt_backend::config)
        .def("queue_storage_format", &tt_backend::queue_storage_format)
        .def("queue_max_in_flight", &tt_backend::queue_max_in_flight)
        .def("queue_in_flight", &tt_backend::queue_in_flight)
        .def("initialize", &tt_backend::initialize, py::call_guard<py::gil_scoped_release>())
        .def("finish", &tt_backend::finish)
        .def("wait_for_idle", &tt_backend::wait_for_idle, py::call_guard<py::gil_scoped_release>())
        .def("create_queue", &tt_backend::create_queue, py::arg("name"), py::arg("data_format"), py::arg("t"),
             py::arg("mblock_m"), py::arg("mblock_n"), py::arg("ublock_rt") = 1, py::arg("ublock_ct") = 1,
             py::arg("num_slots") = 2, py::arg("io_type") = IO_TYPE::Queue, py::arg("input_count") = 1, py::arg("grid_r") = 1,
             py::arg("grid_c") = 1, py::arg("ublock_order") = 0, py::arg("tile_header") = false)
        .def("get_queue_descriptor", &tt_backend::get_queue_descriptor)
        .def("run_matmul", &tt_backend::run_matmul, py::arg("in0"), py::arg("weight"), py::arg("bias"), py::arg("out"),
             py::arg("gelu") = false, py::arg("timeout") = 10, py::arg("approximate") = "none",
             py::call_guard<py::gil_scoped_release>());

    m.def("release_backend_ptr", [](std::shared_ptr<tt_backend> b) { b.reset(); });

    // the reference's five positional arguments, then the two tile-broadcast flags of this build
    m.def("push_input",
          py::overload_cast<const tt_dram_io_desc &, const tt_PytorchTensorDesc &, const bool, const int, const int, const bool, const bool>(
              &backend::push_input),
          py::arg("queue"), py::arg("tensor"), py::arg("push_one"), py::arg("timeout"), py::arg("ram_ptr"),
          py::arg("tile_broadcast_r") = false, py::arg("tile_broadcast_c") = false, py::call_guard<py::gil_scoped_release>());
    m.def("push_input",
          py::overload_cast<const tt_dram_io_desc &, const tt_TilizedTensorDesc &, const int, const int>(&backend::push_input),
          py::call_guard<py::gil_scoped_release>());
    m.def("pop_output", &backend::pop_output, py::call_guard<py::gil_scoped_release>());
    m.def("get_output", &backend::get_output, py::arg("queue"), py::arg("out"), py::arg("pop_one"), py::arg("timeout"), py::arg("rd_ptr"),
          py::arg("narrow_r") = 0, py::arg("narrow_c") = 0, py::call_guard<py::gil_scoped_release>());
    m.def("pad_to_buda_shape", &backend::pad_to_buda_shape);
    m.def("align_up_tile", [](std::uint32_t d) { return align_up_tile(d); });
    m.def("pool_allocations", &backend::pool_allocations);
    m.def("free_tensor", &backend::free_tensor<tt_PytorchTensorDesc>);
    m.def("free_tensor", &backend::free_tensor<tt_TilizedTensorDesc>);
    m.def("tilize_tensor", &backend::tilize_tensor);
    m.def("binarize_tensor", &backend::binarize_tensor<tt_PytorchTensorDesc>);
    m.def("binarize_tensor", &backend::binarize_tensor<tt_TilizedTensorDesc>);
    m.def("debinarize_tensor", &backend::debinarize_tensor<tt_PytorchTensorDesc>);
    m.def("debinarize_tensor", &backend::debinarize_tensor<tt_TilizedTensorDesc>);
    m.def("get_io_size_in_bytes", &backend::get_io_size_in_bytes, py::arg("data_formati"), py::arg("is_untilizesd"),
          py::arg("ublock_ct"), py::arg("ublock_rt"), py::arg("mblock_m"), py::arg("mblock_n"), py::arg("t"),
          py::arg("entries"), py::arg("tile_height") = 32, py::arg("tile_width") = 32);
    m.def("translate_addresses", &backend::translate_addresses, py::call_guard<py::gil_scoped_release>());
    m.def("get_format_from_string", &data_format_from_name, py::arg("format_str"));
    m.def("last_error", &backend::last_error);
}

}  // namespace

PYBIND11_MODULE(_C, m)
{
    m.attr("__name__") = "tt_buda_amd._C";
    m.attr("VERSION") = py::int_(1);
    bind_data_format(m);
    py::module_ m_backend = m.def_submodule("backend_api", "Tensor boundary of the MI355X backend");
    bind_backend(m_backend);
}
