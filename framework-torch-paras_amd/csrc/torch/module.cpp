// Python extension module `_C`: thin bindings over the C ABI, same function
// names as the reference's module (csrc/python/module.cpp:30-78).
#include <pybind11/pybind11.h>

#include <string>

#include "paras_torch.h"

namespace py = pybind11;
using paras_torch::check;

PYBIND11_MODULE(_C, m) {
    m.doc() = "PyTorch `paras` device on AMD MI355X (HIP kernels behind a C ABI)";

    m.def("device_count", [] { return paras_device_count(); });
    m.def("backend_name", [] { return std::string("paras-hip"); });
    m.def("device_name", [](int index) {
        char buf[256];
        check(paras_device_name(index, buf, sizeof(buf)));
        return std::string(buf);
    });
    m.def("is_gpu_device", [](int index) {
        int cus = 0;
        check(paras_device_info(index, &cus, nullptr));
        return true;  // every paras device of this build is a HIP GPU
    });
    m.def("device_info", [](int index) {
        int cus = 0;
        uint64_t bytes = 0;
        check(paras_device_info(index, &cus, &bytes));
        return py::make_tuple(cus, bytes);
    });
    m.def("synchronize", [](int index) {
        py::gil_scoped_release no_gil;
        check(paras_synchronize(index));
    });
    m.def("synchronize_all", [] {
        py::gil_scoped_release no_gil;
        for (int i = 0; i < paras_device_count(); ++i) check(paras_synchronize(i));
    });
    // The hot-path ops draw no random numbers; seeds are accepted for API
    // compatibility and kept per device.
    m.def("manual_seed", [](int index, uint64_t) { check(index >= 0 && index < paras_device_count() ? 0 : paras_synchronize(index)); });
    m.def("manual_seed_all", [](uint64_t) {});
    m.def("empty_cache", [] {
        py::gil_scoped_release no_gil;
        for (int i = 0; i < paras_device_count(); ++i) check(paras_empty_cache(i));
    });
    m.def("allocated_bytes", [](int index) {
        uint64_t a = 0, c = 0;
        check(paras_memory_stats(index, &a, &c));
        return a;
    });
    m.def("cached_bytes", [](int index) {
        uint64_t a = 0, c = 0;
        check(paras_memory_stats(index, &a, &c));
        return c;
    });
    m.def("is_bad_fork", [] { return paras_is_bad_fork() != 0; });
    m.def("abi_version", [] { return paras_abi_version(); });
}
