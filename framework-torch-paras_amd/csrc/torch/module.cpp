// Python extension module `_C`: thin bindings over the C ABI, same function
// names as the reference's module (csrc/python/module.cpp:30-78).
#include <pybind11/pybind11.h>

#include <string>

#include "paras_torch.h"

namespace py = pybind11;
using paras_torch::check;
using paras_torch::hip_device;

PYBIND11_MODULE(_C, m) {
    m.doc() = "PyTorch `paras` device on AMD MI355X (HIP kernels behind a C ABI)";

    m.def("device_count", [] { return paras_torch::device_count_torch(); });
    m.def("device_base", [] { return paras_torch::device_base(); });
    m.def("current_device", [] { return static_cast<int>(paras_torch::current_device()); });
    m.def("backend_name", [] { return std::string("paras-hip"); });
    m.def("device_name", [](int index) {
        char buf[256];
        check(paras_device_name(hip_device(index), buf, sizeof(buf)));
        return std::string(buf);
    });
    m.def("is_gpu_device", [](int index) {
        if (paras_torch::device_base() == 1 && index == 0) return false;   // the reference's host engine slot
        int cus = 0;
        check(paras_device_info(hip_device(index), &cus, nullptr));
        return true;  // every paras device of this build is a HIP GPU
    });
    m.def("device_info", [](int index) {
        int cus = 0;
        uint64_t bytes = 0;
        check(paras_device_info(hip_device(index), &cus, &bytes));
        return py::make_tuple(cus, bytes);
    });
    m.def("synchronize", [](int index) {
        const int hip = hip_device(index);
        py::gil_scoped_release no_gil;
        check(paras_synchronize(hip));
    });
    m.def("synchronize_all", [] {
        py::gil_scoped_release no_gil;
        for (int i = 0; i < paras_device_count(); ++i) check(paras_synchronize(i));
    });
    // The hot-path ops draw no random numbers; seeds are accepted for API
    // compatibility and kept per device.
    m.def("manual_seed", [](int index, uint64_t) { (void)hip_device(index); });
    m.def("manual_seed_all", [](uint64_t) {});
    m.def("empty_cache", [] {
        py::gil_scoped_release no_gil;
        for (int i = 0; i < paras_device_count(); ++i) check(paras_empty_cache(i));
    });
    m.def("allocated_bytes", [](int index) {
        uint64_t a = 0, c = 0;
        check(paras_memory_stats(hip_device(index), &a, &c));
        return a;
    });
    m.def("cached_bytes", [](int index) {
        uint64_t a = 0, c = 0;
        check(paras_memory_stats(hip_device(index), &a, &c));
        return c;
    });
    m.def("is_bad_fork", [] { return paras_is_bad_fork() != 0; });
    m.def("abi_version", [] { return paras_abi_version(); });
}
