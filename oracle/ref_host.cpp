// TEST INFRASTRUCTURE — not part of the shipped library.
//
// Hosts the reference's own header-only CPU Adam (csrc/include/adam_cpu.hpp,
// csrc/include/cpu_info.h) in a pybind11 module so that the oracle restatement
// in this directory can be validated against the real compiled reference, and
// so that bench.py can time the reference's CPU path ("cpu_baseline.kind =
// reference").  The header is included from where it lies under the reference
// checkout (-I<reference>/csrc/include on the command line, see Makefile);
// no reference source is copied here.  The header uses `py::gil_scoped_release`
// (adam_cpu.hpp:64) and expects the `py` alias that the reference declares in
// csrc/include/nccl.hpp:5, hence the alias below.
#include <pybind11/pybind11.h>
#include <cstring>
namespace py = pybind11;
#include "adam_cpu.hpp"

PYBIND11_MODULE(refadam, m) {
    m.def("get_cpu_level", &get_cpu_level);
    m.def("adam_cpu_fp16_launcher", &adam_cpu_fp16_launcher);
    m.def("adam_cpu_bf16_launcher", &adam_cpu_bf16_launcher);
    m.def("to_fp16_from_fp32", &fp16_from_fp32_value_launcher);
    m.def("to_bf16_from_fp32", &bf16_from_fp32_value_launcher);
}
