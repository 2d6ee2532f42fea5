// pybind11 bindings of libave_fp4.so's GEMM entry points (include/ave_fp4.h): the hop through python/src that a
// caller inside the avelang Python package takes.  The reference's extension module exports compiler classes only
// (python/src/avelang_bindings.cc:493-529); these functions are an addition in the same style and with the same
// conventions as the reference's kernel launch path:
//   * a pointer argument is an int, None, or any object with a data_ptr() method
//     (python/avelang/backends/amdgpu/driver.py:154-189);
//   * the GIL is released around the call into the library (driver.py:357-359);
//   * a rejected argument raises ValueError, a HIP failure RuntimeError with the text
//     "ave-lang Error [HIP]: ..." (driver.py:125-138; std::runtime_error -> RuntimeError as in
//     avelang_bindings.cc:44,131-133).
// Every bound function has the name and the argument order of its C symbol and returns 0, so that the Python
// wrappers can call through this module or through the ctypes binding alike.
#include <pybind11/pybind11.h>

#include <cstdint>
#include <stdexcept>
#include <type_traits>
#include <utility>

#include "ave_fp4.h"

namespace py = pybind11;

struct DevPtr {
  uintptr_t value = 0;
};

namespace pybind11 {
namespace detail {
template <>
struct type_caster<DevPtr> {
  PYBIND11_TYPE_CASTER(DevPtr, const_name("pointer"));
  bool load(handle src, bool) {
    if (src.is_none()) {   // a valid null pointer
      value.value = 0;
      return true;
    }
    object held;
    handle number = src;
    if (!PyLong_Check(src.ptr())) {
      if (!hasattr(src, "data_ptr")) throw type_error("Pointer argument must be either uint64 or have data_ptr method");
      held = src.attr("data_ptr")();
      if (!PyLong_Check(held.ptr())) throw type_error("data_ptr method of Pointer object must return 64-bit int");
      number = held;
    }
    const unsigned long long v = PyLong_AsUnsignedLongLong(number.ptr());
    if (PyErr_Occurred()) throw error_already_set();
    value.value = static_cast<uintptr_t>(v);
    return true;
  }
};
}  // namespace detail
}  // namespace pybind11

namespace {

// Python-side type of a C parameter: every pointer becomes a DevPtr, everything else stays.
template <typename T>
struct PyArg {
  using type = T;
  static T to_c(T v) { return v; }
};
template <typename T>
struct PyArg<T*> {
  using type = DevPtr;
  static T* to_c(DevPtr p) { return reinterpret_cast<T*>(p.value); }
};

void check(int rc) {
  if (rc == 0) return;
  const char* msg = ave_fp4_last_error();
  if (rc == AVE_FP4_EINVAL) throw py::value_error(msg);
  throw std::runtime_error(msg && msg[0] ? msg : "ave-lang Error [HIP]: unknown error");
}

// int fn(A...) -> a Python callable with the same arguments that releases the GIL around the call
template <typename... A>
auto launcher(int (*fn)(A...)) {
  return [fn](typename PyArg<A>::type... args) {
    int rc;
    {
      py::gil_scoped_release nogil;
      rc = fn(PyArg<A>::to_c(args)...);
    }
    check(rc);
    return 0;
  };
}

}  // namespace

#define AVE_BIND(name) m.def(#name, launcher(&name))

PYBIND11_MODULE(_ave_fp4_bindings, m) {
  m.doc() = "block-scaled FP4 GEMM for MI355X: pybind11 bindings of libave_fp4.so";
  AVE_BIND(ave_fp4_gemm_mxfp4);
  AVE_BIND(ave_fp4_gemm_mxfp4_ex);
  AVE_BIND(ave_fp4_gemm_mxfp4_ws);
  AVE_BIND(ave_fp4_gemm_mxfp4_noalloc);
  AVE_BIND(ave_fp4_gemm_mxfp4_blocked_scales);
  AVE_BIND(ave_fp4_gemm_mxfp4_swiglu);
  AVE_BIND(ave_fp4_gemm_mxfp4_swiglu_ex);
  AVE_BIND(ave_fp4_gemm_mxfp4_swiglu_quant);
  AVE_BIND(ave_fp4_gemm_mxfp4_swiglu_quant_padded);
  AVE_BIND(ave_fp4_gemm_nvfp4);
  AVE_BIND(ave_fp4_gemm_nvfp4_ex);
  AVE_BIND(ave_fp4_gemm_nvfp4_ws);
  AVE_BIND(ave_fp4_grouped_gemm_mxfp4);
  AVE_BIND(ave_fp4_grouped_gemm_mxfp4_ex);
  AVE_BIND(ave_fp4_grouped_gemm_mxfp4_swiglu);
  AVE_BIND(ave_fp4_grouped_gemm_mxfp4_swiglu_quant);
  AVE_BIND(ave_fp4_grouped_gemm_mxfp4_swiglu_quant_padded);
  AVE_BIND(ave_fp4_quantize_mxfp4_f32);
  AVE_BIND(ave_fp4_quantize_mxfp4_bf16);
  AVE_BIND(ave_fp4_quantize_mxfp4_f32_padded);
  AVE_BIND(ave_fp4_quantize_mxfp4_bf16_padded);
  AVE_BIND(ave_fp4_quantize_nvfp4_f32);
  AVE_BIND(ave_fp4_quantize_nvfp4_bf16);
  m.def("ave_fp4_gemm_mxfp4_workspace_bytes", &ave_fp4_gemm_mxfp4_workspace_bytes);
  m.def("ave_fp4_gemm_nvfp4_workspace_bytes", &ave_fp4_gemm_nvfp4_workspace_bytes);
  m.def("ave_fp4_abi_version", &ave_fp4_abi_version);
  m.def("ave_fp4_last_error", []() { return std::string(ave_fp4_last_error()); });
}
