// Extension-module binding of libstof_hip.so's C ABI (include/stof_abi.h) for Python.
//
// The reference binds its launcher with a pybind11 module per operator
// (src/ops/src/block_attn_mask.cpp:17-56, built by src/setup.py:27-57).  This is the counterpart:
// one module, `_stof_ext`, that exposes every function of the C ABI under its own name.  It holds
// no logic - arguments are converted and the C function is called - and needs no torch header:
// device pointers and the stream arrive as Python ints (tensor.data_ptr(), the raw stream handle),
// None stands for NULL, and an int64[3] stride triple is a sequence of three ints.  Against the
// ctypes binding of the same functions it saves the per-argument marshalling of a 30-argument call
// (about 11 us -> 3 us per attention call), which is what paces launches shorter than that.
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include <array>
#include <cstdint>

#include "stof_abi.h"

namespace py = pybind11;

namespace {

// C parameter type -> the Python-side parameter type and the conversion
template <class T> struct Arg {
  using py_t = T;
  static T get(const T& v) { return v; }
};
template <class T> struct Arg<T*> {   // any pointer: an int address or None
  using py_t = py::object;
  static T* get(const py::object& o) { return o.is_none() ? nullptr : reinterpret_cast<T*>(o.cast<uintptr_t>()); }
};
template <> struct Arg<const int64_t*> {   // the stride triples of the attention entry points
  using py_t = std::array<int64_t, 3>;
  static const int64_t* get(const std::array<int64_t, 3>& a) { return a.data(); }
};

template <class R, class... A>
auto wrap(R (*f)(A...)) {
  return [f](typename Arg<A>::py_t... a) -> R { return f(Arg<A>::get(a)...); };
}

}  // namespace

#define STOF_BIND(name) m.def(#name, wrap(&name))

PYBIND11_MODULE(_stof_ext, m) {
  m.doc() = "pybind11 binding of libstof_hip.so (C ABI of include/stof_abi.h); pointers and streams are ints";
  STOF_BIND(stof_abi_version);
  STOF_BIND(stof_device_compute_units);
  STOF_BIND(stof_probe_clock);
  STOF_BIND(stof_probe_issue_mix);
  m.def("stof_status_string", [](int status) { return py::bytes(stof_status_string(status)); });
  STOF_BIND(stof_block_attn_fwd);
  STOF_BIND(stof_block_attn_fwd_planned);
  STOF_BIND(stof_attn_plan_rows);
  STOF_BIND(stof_attn_plan_bytes);
  STOF_BIND(stof_attn_plan_build);
  STOF_BIND(stof_pack_mask_bits);
  STOF_BIND(stof_rowwise_attn_fwd);
  STOF_BIND(stof_build_lut_workspace_bytes);
  STOF_BIND(stof_build_lut_nnz_offset);
  STOF_BIND(stof_build_lut);
  STOF_BIND(stof_retile_lut);
  STOF_BIND(stof_build_lut_static_max_tiles);
  STOF_BIND(stof_build_lut_static);
  STOF_BIND(stof_lut_additive_blocks);
  STOF_BIND(stof_bias_res_ln);
  STOF_BIND(stof_gemm_bias_act);
  STOF_BIND(stof_gemm_act_gemm_workspace_bytes);
  STOF_BIND(stof_gemm_act_gemm);
  STOF_BIND(stof_gemm_bias_act_splitk_plan);
  STOF_BIND(stof_gemm_bias_act_splitk_workspace_bytes);
  STOF_BIND(stof_gemm_bias_act_splitk);
  STOF_BIND(stof_gemm_bias_res_ln);
  STOF_BIND(stof_bias_res_ln_dt);
  STOF_BIND(stof_gemm_bias_act_dt);
  STOF_BIND(stof_gemm_bias_act_splitk_dt);
  STOF_BIND(stof_gemm_bias_res_ln_cluster_dt);
  STOF_BIND(stof_gemm_bias_res_ln_cluster_bounded);
  STOF_BIND(stof_gemm_bias_res_ln_cluster_workspace_bytes);
  STOF_BIND(stof_gemm_bias_res_ln_cluster);
}
