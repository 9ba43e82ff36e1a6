// Host-side helper of the Python binding: one pass over a Python list of tensors
// that validates it against a tensor table and writes the per-call pointer and
// mode arrays the C ABI takes (yafsdp_gather_in / yafsdp_scatter_out).
//
// The same checks written in Python cost about 0.6 us per tensor (five
// interpreter-level passes); a parameter group with 1,400 tensors then spends
// longer on the host than its kernel runs.  This pass takes about 10 ns per
// tensor.  It moves no tensor data and launches nothing; the kernels and the
// C ABI stay free of torch types.  Any list it does not accept is handed back to
// the Python checks, which raise the descriptive error.
#include <Python.h>
#include <torch/csrc/autograd/python_variable.h>
#include <torch/extension.h>

#include <cstdint>

namespace {

constexpr int kModeSkip = 0, kModeCopy = 1;
constexpr int64_t kRejected = -1000;  // let the Python checks explain

inline int dtype_code(at::ScalarType t) {
  switch (t) {
    case at::kFloat: return 0;
    case at::kBFloat16: return 1;
    case at::kHalf: return 2;
    default: return -1;
  }
}

// tensors: list/tuple of Tensor or None.  modes: None, or list/tuple of ints (0 skip, 1 copy, 2 add).
// numels_addr: int64[n] expected element counts.  ptrs_addr: uint64[n] out.  modes_addr: uint8[n] out.
// Returns the dtype code shared by the live tensors, -1 if every tensor is skipped, kRejected otherwise.
int64_t fill(py::handle tensors, py::handle modes, uint64_t numels_addr, uint64_t ptrs_addr, uint64_t modes_addr,
             bool want_cuda, int64_t device_index) {
  PyObject* seq = tensors.ptr();
  if (!PyList_Check(seq) && !PyTuple_Check(seq)) return kRejected;
  const Py_ssize_t n = PySequence_Fast_GET_SIZE(seq);
  PyObject** items = PySequence_Fast_ITEMS(seq);
  PyObject** mode_items = nullptr;
  if (!modes.is_none()) {
    PyObject* m = modes.ptr();
    if ((!PyList_Check(m) && !PyTuple_Check(m)) || PySequence_Fast_GET_SIZE(m) != n) return kRejected;
    mode_items = PySequence_Fast_ITEMS(m);
  }
  const auto* numels = reinterpret_cast<const int64_t*>(numels_addr);
  auto* ptrs = reinterpret_cast<uint64_t*>(ptrs_addr);
  auto* out_modes = reinterpret_cast<uint8_t*>(modes_addr);
  int code = -1;
  for (Py_ssize_t i = 0; i < n; ++i) {
    PyObject* o = items[i];
    int mode = kModeCopy;
    if (mode_items != nullptr) {
      const long v = PyLong_AsLong(mode_items[i]);
      if (v == -1 && PyErr_Occurred()) {
        PyErr_Clear();
        return kRejected;
      }
      if (v < 0 || v > 2) return kRejected;
      mode = static_cast<int>(v);
    }
    if (o == Py_None) mode = kModeSkip;
    out_modes[i] = static_cast<uint8_t>(mode);
    if (mode == kModeSkip) {
      ptrs[i] = 0;
      continue;
    }
    if (!THPVariable_Check(o)) return kRejected;
    const at::Tensor& t = THPVariable_Unpack(o);
    const int c = dtype_code(t.scalar_type());
    if (c < 0 || (code >= 0 && c != code)) return kRejected;
    code = c;
    if (t.numel() != numels[i] || !t.is_contiguous()) return kRejected;
    const auto dev = t.device();
    if (want_cuda ? !(dev.is_cuda() && dev.index() == device_index) : !dev.is_cpu()) return kRejected;
    ptrs[i] = reinterpret_cast<uint64_t>(t.data_ptr());
  }
  return code;
}

// True if every tensor of the list (None entries aside) is contiguous.
bool all_contiguous(py::handle tensors) {
  PyObject* seq = tensors.ptr();
  if (!PyList_Check(seq) && !PyTuple_Check(seq)) throw py::type_error("expected a list or tuple of tensors");
  const Py_ssize_t n = PySequence_Fast_GET_SIZE(seq);
  PyObject** items = PySequence_Fast_ITEMS(seq);
  for (Py_ssize_t i = 0; i < n; ++i) {
    PyObject* o = items[i];
    if (o == Py_None) continue;
    if (!THPVariable_Check(o)) throw py::type_error("expected a list or tuple of tensors");
    if (!THPVariable_Unpack(o).is_contiguous()) return false;
  }
  return true;
}

}  // namespace

PYBIND11_MODULE(_tensorlist, m) {
  m.attr("REJECTED") = kRejected;
  m.def("fill", &fill, "validate a tensor list against a table and write its pointer / mode arrays");
  m.def("all_contiguous", &all_contiguous);
}
