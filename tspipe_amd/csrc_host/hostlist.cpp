// Host-side helper for the Python adapters: walks Python lists of tensors at
// C++ speed.  A parameter list has 150+ tensors and the per-tensor Python work
// (data_ptr, numel, dtype/device/shape/contiguity checks) costs more than the
// EMA kernel itself; here it is one call.  No GPU work happens in this module.
#include <torch/extension.h>
#include <torch/csrc/autograd/python_variable.h>

#include <cstdint>
#include <vector>

namespace {

enum Status : int {
  kOk = 0,
  kHasNone = 1,        // a student entry is None
  kNotTensor = 2,
  kNotF32 = 3,
  kNotCudaOrMixed = 4, // CPU tensor, or tensors on different devices
  kShapeMismatch = 5,
  kNotContiguous = 6,
};

inline uint64_t mix(uint64_t h, uint64_t v) {
  h ^= v + 0x9e3779b97f4a7c15ull + (h << 6) + (h >> 2);
  return h;
}

// Checks the (student, teacher) pairs of two lists, zip-style (stops at the
// shorter list), and writes data pointers and element counts into the caller's
// arrays (capacity entries each).  Returns (status, pairs, device index,
// shape hash, total elements).  On a non-zero status the arrays are unspecified.
py::tuple pair_info(py::list students, py::list teachers, uintptr_t s_ptr_out, uintptr_t t_ptr_out,
                    uintptr_t numel_out, int64_t capacity) {
  auto* sp = reinterpret_cast<uint64_t*>(s_ptr_out);
  auto* tp = reinterpret_cast<uint64_t*>(t_ptr_out);
  auto* nn = reinterpret_cast<int64_t*>(numel_out);
  const int64_t n = std::min<int64_t>(py::len(students), py::len(teachers));
  if (n > capacity) throw std::runtime_error("pair_info: output arrays too small");
  int status = kOk;
  int device = -1;
  uint64_t hash = 0x243f6a8885a308d3ull;
  int64_t total = 0;
  for (int64_t i = 0; i < n; ++i) {
    PyObject* so = PyList_GET_ITEM(students.ptr(), i);
    PyObject* to = PyList_GET_ITEM(teachers.ptr(), i);
    if (so == Py_None) { status = kHasNone; break; }
    if (!THPVariable_Check(so) || !THPVariable_Check(to)) { status = kNotTensor; break; }
    const at::Tensor& s = THPVariable_Unpack(so);
    const at::Tensor& t = THPVariable_Unpack(to);
    if (s.scalar_type() != at::kFloat || t.scalar_type() != at::kFloat) { status = kNotF32; break; }
    if (!s.is_cuda() || !t.is_cuda()) { status = kNotCudaOrMixed; break; }
    const int ds = s.get_device(), dt = t.get_device();
    if (device < 0) device = dt;
    if (ds != device || dt != device) { status = kNotCudaOrMixed; break; }
    if (s.sizes() != t.sizes()) { status = kShapeMismatch; break; }
    if (!s.is_contiguous() || !t.is_contiguous()) { status = kNotContiguous; break; }
    sp[i] = reinterpret_cast<uint64_t>(s.data_ptr());
    tp[i] = reinterpret_cast<uint64_t>(t.data_ptr());
    nn[i] = t.numel();
    total += nn[i];
    hash = mix(hash, (uint64_t)t.dim());
    for (auto d : t.sizes()) hash = mix(hash, (uint64_t)d);
  }
  return py::make_tuple(status, n, device, hash, total);
}

// Data pointers of a list of tensors into the caller's array.
int64_t data_ptrs(py::list tensors, uintptr_t ptr_out, int64_t capacity) {
  auto* out = reinterpret_cast<uint64_t*>(ptr_out);
  const int64_t n = py::len(tensors);
  if (n > capacity) throw std::runtime_error("data_ptrs: output array too small");
  for (int64_t i = 0; i < n; ++i) {
    PyObject* o = PyList_GET_ITEM(tensors.ptr(), i);
    if (!THPVariable_Check(o)) throw std::runtime_error("data_ptrs: not a tensor");
    out[i] = reinterpret_cast<uint64_t>(THPVariable_Unpack(o).data_ptr());
  }
  return n;
}

// True when every tensor of the list is referenced only by the list itself and
// by the caller's argument handling (Python refcount == expected), and no
// C++ holder keeps its TensorImpl either (a view saved by autograd for a
// backward pass, a tensor list inside another extension): such a holder
// changes neither the Python refcount nor the storage's use count.
bool all_refcounts_equal(py::list tensors, int64_t expected) {
  const int64_t n = py::len(tensors);
  for (int64_t i = 0; i < n; ++i) {
    PyObject* o = PyList_GET_ITEM(tensors.ptr(), i);
    if (Py_REFCNT(o) != expected) return false;
    if (!THPVariable_Check(o) || THPVariable_Unpack(o).use_count() != 1) return false;
  }
  return true;
}

// Test aid: a C++ owner of a tensor that Python cannot see.  hold() keeps the
// tensor alive inside this module until drop() is called.
static std::vector<at::Tensor> g_held;
void hold(const at::Tensor& t) { g_held.push_back(t); }
void drop() { g_held.clear(); }

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("pair_info", &pair_info);
  m.def("data_ptrs", &data_ptrs);
  m.def("all_refcounts_equal", &all_refcounts_equal);
  m.def("hold", &hold);
  m.def("drop", &drop);
}
