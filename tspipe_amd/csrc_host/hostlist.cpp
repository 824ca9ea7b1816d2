// Host-side helper for the Python adapters: walks Python lists of tensors at
// C++ speed.  A parameter list has 150+ tensors and the per-tensor Python work
// (data_ptr, numel, dtype/device/shape/contiguity checks) costs more than the
// EMA kernel itself; here it is one call.  No GPU work happens in this module.
#include <torch/extension.h>
#include <torch/csrc/autograd/python_variable.h>
#include <ATen/detail/CUDAHooksInterface.h>

#include <algorithm>
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

// ---------------------------------------------------------------------------
// InfoNCE as a C++ autograd node.  The arithmetic stays in libtspipe_amd.so:
// this node only owns the buffers and calls the C ABI through the function
// addresses the Python side hands over (bind_abi), on the stream the forward
// was called on.  What it saves over the Python autograd.Function is host
// time: the backward runs on autograd's device thread without taking the
// interpreter lock, which is most of what a step of the loss costs the host.
// ---------------------------------------------------------------------------
typedef size_t (*nce_ws_fn)(int64_t, int64_t, int);
typedef int (*nce_fn)(const void*, const void*, const void*, const void*, int64_t, int64_t, float, void*, float*,
                      void*, void*, int, void*);
typedef int (*scale_fn)(void*, int64_t, int64_t, int64_t, const float*, int, void*);
static nce_ws_fn g_nce_ws = nullptr;
static nce_fn g_nce = nullptr;
static scale_fn g_scale = nullptr;

void bind_abi(uintptr_t nce_ws, uintptr_t nce, uintptr_t scale) {
  g_nce_ws = reinterpret_cast<nce_ws_fn>(nce_ws);
  g_nce = reinterpret_cast<nce_fn>(nce);
  g_scale = reinterpret_cast<scale_fn>(scale);
}

inline int dtype_code(at::ScalarType t) {
  return t == at::kFloat ? 0 : t == at::kBFloat16 ? 1 : t == at::kHalf ? 2 : -1;
}

struct InfoNCENode : public torch::autograd::Function<InfoNCENode> {
  static at::Tensor forward(torch::autograd::AutogradContext* ctx, const at::Tensor& q1, const at::Tensor& k1,
                            const c10::optional<at::Tensor>& q2o, const c10::optional<at::Tensor>& k2o, double tau,
                            int64_t stream) {
    const bool two = q2o.has_value();
    const at::Tensor q2 = two ? *q2o : at::Tensor(), k2 = two ? *k2o : at::Tensor();
    const int64_t n = q1.size(0), c = q1.size(1);
    const int code = dtype_code(q1.scalar_type());
    c10::DeviceGuard guard(q1.device());
    const auto bytes = (int64_t)g_nce_ws(n, c, two ? 2 : 1);
    at::Tensor ws = at::empty({bytes}, q1.options().dtype(at::kByte));
    at::Tensor loss = at::empty({}, q1.options().dtype(at::kFloat));
    at::Tensor g1, g2;
    if (q1.requires_grad()) g1 = at::empty_like(q1);
    if (two && q2.requires_grad()) g2 = at::empty_like(q2);
    const int rc = g_nce(q1.data_ptr(), k1.data_ptr(), two ? q2.data_ptr() : nullptr, two ? k2.data_ptr() : nullptr, n,
                         c, (float)tau, ws.data_ptr(), loss.data_ptr<float>(), g1.defined() ? g1.data_ptr() : nullptr,
                         g2.defined() ? g2.data_ptr() : nullptr, code, reinterpret_cast<void*>(stream));
    TORCH_CHECK(rc == 0, "ts_infonce_fwd_bwd: status ", rc);
    ctx->saved_data["g1"] = g1;
    ctx->saved_data["g2"] = g2;
    ctx->saved_data["stream"] = stream;
    ctx->saved_data["done"] = false;
    return loss;
  }

  static torch::autograd::variable_list backward(torch::autograd::AutogradContext* ctx,
                                                 torch::autograd::variable_list grad_out) {
    TORCH_CHECK(!ctx->saved_data["done"].toBool(),
                "the fused loss keeps one gradient buffer: backward can run once per forward");
    ctx->saved_data["done"] = true;
    // the context lets go of the buffers, so that autograd can adopt them as .grad instead of copying
    at::Tensor g1 = ctx->saved_data["g1"].toTensor(), g2 = ctx->saved_data["g2"].toTensor();
    ctx->saved_data["g1"] = at::Tensor();
    ctx->saved_data["g2"] = at::Tensor();
    void* stream = reinterpret_cast<void*>(ctx->saved_data["stream"].toInt());
    at::Tensor go = grad_out[0];
    if (go.scalar_type() != at::kFloat) go = go.to(at::kFloat);
    for (at::Tensor* g : {&g1, &g2}) {
      if (!g->defined()) continue;
      // grad *= grad_output on the device; the kernel returns at once when it is 1
      const int rc = g_scale(g->data_ptr(), g->size(0), g->size(1), g->size(1), go.data_ptr<float>(),
                             dtype_code(g->scalar_type()), stream);
      TORCH_CHECK(rc == 0, "ts_scale_rows: status ", rc);
    }
    return {g1, at::Tensor(), g2, at::Tensor(), at::Tensor(), at::Tensor()};
  }
};

// Returns None when the call is not of the plain kind (then the Python
// autograd.Function takes it and raises the proper errors): 2-D dense device
// tensors of one shape and dtype, 64 / 128 / 256 features.
py::object infonce(const at::Tensor& q1, const at::Tensor& k1, const c10::optional<at::Tensor>& q2,
                   const c10::optional<at::Tensor>& k2, double tau, int64_t stream) {
  if (!g_nce || !g_nce_ws || !g_scale) return py::none();
  const bool two = q2.has_value();
  if (two != k2.has_value()) return py::none();
  const at::Tensor* all[4] = {&q1, &k1, two ? &*q2 : nullptr, two ? &*k2 : nullptr};
  for (const at::Tensor* t : all) {
    if (!t) continue;
    if (!t->is_cuda() || t->dim() != 2 || !t->is_contiguous() || t->sizes() != q1.sizes() ||
        t->scalar_type() != q1.scalar_type() || t->device() != q1.device())
      return py::none();
  }
  const int64_t c = q1.size(1);
  if ((c != 64 && c != 128 && c != 256) || dtype_code(q1.scalar_type()) < 0 || !(tau >= 0.03)) return py::none();
  if (k1.requires_grad() || (two && k2->requires_grad())) return py::none();
  // without gradient mode nothing is recorded, so no gradient buffer is wanted either
  const bool record = at::GradMode::is_enabled();
  c10::optional<at::Tensor> s2 = q2;
  if (!record && two) s2 = q2->detach();
  at::Tensor loss;
  {
    // allocations and launches need no interpreter: other Python threads (a pipeline's momentum
    // update beside this loss) run meanwhile
    py::gil_scoped_release no_gil;
    loss = InfoNCENode::apply(record ? q1 : q1.detach(), k1, s2, k2, tau, stream);
  }
  return py::cast(loss);
}

// ---------------------------------------------------------------------------
// DeferredBatchNorm's training forward as a C++ autograd node, for the same
// reason: on the feature maps of a network's late stages the kernels take
// 10-30 us and a Python autograd.Function around them 100.  The layer's
// state that changes with every launch -- which half of the reduction
// workspace the next call uses, and the stream that used the workspace last --
// lives in a two-element int64 host tensor shared with the Python module
// (state[0] = parity, state[1] = stream handle), so that Python-side calls of
// the same layer (evaluation mode, the stand-alone statistics) stay in step.
// ---------------------------------------------------------------------------
typedef int (*bn_fwd_fn)(const float*, float*, const float*, const float*, int64_t, int64_t, int64_t, float*, float*,
                         float*, float*, float*, int, float, void*);
typedef int (*bn_bwd_fn)(const float*, const float*, const float*, const float*, const float*, float*, float*, float*,
                         float*, int, int64_t, int64_t, int64_t, int, void*);
static bn_fwd_fn g_bn_fwd = nullptr;
static bn_bwd_fn g_bn_bwd = nullptr;

void bind_bn(uintptr_t fwd, uintptr_t bwd) {
  g_bn_fwd = reinterpret_cast<bn_fwd_fn>(fwd);
  g_bn_bwd = reinterpret_cast<bn_bwd_fn>(bwd);
}

struct BnTrainNode : public torch::autograd::Function<BnTrainNode> {
  static at::Tensor forward(torch::autograd::AutogradContext* ctx, const at::Tensor& x,
                            const c10::optional<at::Tensor>& weight, const c10::optional<at::Tensor>& bias,
                            const at::Tensor& sum, const at::Tensor& sum_squares, const at::Tensor& ws,
                            const at::Tensor& state, double eps, int64_t stream) {
    const int64_t N = x.size(0), C = x.size(1), HW = (N * C) ? x.numel() / (N * C) : 0;
    c10::DeviceGuard guard(x.device());
    at::Tensor y = at::empty_like(x);
    at::Tensor stats = at::empty({2, C}, x.options());  // micro-batch mean, inverse standard deviation
    int64_t* st = state.data_ptr<int64_t>();
    const int parity = (int)st[0];
    const bool has_w = weight.has_value() && weight->defined(), has_b = bias.has_value() && bias->defined();
    const int rc = g_bn_fwd(x.data_ptr<float>(), y.data_ptr<float>(), has_w ? weight->data_ptr<float>() : nullptr,
                            has_b ? bias->data_ptr<float>() : nullptr, N, C, HW, sum.data_ptr<float>(),
                            sum_squares.data_ptr<float>(), stats.data_ptr<float>(), stats.data_ptr<float>() + C,
                            ws.data_ptr<float>() + 3 * C, parity, (float)eps, reinterpret_cast<void*>(stream));
    TORCH_CHECK(rc == 0, "ts_bn_forward_train: status ", rc);
    st[0] = 1 - parity;
    st[1] = stream;
    ctx->save_for_backward({x, stats, has_w ? *weight : at::Tensor()});
    ctx->saved_data["ws"] = ws;
    ctx->saved_data["state"] = state;
    ctx->saved_data["stream"] = stream;
    ctx->saved_data["has_w"] = has_w;
    ctx->saved_data["has_b"] = has_b;
    return y;
  }

  static torch::autograd::variable_list backward(torch::autograd::AutogradContext* ctx,
                                                 torch::autograd::variable_list grad_out) {
    const auto saved = ctx->get_saved_variables();
    const at::Tensor& x = saved[0];
    const at::Tensor& stats = saved[1];
    const at::Tensor& weight = saved[2];
    const bool has_w = ctx->saved_data["has_w"].toBool(), has_b = ctx->saved_data["has_b"].toBool();
    const int64_t stream = ctx->saved_data["stream"].toInt();
    at::Tensor ws = ctx->saved_data["ws"].toTensor(), state = ctx->saved_data["state"].toTensor();
    const int64_t N = x.size(0), C = x.size(1), HW = (N * C) ? x.numel() / (N * C) : 0;
    c10::DeviceGuard guard(x.device());
    at::Tensor dy = grad_out[0].contiguous();
    if (dy.scalar_type() != at::kFloat) dy = dy.to(at::kFloat);
    at::Tensor dx = at::empty_like(x);
    at::Tensor dgb = at::empty({2, C}, x.options());
    int64_t* st = state.data_ptr<int64_t>();
    if (st[1] != 0 && st[1] != stream) {
      // the layer's last call ran on another stream: its use of the workspace must be over first
      // (rare; the Python side orders the two streams with an event instead of this wait)
      at::detail::getCUDAHooks().deviceSynchronize(x.device().index());
    }
    const int parity = (int)st[0];
    const int rc = g_bn_bwd(x.data_ptr<float>(), dy.data_ptr<float>(), stats.data_ptr<float>(),
                            stats.data_ptr<float>() + C, weight.defined() ? weight.data_ptr<float>() : nullptr,
                            dx.data_ptr<float>(), dgb.data_ptr<float>(), dgb.data_ptr<float>() + C,
                            ws.data_ptr<float>() + 3 * C, parity, N, C, HW, 1, reinterpret_cast<void*>(stream));
    TORCH_CHECK(rc == 0, "ts_bn_backward: status ", rc);
    st[0] = 1 - parity;
    st[1] = stream;
    return {dx, has_w ? dgb[0] : at::Tensor(), has_b ? dgb[1] : at::Tensor(), at::Tensor(), at::Tensor(),
            at::Tensor(), at::Tensor(), at::Tensor(), at::Tensor()};
  }
};

// Returns None when the call is not of the plain kind (then the Python path
// takes it): contiguous fp32 device tensors, state on the host.
py::object bn_train(const at::Tensor& x, const c10::optional<at::Tensor>& weight,
                    const c10::optional<at::Tensor>& bias, const at::Tensor& sum, const at::Tensor& sum_squares,
                    const at::Tensor& ws, const at::Tensor& state, double eps, int64_t stream) {
  if (!g_bn_fwd || !g_bn_bwd) return py::none();
  if (!x.is_cuda() || x.scalar_type() != at::kFloat || !x.is_contiguous() || x.dim() < 3) return py::none();
  if (state.is_cuda() || state.scalar_type() != at::kLong || state.numel() != 2 || !state.is_contiguous())
    return py::none();
  const int64_t C = x.size(1);
  if (ws.numel() != 7 * C || ws.scalar_type() != at::kFloat || ws.device() != x.device()) return py::none();
  at::Tensor y;
  {
    py::gil_scoped_release no_gil;
    y = BnTrainNode::apply(x, weight, bias, sum, sum_squares, ws, state, eps, stream);
  }
  return py::cast(y);
}

// ---------------------------------------------------------------------------
// The row losses (KD with its cross-entropy and squared-error riders, squared
// error alone, cosine, BYOL) as one C++ autograd node, for the same reason as
// the two above: at the batch sizes of the CIFAR-sized benchmarks the kernels
// take 7-12 us and a Python autograd.Function around them 50-300.  Each kind
// is the same call sequence as its Python Function, on the same C entry
// points, so both give the same bits.
// ---------------------------------------------------------------------------
typedef size_t (*kd_ws_fn)(int64_t, int64_t, int);
typedef int (*kdce_fn)(const void*, const void*, const uint8_t*, const int64_t*, int64_t, int64_t, int64_t, int64_t,
                       int64_t, float, float, float, void*, float*, void*, int64_t, int, void*);
typedef size_t (*mse_ws_fn)(int64_t, int64_t);
typedef int (*mse_fn)(const void*, const void*, const uint8_t*, int64_t, int64_t, int64_t, int64_t, float, int, int,
                      void*, float*, void*, int64_t, int, void*);
typedef size_t (*cos_ws_fn)(int64_t);
typedef int (*cos_fn)(const void*, const void*, const uint8_t*, int64_t, int64_t, float, void*, float*, void*, int,
                      void*);
typedef int (*byol_fn)(const void*, const void*, const void*, const void*, int64_t, int64_t, float*, float*, void*,
                       void*, int, void*);
static kd_ws_fn g_kd_ws = nullptr;
static kdce_fn g_kdce = nullptr;
static mse_ws_fn g_mse_ws = nullptr;
static mse_fn g_mse = nullptr;
static cos_ws_fn g_cos_ws = nullptr;
static cos_fn g_cos = nullptr;
static byol_fn g_byol = nullptr;

void bind_losses(uintptr_t kd_ws, uintptr_t kdce, uintptr_t mse_ws, uintptr_t mse, uintptr_t cos_ws, uintptr_t cos,
                 uintptr_t byol) {
  g_kd_ws = reinterpret_cast<kd_ws_fn>(kd_ws);
  g_kdce = reinterpret_cast<kdce_fn>(kdce);
  g_mse_ws = reinterpret_cast<mse_ws_fn>(mse_ws);
  g_mse = reinterpret_cast<mse_fn>(mse);
  g_cos_ws = reinterpret_cast<cos_ws_fn>(cos_ws);
  g_cos = reinterpret_cast<cos_fn>(cos);
  g_byol = reinterpret_cast<byol_fn>(byol);
}

enum LossKind : int64_t { kLossKd = 0, kLossMse = 1, kLossCosine = 2, kLossByol = 3 };

struct RowLossNode : public torch::autograd::Function<RowLossNode> {
  // x1 (and x2, BYOL's second student) may require gradients; y1, y2, mask and labels never do.
  // f: kind-specific numbers (see row_loss below); n: kind-specific integers.
  static at::Tensor forward(torch::autograd::AutogradContext* ctx, const at::Tensor& x1, const at::Tensor& y1,
                            const c10::optional<at::Tensor>& x2o, const c10::optional<at::Tensor>& y2o,
                            const c10::optional<at::Tensor>& mask, const c10::optional<at::Tensor>& labels,
                            int64_t kind, std::vector<double> f, std::vector<int64_t> n, int64_t stream) {
    const int64_t V = x1.size(-1), rows = V ? x1.numel() / V : 0;
    const int code = dtype_code(x1.scalar_type());
    c10::DeviceGuard guard(x1.device());
    void* st = reinterpret_cast<void*>(stream);
    const uint8_t* mask_ptr = mask.has_value() ? static_cast<const uint8_t*>(mask->data_ptr()) : nullptr;
    at::Tensor loss = at::empty({}, x1.options().dtype(at::kFloat));
    at::Tensor g1, g2, ws;
    if (x1.requires_grad()) g1 = at::empty_like(x1);
    auto bytes = [&](size_t b) { return at::empty({(int64_t)b}, x1.options().dtype(at::kByte)); };
    int rc = 0;
    const char* what = "";
    switch (kind) {
      case kLossKd: {
        // f = {T, weight, ce_weight, mse_weight}; n = {ignore_index, mse_per_element}
        const double T = f[0];
        ws = bytes(g_kd_ws(rows, V, code));
        what = "ts_kdce_fwd_bwd";
        rc = g_kdce(x1.data_ptr(), y1.data_ptr(), mask_ptr,
                    labels.has_value() ? labels->data_ptr<int64_t>() : nullptr, n[0], rows, V, V, V, (float)(1.0 / T),
                    (float)(T * T * f[1]), (float)f[2], ws.data_ptr(), loss.data_ptr<float>(),
                    g1.defined() ? g1.data_ptr() : nullptr, V, code, st);
        if (rc == 0 && f[3] > 0.0) {
          at::Tensor ws2 = bytes(g_mse_ws(rows, V));
          what = "ts_mse_fwd_bwd";
          rc = g_mse(x1.data_ptr(), y1.data_ptr(), mask_ptr, rows, V, V, V, (float)f[3], (int)n[1], 1, ws2.data_ptr(),
                     loss.data_ptr<float>(), g1.defined() ? g1.data_ptr() : nullptr, V, code, st);
        }
        break;
      }
      case kLossMse:
        // f = {weight}; n = {per_element}
        ws = bytes(g_mse_ws(rows, V));
        what = "ts_mse_fwd_bwd";
        rc = g_mse(x1.data_ptr(), y1.data_ptr(), mask_ptr, rows, V, V, V, (float)f[0], (int)n[0], 0, ws.data_ptr(),
                   loss.data_ptr<float>(), g1.defined() ? g1.data_ptr() : nullptr, V, code, st);
        break;
      case kLossCosine:
        // f = {weight}
        ws = bytes(g_cos_ws(rows));
        what = "ts_cosine_fwd_bwd";
        rc = g_cos(x1.data_ptr(), y1.data_ptr(), mask_ptr, rows, V, (float)f[0], ws.data_ptr(), loss.data_ptr<float>(),
                   g1.defined() ? g1.data_ptr() : nullptr, code, st);
        break;
      default: {
        const bool two = x2o.has_value();
        if (two && x2o->requires_grad()) g2 = at::empty_like(*x2o);
        ws = at::empty({2 * std::max<int64_t>(rows, 1)}, x1.options().dtype(at::kFloat));
        what = "ts_byol_fwd_bwd";
        rc = g_byol(x1.data_ptr(), y1.data_ptr(), two ? x2o->data_ptr() : nullptr, two ? y2o->data_ptr() : nullptr,
                    rows, V, ws.data_ptr<float>(), loss.data_ptr<float>(), g1.defined() ? g1.data_ptr() : nullptr,
                    g2.defined() ? g2.data_ptr() : nullptr, code, st);
      }
    }
    TORCH_CHECK(rc == 0, what, ": status ", rc);
    ctx->saved_data["g1"] = g1;
    ctx->saved_data["g2"] = g2;
    ctx->saved_data["stream"] = stream;
    ctx->saved_data["done"] = false;
    return loss;
  }

  static torch::autograd::variable_list backward(torch::autograd::AutogradContext* ctx,
                                                 torch::autograd::variable_list grad_out) {
    TORCH_CHECK(!ctx->saved_data["done"].toBool(),
                "the fused loss keeps one gradient buffer: backward can run once per forward");
    ctx->saved_data["done"] = true;
    // the context lets go of the buffers, so that autograd can adopt them as .grad instead of copying
    at::Tensor g1 = ctx->saved_data["g1"].toTensor(), g2 = ctx->saved_data["g2"].toTensor();
    ctx->saved_data["g1"] = at::Tensor();
    ctx->saved_data["g2"] = at::Tensor();
    void* stream = reinterpret_cast<void*>(ctx->saved_data["stream"].toInt());
    at::Tensor go = grad_out[0];
    if (go.scalar_type() != at::kFloat) go = go.to(at::kFloat);
    for (at::Tensor* g : {&g1, &g2}) {
      if (!g->defined() || g->numel() == 0) continue;
      const int64_t V = g->size(-1);
      const int rc = g_scale(g->data_ptr(), g->numel() / V, V, V, go.data_ptr<float>(), dtype_code(g->scalar_type()),
                             stream);
      TORCH_CHECK(rc == 0, "ts_scale_rows: status ", rc);
    }
    return {g1,           at::Tensor(), g2,           at::Tensor(), at::Tensor(),
            at::Tensor(), at::Tensor(), at::Tensor(), at::Tensor(), at::Tensor()};
  }
};

// kind 0 (KD): f = {T, weight, ce_weight, mse_weight}, n = {ignore_index, mse_per_element};
// kind 1 (squared error): f = {weight}, n = {per_element}; kind 2 (cosine): f = {weight};
// kind 3 (BYOL): x2 / y2 the second pair or None.
// Returns None when the call is not of the plain kind, and the Python autograd.Function takes it
// (and raises the proper errors): dense device tensors of one shape and floating dtype with at
// least one row, teachers without gradients, a bool / uint8 mask with one entry per row, int64 labels.
py::object row_loss(int64_t kind, const at::Tensor& x1, const at::Tensor& y1, const c10::optional<at::Tensor>& x2,
                    const c10::optional<at::Tensor>& y2, const c10::optional<at::Tensor>& mask,
                    const c10::optional<at::Tensor>& labels, std::vector<double> f, std::vector<int64_t> n,
                    int64_t stream) {
  if (!g_kdce || !g_mse || !g_cos || !g_byol || !g_scale) return py::none();
  if (kind < kLossKd || kind > kLossByol) return py::none();
  if (f.size() < (kind == kLossKd ? 4u : kind == kLossByol ? 0u : 1u)) return py::none();
  if (n.size() < (kind == kLossKd ? 2u : kind == kLossMse ? 1u : 0u)) return py::none();
  if (x2.has_value() != y2.has_value() || (x2.has_value() && kind != kLossByol)) return py::none();
  if (x1.dim() < 1 || (kind == kLossByol && x1.dim() != 2) || x1.numel() == 0) return py::none();
  if (dtype_code(x1.scalar_type()) < 0) return py::none();
  const at::Tensor* all[4] = {&x1, &y1, x2.has_value() ? &*x2 : nullptr, y2.has_value() ? &*y2 : nullptr};
  for (const at::Tensor* t : all) {
    if (!t) continue;
    if (!t->is_cuda() || !t->is_contiguous() || t->sizes() != x1.sizes() || t->scalar_type() != x1.scalar_type() ||
        t->device() != x1.device())
      return py::none();
  }
  if (y1.requires_grad() || (y2.has_value() && y2->requires_grad())) return py::none();
  const int64_t rows = x1.numel() / x1.size(-1);
  if (mask.has_value()) {
    if (kind == kLossByol) return py::none();
    const at::Tensor& m = *mask;
    // (masks of other types mean "not zero" and are converted by the Python path)
    if (!m.is_cuda() || m.device() != x1.device() || !m.is_contiguous() || m.numel() != rows ||
        m.scalar_type() != at::kBool)
      return py::none();
  }
  if (labels.has_value()) {
    const at::Tensor& l = *labels;
    if (kind != kLossKd || !l.is_cuda() || l.device() != x1.device() || !l.is_contiguous() || l.numel() != rows ||
        l.scalar_type() != at::kLong)
      return py::none();
  }
  if (kind == kLossKd && !(f[0] > 0.0)) return py::none();
  // without gradient mode nothing is recorded, so no gradient buffer is wanted either
  const bool record = at::GradMode::is_enabled();
  c10::optional<at::Tensor> s2 = x2;
  if (!record && x2.has_value()) s2 = x2->detach();
  at::Tensor loss;
  {
    py::gil_scoped_release no_gil;
    loss = RowLossNode::apply(record ? x1 : x1.detach(), y1, s2, y2, mask, labels, kind, f, n, stream);
  }
  return py::cast(loss);
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
  m.def("bind_abi", &bind_abi);
  m.def("infonce", &infonce);
  m.def("bind_bn", &bind_bn);
  m.def("bind_losses", &bind_losses);
  m.def("row_loss", &row_loss);
  m.def("bn_train", &bn_train);
  m.def("hold", &hold);
  m.def("drop", &drop);
}
