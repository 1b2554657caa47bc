// PyTorch-side dispatch of the plain, the gated and the channel-major scan in C++: what the reference's pybind11 module
// (csrc/sequential_scan.cpp:13-22: scan_forward, scan_backward, scan_forward_half,
// scan_backward_half) and its two autograd Functions (sequential_scan/scan_cuda.py:13-62) do
// between `scan_cu(alpha, beta)` and the kernel launch, here between the call and the C ABI of
// libfss_scan.so.  Host code only: it allocates the outputs, looks up the stream and the chaining
// workspace, calls fss_scan_fwd_ex / fss_scan_bwd_ex (fss_gated_scan_fwd / fss_gated_scan_bwd for
// `scan_gated`, fss_scan_fwd_cm / fss_scan_bwd_cm for `scan_cm`) and records the autograd node.  A forward and
// a backward through Python Functions and ctypes cost the host 85-120 us, as much as the kernels of
// the headline shape take and several times those of short sequences.
//
// This path only takes the common case: contiguous GPU tensors of the expected type and one
// shape, on the current device, outside autocast, with a workspace of sufficient size already
// registered for the current stream.  Everything else (and every error message) stays with the
// Python wrappers: `scan` returns None and the caller goes through them, and a backward that
// meets anything unusual calls them back.
#include <torch/extension.h>

#include <ATen/TensorSubclassLikeUtils.h>
#include <ATen/autocast_mode.h>
#include <c10/hip/HIPFunctions.h>
#include <c10/hip/HIPStream.h>
#include <torch/csrc/autograd/functions/basic_ops.h>

#include <cstdint>
#include <map>
#include <mutex>
#include <optional>
#include <string>
#include <tuple>
#include <utility>

namespace {

// the C ABI (include/fss_scan.h), reached through addresses the Python side hands over, so that
// this module binds to whichever build of the library the process has loaded
using FwdFn = int (*)(int, const void *, const void *, void *, int64_t, int64_t, int64_t, void *, size_t, void *,
                      const void *);
using BwdFn = int (*)(int, const void *, const void *, const void *, void *, void *, int64_t, int64_t, int64_t,
                      void *, size_t, void *, const void *);
using GatedBwdFn = int (*)(int, const void *, const void *, const void *, const void *, void *, void *, int64_t,
                           int64_t, int64_t, void *, size_t, void *, const void *);
using StateFwdFn = int (*)(int, const void *, const void *, void *, const void *, void *, int64_t, int64_t, int64_t,
                           void *, size_t, void *, const void *);
using NeedFn = size_t (*)(int64_t, int64_t, int64_t, int, int, const void *);
using StrerrorFn = const char *(*)(int);

FwdFn g_fwd = nullptr, g_gated_fwd = nullptr, g_cm_fwd = nullptr;
BwdFn g_bwd = nullptr, g_cm_bwd = nullptr;
GatedBwdFn g_gated_bwd = nullptr;
StateFwdFn g_state_fwd = nullptr;
NeedFn g_need = nullptr, g_cm_need = nullptr;
StrerrorFn g_strerror = nullptr;
// (kind, code, saved tensors, grad_out) -> [two gradients], the Python wrappers'; never destroyed
// (the interpreter may be gone by the time statics are)
py::object *g_slow_backward = nullptr;

// kind of scan.  Plain and gated: (bs, seq, d) tensors, the `dir` values of fss_workspace_bytes for the
// two directions are 2*kind and 2*kind+1.  Channel-major: (bs, d, seq) tensors, fss_cm_workspace_bytes.
constexpr int kPlain = 0, kGated = 1, kChannelMajor = 2;
// the Python side reinitialises a workspace long before its 32-bit launch counter wraps
constexpr int64_t kLaunchLimit = (static_cast<int64_t>(1) << 31) - 16;

// A chaining workspace the Python side owns and has registered for (device, stream): its memory,
// the pinned host word a kernel sets when a chunk gave up waiting, and the launch count both
// sides add to.
struct Workspace {
  void *ptr = nullptr;
  size_t size = 0;
  const volatile uint32_t *flag = nullptr;
  int64_t *launches = nullptr;
};

std::mutex g_lock;
std::map<std::pair<int, uintptr_t>, Workspace> g_workspaces;
std::map<std::tuple<int, int, int64_t, int64_t, int64_t>, size_t> g_needs;  // (kind, code, bs, seq, d) -> bytes, both directions

at::ScalarType dtype_of(int64_t code) {
  return code == 0 ? at::kBFloat16 : code == 1 ? at::kFloat : at::kHalf;
}

size_t workspace_need(int kind, int code, int64_t bs, int64_t seq, int64_t d) {
  const auto key = std::make_tuple(kind, code, bs, seq, d);
  std::lock_guard<std::mutex> guard(g_lock);
  auto it = g_needs.find(key);
  if (it != g_needs.end()) return it->second;
  // (bs, seq, d) are the tensor's three sizes in order: (bs, d, seq) for the channel-major kind
  const size_t fwd = kind == kChannelMajor ? g_cm_need(bs, seq, d, code, 0, nullptr) : g_need(bs, seq, d, code, 2 * kind, nullptr);
  const size_t bwd = kind == kChannelMajor ? g_cm_need(bs, seq, d, code, 1, nullptr) : g_need(bs, seq, d, code, 2 * kind + 1, nullptr);
  if (g_needs.size() > 4096) g_needs.clear();
  const size_t need = fwd > bwd ? fwd : bwd;
  g_needs[key] = need;
  return need;
}

// The registered workspace of (device, stream) if it can take this launch now.
bool usable_workspace(int device, void *stream, size_t need, Workspace &out) {
  std::lock_guard<std::mutex> guard(g_lock);
  auto it = g_workspaces.find({device, reinterpret_cast<uintptr_t>(stream)});
  if (it == g_workspaces.end()) return false;
  const Workspace &ws = it->second;
  if (ws.size < need || *ws.flag != 0 || *ws.launches >= kLaunchLimit) return false;
  ++*ws.launches;
  out = ws;
  return true;
}

bool plain_tensor(const at::Tensor &t, at::ScalarType dtype) {
  return t.defined() && t.is_cuda() && t.scalar_type() == dtype && t.dim() == 3 && t.is_contiguous() &&
         t.layout() == at::kStrided && !at::isTensorSubclassLike(t);
}

[[noreturn]] void raise_status(int rc) {
  throw std::runtime_error("fss_scan status " + std::to_string(rc) + ": " + (g_strerror ? g_strerror(rc) : "?"));
}

// (called with everything checked)
at::Tensor launch_forward(int kind, const at::Tensor &alpha, const at::Tensor &beta, int code, const Workspace &ws,
                          void *stream) {
  at::Tensor h = at::empty_like(alpha);
  const int rc = (kind == kGated ? g_gated_fwd : kind == kChannelMajor ? g_cm_fwd : g_fwd)(code, alpha.data_ptr(), beta.data_ptr(), h.data_ptr(),
                                                        alpha.size(0), alpha.size(1), alpha.size(2), ws.ptr, ws.size,
                                                        stream, nullptr);
  if (rc != 0) raise_status(rc);
  return h;
}

struct ScanNode : public torch::autograd::Function<ScanNode> {
  // (alpha, beta) of the plain scan or (gate, x) of the gated one
  static at::Tensor forward(torch::autograd::AutogradContext *ctx, const at::Tensor &alpha, const at::Tensor &beta,
                            int64_t code, int64_t kind, int64_t ws_ptr, int64_t ws_size, int64_t stream) {
    Workspace ws;
    ws.ptr = reinterpret_cast<void *>(ws_ptr);
    ws.size = static_cast<size_t>(ws_size);
    at::Tensor h = launch_forward(static_cast<int>(kind), alpha, beta, static_cast<int>(code), ws,
                                  reinterpret_cast<void *>(stream));
    // (alpha, h): the output itself, no extra activation memory (reference scan_cuda.py:20,42);
    // the gated backward also needs x
    if (kind == kGated)
      ctx->save_for_backward({alpha, beta, h});
    else
      ctx->save_for_backward({alpha, h});
    ctx->saved_data["code"] = code;
    ctx->saved_data["kind"] = kind;
    return h;
  }

  static torch::autograd::variable_list backward(torch::autograd::AutogradContext *ctx,
                                                 torch::autograd::variable_list grads) {
    const auto saved = ctx->get_saved_variables();
    const int code = static_cast<int>(ctx->saved_data["code"].toInt());
    const int kind = static_cast<int>(ctx->saved_data["kind"].toInt());
    const at::Tensor &alpha = saved[0], &h = saved.back();
    at::Tensor dout = grads[0];
    at::Tensor grad_alpha, grad_beta;
    bool done = false;
    const at::ScalarType dtype = dtype_of(code);
    bool plain = dout.defined() && dout.is_cuda() && dout.scalar_type() == dtype && dout.sizes() == alpha.sizes() &&
                 dout.device() == alpha.device() && dout.layout() == at::kStrided && !at::isTensorSubclassLike(dout) &&
                 alpha.device().index() == c10::hip::current_device();
    for (const auto &t : saved) plain = plain && plain_tensor(t, dtype);
    if (plain) {
      const int device = alpha.device().index();
      void *stream = c10::hip::getCurrentHIPStream(static_cast<c10::DeviceIndex>(device)).stream();
      Workspace ws;
      if (usable_workspace(device, stream, workspace_need(kind, code, alpha.size(0), alpha.size(1), alpha.size(2)), ws)) {
        if (!dout.is_contiguous()) dout = dout.contiguous();
        grad_alpha = at::empty_like(alpha);
        grad_beta = at::empty_like(alpha);
        const int rc =
            kind == kGated
                ? g_gated_bwd(code, alpha.data_ptr(), saved[1].data_ptr(), h.data_ptr(), dout.data_ptr(),
                              grad_alpha.data_ptr(), grad_beta.data_ptr(), alpha.size(0), alpha.size(1), alpha.size(2),
                              ws.ptr, ws.size, stream, nullptr)
                : (kind == kChannelMajor ? g_cm_bwd : g_bwd)(code, alpha.data_ptr(), h.data_ptr(), dout.data_ptr(),
                                                             grad_alpha.data_ptr(), grad_beta.data_ptr(), alpha.size(0),
                                                             alpha.size(1), alpha.size(2), ws.ptr, ws.size, stream, nullptr);
        if (rc != 0) raise_status(rc);
        done = true;
      }
    }
    if (!done) {
      py::gil_scoped_acquire gil;
      TORCH_CHECK(g_slow_backward != nullptr, "fss_torch_binding.init was not called");
      py::object result = (*g_slow_backward)(kind, code, std::vector<at::Tensor>(saved.begin(), saved.end()), dout);
      auto pair = result.cast<std::vector<at::Tensor>>();
      TORCH_CHECK(pair.size() == 2, "the Python backward returned ", pair.size(), " tensors");
      grad_alpha = pair[0];
      grad_beta = pair[1];
    }
    torch::autograd::variable_list out = {grad_alpha, grad_beta};
    if (at::GradMode::is_enabled() && grads[0].defined() && grads[0].requires_grad()) {
      // backward(create_graph=True) with a gradient that is itself differentiable: as
      // torch.autograd.function.once_differentiable, the results come back behind a node that
      // raises when anything differentiates through them
      for (auto &t : out) {
        t = t.detach();
        t.set_requires_grad(true);
      }
      auto err = std::make_shared<torch::autograd::DelayedError>(
          "trying to differentiate twice a function that was marked with @once_differentiable", 2);
      out = (*err)(std::move(out));
    }
    out.resize(7);  // nothing for code, kind, workspace and stream
    return out;
  }
};

void init(uintptr_t fwd, uintptr_t bwd, uintptr_t gated_fwd, uintptr_t gated_bwd, uintptr_t state_fwd, uintptr_t cm_fwd,
          uintptr_t cm_bwd, uintptr_t need, uintptr_t cm_need, uintptr_t strerror_fn, py::object slow_backward) {
  std::lock_guard<std::mutex> guard(g_lock);
  g_fwd = reinterpret_cast<FwdFn>(fwd);
  g_bwd = reinterpret_cast<BwdFn>(bwd);
  g_gated_fwd = reinterpret_cast<FwdFn>(gated_fwd);
  g_gated_bwd = reinterpret_cast<GatedBwdFn>(gated_bwd);
  g_state_fwd = reinterpret_cast<StateFwdFn>(state_fwd);
  g_cm_fwd = reinterpret_cast<FwdFn>(cm_fwd);
  g_cm_bwd = reinterpret_cast<BwdFn>(cm_bwd);
  g_need = reinterpret_cast<NeedFn>(need);
  g_cm_need = reinterpret_cast<NeedFn>(cm_need);
  g_strerror = reinterpret_cast<StrerrorFn>(strerror_fn);
  g_slow_backward = new py::object(std::move(slow_backward));
  g_needs.clear();
}

void register_workspace(int device, uintptr_t stream, uintptr_t ptr, size_t size, uintptr_t flag, uintptr_t launches) {
  std::lock_guard<std::mutex> guard(g_lock);
  Workspace ws;
  ws.ptr = reinterpret_cast<void *>(ptr);
  ws.size = size;
  ws.flag = reinterpret_cast<const volatile uint32_t *>(flag);
  ws.launches = reinterpret_cast<int64_t *>(launches);
  g_workspaces[{device, stream}] = ws;
}

void forget_workspaces() {
  std::lock_guard<std::mutex> guard(g_lock);
  g_workspaces.clear();
}

// h of the scan, recorded for autograd when an input asks for it; None when this path does not
// cover the call.  `code`: 0 bf16, 1 fp32, 2 fp16 (FSS_BF16, FSS_F32, FSS_F16); `kind`: 0 the plain
// scan of (alpha, beta), 1 the gated scan of (gate, x).
std::optional<at::Tensor> dispatch(const at::Tensor &alpha, const at::Tensor &beta, int64_t code, int kind) {
  if (!g_fwd || code < 0 || code > 2) return std::nullopt;
  const at::ScalarType dtype = dtype_of(code);
  if (!plain_tensor(alpha, dtype) || !plain_tensor(beta, dtype)) return std::nullopt;
  if (alpha.sizes() != beta.sizes() || alpha.device() != beta.device() || alpha.numel() == 0) return std::nullopt;
  if (at::autocast::is_autocast_enabled(at::kCUDA)) return std::nullopt;
  const int device = alpha.device().index();
  if (device != c10::hip::current_device()) return std::nullopt;
  void *stream = c10::hip::getCurrentHIPStream(static_cast<c10::DeviceIndex>(device)).stream();
  Workspace ws;
  if (!usable_workspace(device, stream,
                        workspace_need(kind, static_cast<int>(code), alpha.size(0), alpha.size(1), alpha.size(2)), ws))
    return std::nullopt;
  if (at::GradMode::is_enabled() && (alpha.requires_grad() || beta.requires_grad()))
    return ScanNode::apply(alpha, beta, code, static_cast<int64_t>(kind),
                           static_cast<int64_t>(reinterpret_cast<uintptr_t>(ws.ptr)), static_cast<int64_t>(ws.size),
                           static_cast<int64_t>(reinterpret_cast<uintptr_t>(stream)));
  return launch_forward(kind, alpha, beta, static_cast<int>(code), ws, stream);
}

std::optional<at::Tensor> scan(const at::Tensor &alpha, const at::Tensor &beta, int64_t code) {
  return dispatch(alpha, beta, code, kPlain);
}

// (the storage type is the gate's: bf16, fp32 or fp16)
std::optional<at::Tensor> scan_gated(const at::Tensor &gate, const at::Tensor &x) {
  if (!gate.defined()) return std::nullopt;
  const at::ScalarType t = gate.scalar_type();
  const int64_t code = t == at::kBFloat16 ? 0 : t == at::kFloat ? 1 : t == at::kHalf ? 2 : -1;
  return dispatch(gate, x, code, kGated);
}

// (bs, d_model, seq) tensors, time contiguous; the storage type is alpha's
std::optional<at::Tensor> scan_cm(const at::Tensor &alpha, const at::Tensor &beta) {
  if (!alpha.defined()) return std::nullopt;
  const at::ScalarType t = alpha.scalar_type();
  const int64_t code = t == at::kBFloat16 ? 0 : t == at::kFloat ? 1 : t == at::kHalf ? 2 : -1;
  return dispatch(alpha, beta, code, kChannelMajor);
}

// (h, h_last) of the scan that starts from the fp32 state `h_before` (bs, d) - zeros when absent -
// for calls that need no gradient: the step of a streaming decode loop, where the sequence is a
// few tokens and the host's time is all there is.  None for anything else.
std::optional<std::tuple<at::Tensor, at::Tensor>> scan_state(const at::Tensor &alpha, const at::Tensor &beta,
                                                             const std::optional<at::Tensor> &h_before) {
  if (!g_state_fwd || !alpha.defined()) return std::nullopt;
  const at::ScalarType t = alpha.scalar_type();
  const int code = t == at::kBFloat16 ? 0 : t == at::kFloat ? 1 : t == at::kHalf ? 2 : -1;
  if (code < 0 || !plain_tensor(alpha, t) || !plain_tensor(beta, t)) return std::nullopt;
  if (alpha.sizes() != beta.sizes() || alpha.device() != beta.device() || alpha.numel() == 0) return std::nullopt;
  const bool with_state = h_before.has_value() && h_before->defined();
  if (with_state) {
    const at::Tensor &h0 = *h_before;
    if (!h0.is_cuda() || h0.scalar_type() != at::kFloat || h0.dim() != 2 || h0.size(0) != alpha.size(0) ||
        h0.size(1) != alpha.size(2) || !h0.is_contiguous() || h0.device() != alpha.device() ||
        at::isTensorSubclassLike(h0))
      return std::nullopt;
  }
  if (at::GradMode::is_enabled() &&
      (alpha.requires_grad() || beta.requires_grad() || (with_state && h_before->requires_grad())))
    return std::nullopt;
  if (at::autocast::is_autocast_enabled(at::kCUDA)) return std::nullopt;
  const int device = alpha.device().index();
  if (device != c10::hip::current_device()) return std::nullopt;
  void *stream = c10::hip::getCurrentHIPStream(static_cast<c10::DeviceIndex>(device)).stream();
  Workspace ws;
  if (!usable_workspace(device, stream, workspace_need(kPlain, code, alpha.size(0), alpha.size(1), alpha.size(2)), ws))
    return std::nullopt;
  at::Tensor h = at::empty_like(alpha);
  // (every channel's entry is written by the wave that holds the sequence's last step)
  at::Tensor h_last = at::empty({alpha.size(0), alpha.size(2)}, alpha.options().dtype(at::kFloat));
  const int rc = g_state_fwd(code, alpha.data_ptr(), beta.data_ptr(), h.data_ptr(),
                             with_state ? h_before->data_ptr() : nullptr, h_last.data_ptr(), alpha.size(0),
                             alpha.size(1), alpha.size(2), ws.ptr, ws.size, stream, nullptr);
  if (rc != 0) raise_status(rc);
  return std::make_tuple(h, h_last);
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.doc() = "C++ dispatch of the plain scan over the C ABI of libfss_scan.so";
  m.def("init", &init,
        "addresses of fss_scan_fwd_ex, fss_scan_bwd_ex, fss_gated_scan_fwd, fss_gated_scan_bwd, fss_scan_fwd_state, "
        "fss_scan_fwd_cm, fss_scan_bwd_cm, fss_workspace_bytes, fss_cm_workspace_bytes, fss_strerror; the Python backward");
  m.def("register_workspace", &register_workspace, "device, stream, pointer, bytes, address of the flag word, address of the launch count");
  m.def("forget_workspaces", &forget_workspaces);
  m.def("scan", &scan, "h, or None when the call is not the common case");
  m.def("scan_gated", &scan_gated, "h of the gated scan, or None when the call is not the common case");
  m.def("scan_cm", &scan_cm, "h of the channel-major scan, or None when the call is not the common case");
  m.def("scan_state", &scan_state, py::arg("alpha"), py::arg("beta"), py::arg("h_before") = py::none(),
        "(h, h_last) without gradients, or None when the call is not the common case");
}
