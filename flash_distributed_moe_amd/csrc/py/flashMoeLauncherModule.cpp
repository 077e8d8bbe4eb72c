// The `flashMoeLauncher` Python extension: class MoeKernelLauncher over this
// library's launcher, with the surface of the reference's extension
// (python/pyMoeLauncherTorch.cpp:115-133: getDistributedUniqueId / create /
// launch / destroy / valid, same argument names and order), so the reference's
// callers (test/singleGPU/python/flashMoeOp.py:1, test_pythonBinding.py:5-40)
// import and run unchanged. Differences: bfloat16 tensors are admitted next to
// float32 (the reference checks for float32, pyMoeLauncherTorch.cpp:28-29);
// `create` reads E, H, I and the dtype off the tensors and goes through
// CreateLauncherEx, with optional top_k (default 8, the reference's compile-time
// value), router_bias, sched, flags (left out: a packed copy of the expert weights is kept, see
// create), norm_weight and norm_eps; rank / world_size other than 0 / 1 are refused. torch supplies device pointers and the current stream, nothing
// else.
#include <ATen/hip/HIPContext.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <hip/hip_runtime.h>
#include <pybind11/pybind11.h>
#include <torch/extension.h>

#include <cstring>
#include <stdexcept>
#include <string>

#include "../../../include/iMoeKernelLauncher.h"

namespace py = pybind11;

namespace {

void check_hip(hipError_t e, const char* what) {
  TORCH_CHECK(e == hipSuccess, what, " failed: ", hipGetErrorString(e), " (hipError_t ",
              static_cast<int>(e), ")");
}

void check_tensor(const at::Tensor& t, const char* name, bool any_float = true) {
  TORCH_CHECK(t.defined(), name, " tensor is undefined");
  TORCH_CHECK(t.is_cuda(), name, " must be a CUDA tensor (ROCm)");
  TORCH_CHECK(t.scalar_type() == at::kFloat || (any_float && t.scalar_type() == at::kBFloat16), name,
              any_float ? " must be float32 or bfloat16" : " must be float32");
  TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
}

// (torch on ROCm presents its HIP devices and streams under the name "cuda")
hipStream_t current_stream() { return c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream(); }
using DeviceGuard = c10::hip::HIPGuardMasqueradingAsCUDA;

class Launcher {
 public:
  static py::bytes unique_id(bool empty) {
    const moe::DistributedUniqueId id = ::GetDistributedUniqueId(empty);
    return py::bytes(reinterpret_cast<const char*>(id.data), sizeof(id.data));
  }

  void create(const at::Tensor& gate, const at::Tensor& ffn1, const at::Tensor& ffn2, int max_tokens,
              const py::bytes& uid, int rank, int world_size, int top_k,
              const c10::optional<at::Tensor>& router_bias, int sched, const py::object& flags_arg,
              const c10::optional<at::Tensor>& norm_weight, double norm_eps) {
    // flags left out, as in a call written against the reference: the launcher keeps a packed
    // copy of the expert weights (the layout the kernels read at full rate; +3*E*H*I elements
    // of device memory, announced once per process). flags=0 reads the row-major tensors.
    const int flags = flags_arg.is_none() ? static_cast<int>(FLASH_MOE_FLAG_PACK_WEIGHTS) : flags_arg.cast<int>();
    TORCH_CHECK(impl_ == nullptr, "Launcher already created");
    TORCH_CHECK(gate.defined() && ffn1.defined() && ffn2.defined(), "weight tensor is undefined");
    TORCH_CHECK(gate.dim() == 2 && ffn1.dim() == 3 && ffn2.dim() == 3,
                "weights must be [E,H], [E,2I,H], [E,H,I]");
    const auto experts = gate.size(0), hidden = gate.size(1), inter = ffn2.size(2);
    TORCH_CHECK(world_size > 0, "world_size must be positive");
    TORCH_CHECK(ffn1.size(0) == experts / world_size && ffn2.size(0) == experts / world_size,
                "expert count of the ffn weights");
    TORCH_CHECK(ffn1.size(1) == 2 * inter && ffn1.size(2) == hidden, "ffn1 must be [E, 2I, H]");
    TORCH_CHECK(ffn2.size(1) == hidden, "ffn2 must be [E, H, I]");
    check_tensor(gate, "gate_weights");
    check_tensor(ffn1, "ffn1_expert_weights");
    check_tensor(ffn2, "ffn2_expert_weights");
    TORCH_CHECK(gate.scalar_type() == ffn1.scalar_type() && gate.scalar_type() == ffn2.scalar_type(),
                "all weights must share one dtype");
    const std::string id = uid;
    TORCH_CHECK(id.size() == sizeof(moe::DistributedUniqueId::data), "uid must be 128 bytes");
    TORCH_CHECK(world_size == 1 && rank == 0,
                "only rank 0 of a world of 1 is supported (no inter-GPU transport)");
    FlashMoeLayerDesc d{};
    d.experts = static_cast<int>(experts);
    d.hidden = static_cast<int>(hidden);
    d.intermediate = static_cast<int>(inter);
    d.top_k = top_k;
    d.dtype = gate.scalar_type() == at::kBFloat16 ? FLASH_MOE_BF16 : FLASH_MOE_F32;
    d.max_tokens = max_tokens;
    d.sched = sched;
    d.flags = flags;
    d.gate_weights = gate.data_ptr();
    d.ffn1_weights = ffn1.data_ptr();
    d.ffn2_weights = ffn2.data_ptr();
    if (router_bias.has_value() && router_bias->defined()) {
      check_tensor(*router_bias, "router_bias", false);
      TORCH_CHECK(router_bias->dim() == 1 && router_bias->size(0) == experts, "router_bias must be [E]");
      d.router_bias = router_bias->data_ptr<float>();
      bias_ = *router_bias;
    }
    if (flags & FLASH_MOE_FLAG_RMSNORM) {
      TORCH_CHECK(norm_weight.has_value() && norm_weight->defined(), "FLAG_RMSNORM needs norm_weight");
      check_tensor(*norm_weight, "norm_weight");
      TORCH_CHECK(norm_weight->scalar_type() == gate.scalar_type() && norm_weight->dim() == 1 &&
                      norm_weight->size(0) == hidden,
                  "norm_weight must be [H] in the weights' dtype");
      d.norm_weight = norm_weight->data_ptr();
      d.norm_eps = norm_eps;
      norm_ = *norm_weight;
    }
    const DeviceGuard guard(gate.device());
    check_hip(CreateLauncherEx(&impl_, &d, current_stream()), "CreateLauncher");
    // the library borrows the weights: they live as long as the launcher
    gate_ = gate;
    ffn1_ = ffn1;
    ffn2_ = ffn2;
    hidden_ = hidden;
  }

  void launch(const at::Tensor& tokens, const at::Tensor& output) {
    if (impl_ == nullptr) throw std::runtime_error("Launcher was destroyed");
    check_tensor(tokens, "tokens");
    check_tensor(output, "output");
    TORCH_CHECK(tokens.scalar_type() == gate_.scalar_type() && output.scalar_type() == gate_.scalar_type(),
                "tokens and output must have the weights' dtype");
    TORCH_CHECK(tokens.dim() == 2 && tokens.size(1) == hidden_, "tokens must be [tokens, hidden]");
    TORCH_CHECK(output.sizes() == tokens.sizes(), "output shape must equal tokens shape");
    const DeviceGuard guard(gate_.device());
    check_hip(impl_->Launch(tokens.data_ptr(), output.data_ptr(), static_cast<int>(tokens.size(0)),
                            current_stream()),
              "Launch");
  }

  void destroy() {
    if (impl_ == nullptr) return;
    const DeviceGuard guard(gate_.device());
    check_hip(DestroyLauncher(impl_, current_stream()), "DestroyLauncher");
    impl_ = nullptr;
    gate_ = ffn1_ = ffn2_ = bias_ = norm_ = at::Tensor();
  }

  bool valid() const { return impl_ != nullptr; }

  // the C handle, for flashMoeReadRouting / flashMoeStatus through ctypes
  uintptr_t handle() const { return reinterpret_cast<uintptr_t>(LauncherHandle(impl_)); }

  ~Launcher() {
    // a launcher that is dropped without destroy() still gives its workspace back
    if (impl_ != nullptr) (void)DestroyLauncher(impl_, nullptr);
  }

 private:
  moe::IMoeKernelLauncher* impl_ = nullptr;
  at::Tensor gate_, ffn1_, ffn2_, bias_, norm_;
  int64_t hidden_ = 0;
};

// Rewrites ffn1 [E,2I,H] and ffn2 [E,H,I] into the packed layout where they lie (no second
// copy); create(..., flags=FLAG_WEIGHTS_PREPACKED) takes them afterwards.
void pack_weights_in_place(const at::Tensor& ffn1, const at::Tensor& ffn2) {
  check_tensor(ffn1, "ffn1_expert_weights");
  check_tensor(ffn2, "ffn2_expert_weights");
  TORCH_CHECK(ffn1.dim() == 3 && ffn2.dim() == 3 && ffn1.scalar_type() == ffn2.scalar_type(),
              "weights must be [E,2I,H] and [E,H,I] of one dtype");
  const int experts = static_cast<int>(ffn1.size(0)), hidden = static_cast<int>(ffn1.size(2)),
            inter = static_cast<int>(ffn2.size(2));
  TORCH_CHECK(ffn1.size(1) == 2 * inter && ffn2.size(0) == experts && ffn2.size(1) == hidden,
              "weights must be [E,2I,H] and [E,H,I]");
  const int dtype = ffn1.scalar_type() == at::kBFloat16 ? FLASH_MOE_BF16 : FLASH_MOE_F32;
  const DeviceGuard guard(ffn1.device());
  check_hip(static_cast<hipError_t>(flashMoePackWeightsInPlace(dtype, experts, hidden, inter, 0,
                                                               ffn1.data_ptr(), current_stream())),
            "flashMoePackWeightsInPlace");
  check_hip(static_cast<hipError_t>(flashMoePackWeightsInPlace(dtype, experts, hidden, inter, 1,
                                                               ffn2.data_ptr(), current_stream())),
            "flashMoePackWeightsInPlace");
}

}  // namespace

PYBIND11_MODULE(flashMoeLauncher, m) {
  m.doc() = "MI355X fused MoE layer launcher (drop-in for the reference's flashMoeLauncher extension)";
  m.attr("SCHED_AUTO") = static_cast<int>(FLASH_MOE_SCHED_AUTO);
  m.attr("SCHED_STREAM") = static_cast<int>(FLASH_MOE_SCHED_STREAM);
  m.attr("SCHED_TILED") = static_cast<int>(FLASH_MOE_SCHED_TILED);
  m.attr("FLAG_PACK_WEIGHTS") = static_cast<int>(FLASH_MOE_FLAG_PACK_WEIGHTS);
  m.attr("FLAG_WEIGHTS_PREPACKED") = static_cast<int>(FLASH_MOE_FLAG_WEIGHTS_PREPACKED);
  m.attr("FLAG_RMSNORM") = static_cast<int>(FLASH_MOE_FLAG_RMSNORM);
  m.attr("FLAG_RESIDUAL") = static_cast<int>(FLASH_MOE_FLAG_RESIDUAL);
  m.def("pack_weights_in_place", &pack_weights_in_place, py::arg("ffn1_expert_weights"),
        py::arg("ffn2_expert_weights"));
  py::class_<Launcher>(m, "MoeKernelLauncher")
      .def(py::init())
      .def_static("getDistributedUniqueId", &Launcher::unique_id, py::arg("empty") = false,
                  "128 zero bytes: there is no inter-GPU transport to identify.")
      .def("create", &Launcher::create, py::arg("gate_weights"), py::arg("ffn1_expert_weights"),
           py::arg("ffn2_expert_weights"), py::arg("max_tokens"), py::arg("uid"), py::arg("rank"),
           py::arg("world_size"), py::arg("top_k") = 8, py::arg("router_bias") = py::none(),
           py::arg("sched") = static_cast<int>(FLASH_MOE_SCHED_AUTO), py::arg("flags") = py::none(),
           py::arg("norm_weight") = py::none(), py::arg("norm_eps") = 1e-6)
      .def("launch", &Launcher::launch, py::arg("tokens"), py::arg("output"))
      .def("destroy", &Launcher::destroy)
      .def_property_readonly("valid", &Launcher::valid)
      .def_property_readonly("handle", &Launcher::handle);
}
