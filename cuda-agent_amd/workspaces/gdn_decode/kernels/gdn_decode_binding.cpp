// torch-facing wrapper of gdn_decode_launcher (pattern: agent_workdir/kernels/axpby_binding.cpp:17-44).
// Validation, output allocation and stream lookup only; no torch compute op is called.
#include <torch/types.h>
#include <torch/csrc/utils/pybind.h>
#include <hip/hip_runtime_api.h>
#include <c10/hip/HIPStream.h>

#include <tuple>

#include "../binding_registry.h"

extern "C" void gdn_decode_launcher(float* o, float* state, const void* q, const void* k,
                                    const void* v, const float* g, const float* beta, int batch,
                                    int n_v_heads, int n_qk_heads, int dk, int dv, int qkv_dtype,
                                    int config, hipStream_t stream);
extern "C" int cuda_agent_amd_last_status(void);

// Returns (o, state); `state` is the tensor that was passed in, updated in place.
static std::tuple<torch::Tensor, torch::Tensor> gdn_decode_forward(
    torch::Tensor q, torch::Tensor k, torch::Tensor v, torch::Tensor g, torch::Tensor beta,
    torch::Tensor state, int config = 0) {
    const torch::Tensor* all[] = {&q, &k, &v, &g, &beta, &state};
    const char* names[] = {"q", "k", "v", "g", "beta", "state"};
    for (int i = 0; i < 6; ++i) {
        TORCH_CHECK(all[i]->is_cuda(), names[i], " must be a GPU tensor");
        TORCH_CHECK(all[i]->is_contiguous(), names[i], " must be contiguous");
        TORCH_CHECK(all[i]->get_device() == state.get_device(), names[i], " is on another device");
    }
    TORCH_CHECK(state.dim() == 4, "state must be [B, Hv, dk, dv]");
    const int64_t B = state.size(0), Hv = state.size(1), dk = state.size(2), dv = state.size(3);
    TORCH_CHECK(q.dim() == 3 && q.size(0) == B && q.size(2) == dk, "q must be [B, Hqk, dk]");
    const int64_t Hqk = q.size(1);
    TORCH_CHECK(k.sizes() == q.sizes(), "k must have q's shape");
    TORCH_CHECK(v.dim() == 3 && v.size(0) == B && v.size(1) == Hv && v.size(2) == dv,
                "v must be [B, Hv, dv]");
    TORCH_CHECK(g.dim() == 2 && g.size(0) == B && g.size(1) == Hv, "g must be [B, Hv]");
    TORCH_CHECK(beta.sizes() == g.sizes(), "beta must be [B, Hv]");
    TORCH_CHECK(Hqk > 0 && Hv % Hqk == 0, "Hv must be a multiple of Hqk");
    TORCH_CHECK(dk == 128 && dv == 128, "only dk == dv == 128 is built");
    TORCH_CHECK(state.dtype() == torch::kFloat32, "state must be float32");
    TORCH_CHECK(g.dtype() == torch::kFloat32 && beta.dtype() == torch::kFloat32,
                "g and beta must be float32");
    TORCH_CHECK(q.dtype() == k.dtype() && q.dtype() == v.dtype(), "q, k, v must share a dtype");
    TORCH_CHECK(q.dtype() == torch::kFloat32 || q.dtype() == torch::kBFloat16,
                "q, k, v must be float32 or bfloat16");
    TORCH_CHECK(B * Hv * 4 <= INT32_MAX, "too many heads for one launch");

    auto o = torch::empty({B, Hv, dv}, state.options());
    hipStream_t stream = c10::hip::getCurrentHIPStream(state.get_device()).stream();
    gdn_decode_launcher(o.data_ptr<float>(), state.data_ptr<float>(), q.data_ptr(), k.data_ptr(),
                        v.data_ptr(), g.data_ptr<float>(), beta.data_ptr<float>(),
                        static_cast<int>(B), static_cast<int>(Hv), static_cast<int>(Hqk),
                        static_cast<int>(dk), static_cast<int>(dv),
                        q.dtype() == torch::kFloat32 ? 0 : 1, config, stream);
    const int status = cuda_agent_amd_last_status();
    TORCH_CHECK(status == 0, "gdn_decode_launcher rejected the launch, status ", status);
    return std::make_tuple(o, state);
}

static void register_gdn_decode(pybind11::module& m) {
    m.def("gdn_decode_forward", &gdn_decode_forward, py::arg("q"), py::arg("k"), py::arg("v"),
          py::arg("g"), py::arg("beta"), py::arg("state"), py::arg("config") = 0);
}

REGISTER_BINDING(gdn_decode, register_gdn_decode);
