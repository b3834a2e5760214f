// torch-facing wrapper of moe_fp8_launcher (pattern: agent_workdir/kernels/axpby_binding.cpp:17-44).
// Validation, allocation of the output and of the layer's workspace, stream lookup; no torch
// compute op is called.
#include <torch/types.h>
#include <torch/csrc/utils/pybind.h>
#include <hip/hip_runtime_api.h>
#include <c10/hip/HIPStream.h>

#include "../binding_registry.h"

extern "C" void moe_fp8_launcher(void* out, const void* x, const float* logits, const void* w13_q,
                                 const float* w13_s, const void* w2_q, const float* w2_s,
                                 void* workspace, size_t workspace_bytes, int tokens, int hidden,
                                 int inter, int n_experts, int top_k, int out_dtype, int config,
                                 hipStream_t stream);
extern "C" size_t moe_fp8_workspace_bytes(int tokens, int hidden, int inter, int n_experts, int top_k);
extern "C" int cuda_agent_amd_last_status(void);

static torch::Tensor moe_fp8_forward(torch::Tensor x, torch::Tensor logits, torch::Tensor w13_q,
                                     torch::Tensor w13_s, torch::Tensor w2_q, torch::Tensor w2_s,
                                     int top_k, int config = 0) {
    const torch::Tensor* all[] = {&x, &logits, &w13_q, &w13_s, &w2_q, &w2_s};
    const char* names[] = {"x", "logits", "w13_q", "w13_s", "w2_q", "w2_s"};
    for (int i = 0; i < 6; ++i) {
        TORCH_CHECK(all[i]->is_cuda(), names[i], " must be a GPU tensor");
        TORCH_CHECK(all[i]->is_contiguous(), names[i], " must be contiguous");
        TORCH_CHECK(all[i]->get_device() == x.get_device(), names[i], " is on another device");
    }
    TORCH_CHECK(x.dim() == 2 && logits.dim() == 2 && w13_q.dim() == 3 && w2_q.dim() == 3,
                "x [T,H], logits [T,E], w13_q [E,2I,H], w2_q [E,H,I]");
    const int64_t T = x.size(0), H = x.size(1), E = w13_q.size(0), I = w13_q.size(1) / 2;
    TORCH_CHECK(logits.size(0) == T && logits.size(1) == E, "logits must be [T, E]");
    TORCH_CHECK(w13_q.size(1) == 2 * I && w13_q.size(2) == H, "w13_q must be [E, 2I, H]");
    TORCH_CHECK(w2_q.size(0) == E && w2_q.size(1) == H && w2_q.size(2) == I, "w2_q must be [E, H, I]");
    TORCH_CHECK(H % 128 == 0 && I % 128 == 0, "hidden and inter must be multiples of 128");
    TORCH_CHECK(w13_s.dim() == 3 && w13_s.size(0) == E && w13_s.size(1) == 2 * I / 128 &&
                    w13_s.size(2) == H / 128, "w13_s must be [E, 2I/128, H/128]");
    TORCH_CHECK(w2_s.dim() == 3 && w2_s.size(0) == E && w2_s.size(1) == H / 128 &&
                    w2_s.size(2) == I / 128, "w2_s must be [E, H/128, I/128]");
    TORCH_CHECK(x.dtype() == torch::kBFloat16, "x must be bfloat16");
    TORCH_CHECK(logits.dtype() == torch::kFloat32, "logits must be float32");
    TORCH_CHECK(w13_q.dtype() == torch::kFloat8_e4m3fn && w2_q.dtype() == torch::kFloat8_e4m3fn,
                "expert weights must be float8_e4m3fn");
    TORCH_CHECK(w13_s.dtype() == torch::kFloat32 && w2_s.dtype() == torch::kFloat32,
                "block scales must be float32");
    TORCH_CHECK(E <= 512 && top_k >= 1 && top_k <= E && top_k <= 64, "n_experts <= 512, 1 <= top_k <= min(E, 64)");
    TORCH_CHECK(T * top_k <= INT32_MAX / 4, "too many (token, expert) pairs");

    auto out = torch::empty({T, H}, x.options());
    const size_t ws_bytes = moe_fp8_workspace_bytes((int)T, (int)H, (int)I, (int)E, top_k);
    auto workspace = torch::empty({(int64_t)ws_bytes}, x.options().dtype(torch::kUInt8));
    hipStream_t stream = c10::hip::getCurrentHIPStream(x.get_device()).stream();
    moe_fp8_launcher(out.data_ptr(), x.data_ptr(), logits.data_ptr<float>(), w13_q.data_ptr(),
                     w13_s.data_ptr<float>(), w2_q.data_ptr(), w2_s.data_ptr<float>(),
                     workspace.data_ptr(), ws_bytes, (int)T, (int)H, (int)I, (int)E, top_k, 0, config,
                     stream);
    const int status = cuda_agent_amd_last_status();
    TORCH_CHECK(status == 0, "moe_fp8_launcher rejected the launch, status ", status);
    return out;
}

static void register_moe_fp8(pybind11::module& m) {
    m.def("moe_fp8_forward", &moe_fp8_forward, py::arg("x"), py::arg("logits"), py::arg("w13_q"),
          py::arg("w13_s"), py::arg("w2_q"), py::arg("w2_s"), py::arg("top_k"), py::arg("config") = 0);
}

REGISTER_BINDING(moe_fp8, register_moe_fp8);
