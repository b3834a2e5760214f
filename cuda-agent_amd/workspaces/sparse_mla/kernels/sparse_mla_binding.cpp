// torch-facing wrapper of sparse_mla_decode_launcher (pattern:
// agent_workdir/kernels/axpby_binding.cpp:17-44). Validation, allocation of the output and of
// the split workspace, stream lookup; no torch compute op is called.
#include <torch/types.h>
#include <torch/csrc/utils/pybind.h>
#include <hip/hip_runtime_api.h>
#include <c10/hip/HIPStream.h>

#include "../binding_registry.h"

extern "C" void sparse_mla_decode_launcher(void* out, const void* q, const void* kv, const int* idx,
                                           void* workspace, size_t workspace_bytes, int batch,
                                           int n_heads, int n_kv_rows, int topk, int d_qk, int d_v,
                                           float sm_scale, int out_dtype, int config,
                                           hipStream_t stream);
extern "C" size_t sparse_mla_decode_workspace_bytes(int batch, int n_heads, int topk, int config);
extern "C" int cuda_agent_amd_last_status(void);

static torch::Tensor sparse_mla_forward(torch::Tensor q, torch::Tensor kv, torch::Tensor idx,
                                        double sm_scale, int config = 0) {
    const torch::Tensor* all[] = {&q, &kv, &idx};
    const char* names[] = {"q", "kv", "idx"};
    for (int i = 0; i < 3; ++i) {
        TORCH_CHECK(all[i]->is_cuda(), names[i], " must be a GPU tensor");
        TORCH_CHECK(all[i]->is_contiguous(), names[i], " must be contiguous");
        TORCH_CHECK(all[i]->get_device() == q.get_device(), names[i], " is on another device");
    }
    TORCH_CHECK(q.dim() == 3 && kv.dim() == 3 && idx.dim() == 2, "q [B,H,576], kv [B,N,576], idx [B,topk]");
    const int64_t B = q.size(0), H = q.size(1), D = q.size(2), N = kv.size(1), topk = idx.size(1);
    TORCH_CHECK(kv.size(0) == B && idx.size(0) == B, "batch sizes differ");
    TORCH_CHECK(D == 576 && kv.size(2) == 576, "only 576-dim latent rows (512 + 64) are built");
    TORCH_CHECK(H == 32 || H == 64 || H % 128 == 0, "heads must be 32, 64 or a multiple of 128");
    TORCH_CHECK(q.dtype() == torch::kBFloat16 && kv.dtype() == torch::kBFloat16, "q, kv must be bfloat16");
    TORCH_CHECK(idx.dtype() == torch::kInt32, "idx must be int32");
    TORCH_CHECK(topk >= 1 && N >= 1 && N <= INT32_MAX && topk <= INT32_MAX && B <= 65535, "size out of range");

    auto out = torch::empty({B, H, 512}, q.options());
    const size_t ws_bytes = sparse_mla_decode_workspace_bytes((int)B, (int)H, (int)topk, config);
    auto workspace = torch::empty({(int64_t)ws_bytes}, q.options().dtype(torch::kUInt8));
    hipStream_t stream = c10::hip::getCurrentHIPStream(q.get_device()).stream();
    sparse_mla_decode_launcher(out.data_ptr(), q.data_ptr(), kv.data_ptr(), idx.data_ptr<int>(),
                               workspace.data_ptr(), ws_bytes, (int)B, (int)H, (int)N, (int)topk, 576,
                               512, static_cast<float>(sm_scale), 0, config, stream);
    const int status = cuda_agent_amd_last_status();
    TORCH_CHECK(status == 0, "sparse_mla_decode_launcher rejected the launch, status ", status);
    return out;
}

static void register_sparse_mla(pybind11::module& m) {
    m.def("sparse_mla_forward", &sparse_mla_forward, py::arg("q"), py::arg("kv"), py::arg("idx"),
          py::arg("sm_scale"), py::arg("config") = 0);
}

REGISTER_BINDING(sparse_mla, register_sparse_mla);
