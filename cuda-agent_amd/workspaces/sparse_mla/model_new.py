# Extension side of the pair (agent_workdir/model_new.py:6-13): same constructor as Model,
# forward is one call into the compiled gfx950 kernels (split kernel + merge).
import torch
import torch.nn as nn
import cuda_extension


class ModelNew(nn.Module):

    def __init__(self, n_heads: int, d_qk: int, d_v: int) -> None:
        super().__init__()
        self.n_heads = n_heads
        self.d_qk = d_qk
        self.d_v = d_v
        self.sm_scale = 192 ** -0.5

    def forward(self, q, kv, idx):
        return cuda_extension.sparse_mla_forward(q, kv, idx, self.sm_scale, 0)
