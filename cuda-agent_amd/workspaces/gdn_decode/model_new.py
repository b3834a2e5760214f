# Extension side of the pair (agent_workdir/model_new.py:6-13): same constructor as Model,
# forward is one call into the compiled gfx950 kernel. Returns the tuple (o, state) with
# `state` updated in place, like Model.
import torch
import torch.nn as nn
import cuda_extension


class ModelNew(nn.Module):

    def __init__(self, n_v_heads: int, n_qk_heads: int, dk: int, dv: int) -> None:
        super().__init__()
        self.n_v_heads = n_v_heads
        self.n_qk_heads = n_qk_heads
        self.dk = dk
        self.dv = dv

    def forward(self, q, k, v, g, beta, state):
        return cuda_extension.gdn_decode_forward(q, k, v, g, beta, state, 0)
