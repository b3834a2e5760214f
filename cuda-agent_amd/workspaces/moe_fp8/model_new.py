# Extension side of the pair (agent_workdir/model_new.py:6-13): same constructor and buffers as
# Model (filled by load_state_dict, so they are only allocated here), forward is one call into
# the compiled gfx950 kernels (route, sort, quantise, grouped e4m3 GEMMs, combine).
import torch
import torch.nn as nn
import cuda_extension

GROUP = 128


class ModelNew(nn.Module):

    def __init__(self, hidden: int, inter: int, n_experts: int, top_k: int) -> None:
        super().__init__()
        self.hidden, self.inter, self.n_experts, self.top_k = hidden, inter, n_experts, top_k
        self.register_buffer('w13_q', torch.empty(n_experts, 2 * inter, hidden, dtype=torch.float8_e4m3fn))
        self.register_buffer('w13_s', torch.empty(n_experts, 2 * inter // GROUP, hidden // GROUP))
        self.register_buffer('w2_q', torch.empty(n_experts, hidden, inter, dtype=torch.float8_e4m3fn))
        self.register_buffer('w2_s', torch.empty(n_experts, hidden // GROUP, inter // GROUP))

    def forward(self, x, logits):
        return cuda_extension.moe_fp8_forward(x, logits, self.w13_q, self.w13_s, self.w2_q, self.w2_s,
                                              self.top_k, 0)
