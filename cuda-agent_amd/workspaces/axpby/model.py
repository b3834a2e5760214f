# Task definition of the smoke workspace: the eager reference for out = alpha * a + b.
# Same operator, shapes and constructor argument as the reference workspace's example task
# (agent_workdir/model.py:9-26). This file is the fixed side of the pair; model_new.py is the
# side that calls the compiled extension.
import torch
import torch.nn as nn


class Model(nn.Module):

    def __init__(self, alpha: float) -> None:
        super().__init__()
        self.alpha = alpha

    def forward(self, a, b):
        return self.alpha * a + b


def get_inputs():
    return [torch.randn(1, 128), torch.randn(1, 128)]


def get_init_inputs():
    return [2.0]
