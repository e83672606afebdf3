"""GPT-2 style Conv1D with ``skip_bias_add`` (reference:
``oslo/torch/nn/modules/conv.py:5-42``): a linear layer with transposed weight
``[nx, nf]``; with ``skip_bias_add=True`` it returns ``(x @ W, bias)``."""
import torch
import torch.nn as nn


class Conv1D(nn.Module):
    def __init__(self, nf, nx, skip_bias_add=False):
        super().__init__()
        self.nf = nf
        self.skip_bias_add = skip_bias_add
        self.weight = nn.Parameter(nn.init.normal_(torch.empty(nx, nf), std=0.02))
        self.bias = nn.Parameter(torch.zeros(nf))

    def forward(self, x):
        flat = x.reshape(-1, x.size(-1))
        size_out = x.size()[:-1] + (self.nf,)
        if self.skip_bias_add:
            return torch.mm(flat, self.weight).view(size_out), self.bias
        return torch.addmm(self.bias, flat, self.weight).view(size_out)
