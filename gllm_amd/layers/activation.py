import math

import torch
import torch.nn as nn

from gllm_amd import ops


class SiluAndMul(nn.Module):
    def forward(self, x):
        return ops.silu_and_mul(x)


class ReLU2(nn.Module):
    """max(z, 0)^2."""

    def forward(self, x):
        return ops.relu2(x)


class XIELU(nn.Module):
    """xIELU with two learned numbers (p, q) per layer:

        z > 0:   softplus(p) z^2 + z / 2
        z <= 0:  (1/2 + softplus(q)) (exp(z) - 1 - z) + z / 2

    ``raw`` holds (p, q) in fp32; the two coefficients are formed once
    on the host (they are launch arguments of the kernel, so a captured
    graph keeps them)."""

    def __init__(self):
        super().__init__()
        self.raw = nn.Parameter(torch.zeros(2, dtype=torch.float32),
                                requires_grad=False)
        self._coef = None

    def load(self, w: torch.Tensor):
        assert w.numel() == 2
        self.raw.data.copy_(w.reshape(2).to(torch.float32))
        self._coef = None

    @staticmethod
    def _softplus(v: float) -> float:
        return max(v, 0.0) + math.log1p(math.exp(-abs(v)))

    def coefficients(self):
        if self._coef is None:
            p, q = self.raw.detach().cpu().tolist()
            self._coef = (self._softplus(p), 0.5 + self._softplus(q))
        return self._coef

    def forward(self, x):
        a_pos, a_neg = self.coefficients()
        return ops.xielu(x, a_pos, a_neg)
