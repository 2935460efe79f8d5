"""The toy model behind the committed packed-checkpoint fixtures: one plain linear, one norm and two QuantLinear
layers (with and without bias).  tests/golden/make_checkpoint_fixture.py built it from the reference's QuantLinear
when it wrote the fixtures; the tests build the same model from this repository's QuantLinear."""
import torch
import torch.nn as nn

QPARAMS = {"w": {"bit": 4, "sym": True}, "act": {"bit": 4, "sym": True}}


def build_toy(quant_linear_cls, seed: int = 0) -> nn.Module:
    torch.manual_seed(seed)

    class Toy(nn.Module):
        def __init__(self):
            super().__init__()
            self.pre = nn.Linear(8, 64)
            self.norm = nn.LayerNorm(64)
            self.q1 = quant_linear_cls(nn.Linear(64, 128, bias=True), {"w": "lsq", "act": "dynamic"}, QPARAMS)
            self.q2 = quant_linear_cls(nn.Linear(128, 128, bias=False), {"w": "lsq", "act": "dynamic"}, QPARAMS)

        def forward(self, x):
            return self.q2(self.q1(self.norm(self.pre(x))))

    return Toy()
