"""A stand-in for peft 0.3's LoRA Linear, for tests: peft is not installed here. The class sits in a module named
`peft.tuners.lora` and is called `Linear`, which is what the LoRA detection looks at, and has peft 0.3's layout:
`lora_A` / `lora_B` are ModuleDicts of bias-free Linears keyed by adapter name, added to the base Linear's output."""
import sys
import types
from contextlib import contextmanager

import torch.nn.functional as F
from torch import nn


class Linear(nn.Linear):
    def __init__(self, in_features, out_features, r=4, lora_alpha=8, bias=True):
        super().__init__(in_features, out_features, bias=bias)
        self.lora_A = nn.ModuleDict({"default": nn.Linear(in_features, r, bias=False)})
        self.lora_B = nn.ModuleDict({"default": nn.Linear(r, out_features, bias=False)})
        self.scaling = lora_alpha / r

    def forward(self, x):
        return F.linear(x, self.weight, self.bias) + self.lora_B["default"](self.lora_A["default"](x)) * self.scaling


Linear.__module__ = "peft.tuners.lora"


@contextmanager
def installed(version="0.3.0"):
    """Makes `peft` (with `__version__`) and `peft.tuners.lora` importable for the duration."""
    saved = {k: sys.modules.get(k) for k in ("peft", "peft.tuners", "peft.tuners.lora")}
    peft, tuners, lora = types.ModuleType("peft"), types.ModuleType("peft.tuners"), types.ModuleType("peft.tuners.lora")
    peft.__version__, peft.tuners, tuners.lora, lora.Linear = version, tuners, lora, Linear
    sys.modules.update({"peft": peft, "peft.tuners": tuners, "peft.tuners.lora": lora})
    try:
        yield lora
    finally:
        for k, v in saved.items():
            if v is None:
                sys.modules.pop(k, None)
            else:
                sys.modules[k] = v
