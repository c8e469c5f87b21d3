"""int8 weight-only shard Linears with outlier columns kept in 16 bits, from the Python layer.

The reference has no int8 code of its own: its users quantise the wrapped model with a third-party library before or
after `tp.tensor_parallel` (README of the reference, LLM.int8 notebooks). This module is that step for the shards of this
package: `quantize_linears_` turns the 16-bit Linears of a module tree (the rank shards of a `tp.TensorParallel`, or any
module on a HIP device) into `ShardLinearW8`, whose forward is `tpamd_linear_w8`. The definition is closed form:

  O        = the outlier input columns of a Linear (chosen by the caller, sorted)
  scale[n] = max over k not in O of |W[n,k]| / 127            (1.0 where that max is 0)
  Wq[n,k]  = clamp(round_half_even(W[n,k] / scale[n]), -127, 127) for k not in O, 0 for k in O
  y        = x . (Wq * scale[:,None])^T  +  x[:, O] . W[:, O]^T  (+ bias)

The quantiser runs on the device with torch's elementwise ops (it runs once per weight); the Linear itself runs on the
library's kernels only. A quantised Linear no longer has a `weight`: `save_tensor_parallel`, which rebuilds the full
weights of the original model from the shards, refuses a model that holds one; its shards can be saved as they are.
"""
from __future__ import annotations

from typing import Callable, Mapping, Optional, Sequence, Tuple, Union

import torch
from torch import nn

from . import _native
from . import shard_modules
from .shard_modules import _guard, is_conv1d

OutlierChoice = Union[None, Mapping[str, Sequence[int]], Callable[[str, nn.Module], Optional[Sequence[int]]]]


def quantize_rows(w: torch.Tensor, outlier_cols: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """w [N, K] (bfloat16 / float16 / float32, on a HIP device) -> (wq int8 [N, K], scale float32 [N],
    outlier_idx int32 [n_out] sorted, w_out [N, n_out] in w's dtype) by the definition in the module docstring."""
    _native.require_device(w, "quantize_rows")
    if w.dim() != 2:
        raise ValueError(f"quantize_rows: expected a [N, K] weight, got {tuple(w.shape)}")
    N, K = w.shape
    if outlier_cols is None:
        cols = torch.empty(0, dtype=torch.int64, device=w.device)
    else:
        cols = torch.as_tensor(outlier_cols, dtype=torch.int64, device=w.device).flatten()
        if cols.numel() and (int(cols.min()) < 0 or int(cols.max()) >= K):
            raise ValueError(f"quantize_rows: outlier columns must lie in [0, {K})")
        cols = torch.unique(cols)  # sorted, no repeats
    keep = torch.ones(K, dtype=torch.bool, device=w.device)
    keep[cols] = False
    q = torch.empty((N, K), dtype=torch.int8, device=w.device)
    scale = torch.empty(N, dtype=torch.float32, device=w.device)
    # The definition's two divisions are float32 divisions rounded correctly. The device's float32 division is allowed an
    # error of a unit in the last place, which would move a quotient across a rounding boundary now and then: they are
    # done in float64 and rounded to float32 instead, which gives the correctly rounded float32 quotient. Blocks of rows
    # bound the temporaries.
    for r0 in range(0, N, 4096):
        wd = w.detach()[r0:r0 + 4096].double()
        absmax = wd.abs().masked_fill(~keep, 0.0).amax(dim=1) if K else wd.new_zeros(wd.shape[0])
        sc = (absmax / 127.0).float()
        sc = torch.where(sc == 0, torch.ones_like(sc), sc)
        quot = (wd / sc.double()[:, None]).float()
        q[r0:r0 + 4096] = torch.round(quot).clamp_(-127, 127).to(torch.int8)  # torch.round: ties to even
        scale[r0:r0 + 4096] = sc
    q[:, ~keep] = 0
    return q, scale, cols.to(torch.int32), w.detach()[:, cols].contiguous()


class ShardLinearW8(nn.Module):
    """A Linear whose weight is stored as int8 rows with one float32 scale each, plus the outlier input columns in the
    activation dtype; the forward is `tpamd_linear_w8`. Inference only."""

    def __init__(self, wq: torch.Tensor, scale: torch.Tensor, outlier_idx: torch.Tensor, w_out: torch.Tensor,
                 bias: Optional[torch.Tensor], dtype: torch.dtype):
        super().__init__()
        if dtype not in (torch.bfloat16, torch.float16):
            raise TypeError(f"ShardLinearW8: activations must be bfloat16 or float16, got {dtype}")
        self.out_features, self.in_features = wq.shape
        self.dtype = dtype
        self.register_buffer("wq", wq.contiguous())
        self.register_buffer("scale", scale.contiguous())
        self.register_buffer("outlier_idx", outlier_idx.to(torch.int32).contiguous())
        self.register_buffer("w_out", w_out.to(dtype).contiguous())
        self.register_buffer("bias", None if bias is None else bias.detach().to(dtype).contiguous())

    @classmethod
    def from_weight(cls, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
                    outlier_cols: Optional[Sequence[int]] = None) -> "ShardLinearW8":
        """Quantise a [out, in] weight that lives on a HIP device."""
        if weight.dtype not in (torch.bfloat16, torch.float16):
            raise TypeError(f"ShardLinearW8: the weight must be bfloat16 or float16, got {weight.dtype}")
        wq, scale, idx, w_out = quantize_rows(weight, None if outlier_cols is None else torch.as_tensor(outlier_cols))
        return cls(wq, scale, idx, w_out, bias, weight.dtype)

    def forward(self, input: torch.Tensor) -> torch.Tensor:  # noqa: A002
        if input.dtype != self.dtype:
            raise TypeError(f"ShardLinearW8: the input is {input.dtype}, the Linear was quantised for {self.dtype}")
        n_out = self.outlier_idx.numel()
        out = _native.linear_w8(input.detach(), self.wq, self.scale, self.outlier_idx if n_out else None,
                                self.w_out if n_out else None, self.bias)
        return _guard(out, input)

    def extra_repr(self) -> str:
        return (f"in_features={self.in_features}, out_features={self.out_features}, bias={self.bias is not None}, "
                f"outlier_columns={self.outlier_idx.numel()}, dtype={self.dtype}")


def _outliers_of(choice: OutlierChoice, name: str, module: nn.Module) -> Optional[Sequence[int]]:
    if choice is None:
        return None
    if callable(choice):
        return choice(name, module)
    return choice.get(name)


def quantize_linears_(module: nn.Module, outlier_cols: OutlierChoice = None,
                      skip: Callable[[str, nn.Module], bool] = lambda name, m: False) -> int:
    """Replace, in place, every 16-bit `nn.Linear` (and transformers `Conv1D`) under `module` whose weight lives on a HIP
    device by a `ShardLinearW8`. `outlier_cols`: the outlier input columns per Linear, as a mapping from the Linear's name
    under `module` (as in `module.named_modules()`) or as a function of (name, Linear); none by default. `skip(name,
    Linear)` keeps a Linear as it is (an output head, say). Returns how many were replaced."""
    replaced = 0
    for parent_name, parent in list(module.named_modules()):
        for child_name, child in list(parent.named_children()):
            name = f"{parent_name}.{child_name}" if parent_name else child_name
            conv1d = is_conv1d(child)
            if not (isinstance(child, nn.Linear) or conv1d) or isinstance(child, ShardLinearW8):
                continue
            w = child.weight
            if w.device.type != "cuda" or w.dtype not in (torch.bfloat16, torch.float16) or skip(name, child):
                continue
            weight = w.detach().t() if conv1d else w.detach()  # Conv1D keeps [in, out]
            new = ShardLinearW8.from_weight(weight, getattr(child, "bias", None), _outliers_of(outlier_cols, name, child))
            setattr(parent, child_name, new)
            replaced += 1
            # a SiLU-gated MLP block whose fused forward reads gate_proj.weight / up_proj.weight goes back to its own forward
            fused = parent.__dict__.get("forward")
            if getattr(fused, "__func__", None) in (shard_modules._gated_mlp_forward, shard_modules._gated_mlp_first_forward):
                del parent.forward
    return replaced
