"""Shard-local compute modules: the Linear layers of a rank's shard run on the HIP kernels.

In the reference a shard is a deep copy of the user's module whose `torch.nn.Linear`s hold sliced weights and
run ATen GEMMs (src/tensor_parallel/shard.py:160,184-187; wrapper.py:69-72). Here every `nn.Linear` of a shard
is re-classed to `ShardLinear` (same parameters, same attributes, still an `nn.Linear`), and SiLU-gated MLP
blocks with `gate_proj` / `up_proj` / `down_proj` children get a fused gate/up forward. transformers' `Conv1D`
(GPT-2's c_attn / c_proj / c_fc: weight kept as [in, out] and multiplied as x @ w, sliced by
src/tensor_parallel/slicing_configs.py:192-201) is re-classed to a subclass whose forward is the same `tpamd_linear`:
its weight keeps the [in, out] shape every rule and state dict expects but is stored with the `in` axis fastest, which
is the kernel's [out, in] layout; the transposing mover writes it that way while slicing, or once at the first forward.

Inference only: the kernels have no backward; asking for one raises. Autocast is not applied by these modules: the
input must already have the weight's dtype (a mismatch raises TypeError where `nn.Linear` under autocast would cast).
"""
from __future__ import annotations

import types

import torch
from torch import nn

from . import _native
from .slicing import is_k_major


class _NoBackward(torch.autograd.Function):
    """Marks a kernel result so that a backward pass through it fails loudly instead of silently stopping."""

    @staticmethod
    def forward(ctx, out, *inputs):
        return out.view_as(out)

    @staticmethod
    def backward(ctx, *grads):
        raise NotImplementedError("tensor_parallel_amd kernels are inference-only: no backward is implemented")


def _guard(out: torch.Tensor, *inputs: torch.Tensor) -> torch.Tensor:
    if torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in inputs):
        return _NoBackward.apply(out, *inputs)
    return out


def linear_in_context(module: nn.Module, x: torch.Tensor, w: torch.Tensor, bias) -> torch.Tensor:
    """`tpamd_linear` for a shard's Linear. Inside a wrapped module whose output goes to a "sum" rule
    (collectives.SumContext) the Linear that was seen to produce that output adds the partial sums already waiting in
    the reduction, in its epilogue (`tpamd_linear_add`): the product rounded to the dtype, then one rounded add, which
    is the same arithmetic as the reduction kernel's step."""
    from .collectives import current_sum_context

    ctx = current_sum_context()
    b = None if bias is None else bias.detach()
    if ctx is None:
        return _guard(_native.linear(x.detach(), w.detach(), b), x, w, bias)
    key = id(module)
    ctx.calls[key] = ctx.calls.get(key, 0) + 1
    addend = None
    if module.__dict__.get("_tp_feeds_sum") is ctx.owner and ctx.owner is not None:
        if ctx.fused_out is not None:
            raise RuntimeError("tensor_parallel_amd: the Linear that feeds a \"sum\" rule ran twice in one call of its module "
                               "after adding the waiting partial sums; set TPAMD_FUSE_SUM=0")
        waiting = ctx.op.addend_for(ctx.rank)
        if waiting is not None:
            t, mask = waiting
            if t.dtype == x.dtype and t.device == x.device and t.shape == (*x.shape[:-1], w.shape[0]):
                addend, ctx.fused_mask = t.detach(), mask
    out = _guard(_native.linear(x.detach(), w.detach(), b, addend=addend), x, w, bias)
    if addend is not None:
        ctx.fused_out = out
    ctx.last_linear, ctx.last_out = module, out
    return out


class ShardLinear(nn.Linear):
    """`nn.Linear` whose forward is `tpamd_linear` on the shard's (sliced) weight."""

    def forward(self, input: torch.Tensor) -> torch.Tensor:  # noqa: A002
        return linear_in_context(self, input, self.weight, self.bias)


def is_conv1d(module: nn.Module) -> bool:
    """transformers.pytorch_utils.Conv1D (or a subclass): a Linear whose weight is [in, out]."""
    return any(c.__name__ == "Conv1D" and c.__module__.split(".")[0] == "transformers" for c in type(module).__mro__) and \
        isinstance(getattr(module, "weight", None), torch.Tensor)


def _conv1d_forward(self, x: torch.Tensor) -> torch.Tensor:
    w = self.weight
    if not is_k_major(w):  # a weight assigned after the shard was built: lay it out for the kernel, once
        with torch.no_grad():
            w.data = _native.transpose_regions(w.data.contiguous(), [(0, w.shape[1])]).t()
    return linear_in_context(self, x, w.t(), getattr(self, "bias", None))


_conv1d_classes: dict = {}


def _shard_conv1d_class(base: type) -> type:
    """Subclass of the module's own Conv1D class with the kernel forward (isinstance checks keep working)."""
    cls = _conv1d_classes.get(base)
    if cls is None:
        cls = _conv1d_classes[base] = type("ShardConv1D", (base,), {"forward": _conv1d_forward, "__doc__": "Conv1D whose forward is `tpamd_linear` "
                                                                   "on the shard's weight, stored with its input axis fastest."})
    return cls


def _is_silu(fn) -> bool:
    if isinstance(fn, nn.SiLU):
        return True
    name = type(fn).__name__.lower()
    return name in ("silu", "siluactivation", "swish") or fn is torch.nn.functional.silu


def _gated_mlp_forward(self, x: torch.Tensor) -> torch.Tensor:
    gate, up, down = self.gate_proj, self.up_proj, self.down_proj
    h = _native.swiglu_up(x.detach(), gate.weight.detach(), up.weight.detach())
    h = _guard(h, x, gate.weight, up.weight)
    return down(h)


def _has_hooks(module: nn.Module) -> bool:
    return bool(module._forward_hooks or module._forward_pre_hooks or getattr(module, "_forward_hooks_with_kwargs", None)
                or getattr(module, "_forward_pre_hooks_with_kwargs", None))


def is_gated_silu_mlp(module: nn.Module) -> bool:
    # only the module's own children count: a wrapper forwards attribute lookups to the module it wraps
    parts = [module._modules.get(n) for n in ("gate_proj", "up_proj", "down_proj")]
    if not all(isinstance(p, nn.Linear) for p in parts):
        return False
    gate, up, _ = parts
    if gate.bias is not None or up.bias is not None or gate.weight.dtype not in (torch.bfloat16, torch.float16):
        return False
    if gate.weight.shape != up.weight.shape:
        return False
    # the fused forward reads the two weights directly: hooks on gate_proj / up_proj would be skipped, so leave such
    # blocks to their own forward (their Linears still run on the kernels)
    if _has_hooks(gate) or _has_hooks(up) or "forward" in module.__dict__:
        return False
    act = module._modules.get("act_fn", module.__dict__.get("act_fn"))
    return _is_silu(act)


def _gated_mlp_first_forward(self, x: torch.Tensor) -> torch.Tensor:
    """First call of a block that looks like a SiLU-gated MLP: its own forward and the fused one both run on this input.
    If they agree the fused forward takes over, otherwise the block keeps its own (a forward that slices its weights
    for pretraining_tp, adds projections or orders the operations differently is not this pattern)."""
    del self.forward  # the class's forward is visible again
    own = type(self).forward(self, x)
    try:
        fused = _gated_mlp_forward(self, x)
        same = isinstance(own, torch.Tensor) and own.shape == fused.shape and torch.allclose(
            own.detach().float(), fused.detach().float(), rtol=2e-2, atol=2e-2 * float(own.detach().float().std()) + 1e-6)
    except (TypeError, ValueError, RuntimeError):
        same = False
    if same:
        self.forward = types.MethodType(_gated_mlp_forward, self)
    return own


def install_shard_kernels(shard: nn.Module) -> None:
    """Route the shard's Linear layers (and gated MLP blocks) to the HIP kernels, in place."""
    for module in shard.modules():
        if type(module) is nn.Linear:
            module.__class__ = ShardLinear
        elif is_conv1d(module) and type(module).__name__ == "Conv1D" and module.weight.dim() == 2 and module.weight.dtype in (torch.bfloat16, torch.float16, torch.float32):
            module.__class__ = _shard_conv1d_class(type(module))
    for module in shard.modules():
        if is_gated_silu_mlp(module):
            module.forward = types.MethodType(_gated_mlp_first_forward, module)
