"""A block with LoRA Linears (stand-in for peft 0.3's layout, peft is not installed) run as rank shards: the rules
that `add_lora_rules` derives must reproduce the unsplit block (reference: src/tensor_parallel/config.py:128-154)."""
from copy import deepcopy

import pytest
import torch

import tensor_parallel_amd as tp

import lora_standin
from test_lora_rules import Block, rules

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


@pytest.mark.parametrize("world", [2, 3])
def test_lora_block_as_rank_shards(world):
    torch.manual_seed(0)
    block = Block().eval()
    with torch.no_grad():
        for p in block.parameters():
            p.normal_(0.0, 0.3)
    x = torch.randn(5, 16, generator=torch.Generator().manual_seed(1))
    with torch.no_grad():
        ref = block(x)
    with lora_standin.installed():
        model_tp = tp.TensorParallel(deepcopy(block), [DEV] * world, tensor_parallel_config=rules(world), sharded=False)
    shard = model_tp.module_shards[0]
    up, down = shard.up, shard.down.tp_wrapped_module
    assert up.lora_B["default"].weight.shape[0] == up.weight.shape[0] < 32 and up.lora_A["default"].weight.shape == (4, 16)
    assert down.weight.shape[1] < 32 and down.lora_A["default"].tp_wrapped_module.weight.shape == (4, 32)
    with torch.no_grad():
        out = model_tp(x.to(DEV))
    torch.testing.assert_close(out.cpu(), ref, rtol=1e-5, atol=1e-5 * ref.abs().max().item())
