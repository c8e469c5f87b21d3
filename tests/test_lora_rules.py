"""LoRA rules (reference: src/tensor_parallel/config.py:128-154, utils.py:131-144) on a stand-in for peft's LoRA Linear.
parity unpinned against real peft: it is not installed; what is checked is the rule set the reference's code would
derive for peft 0.3's module layout, derived here by hand."""
import pytest
import torch
from torch import nn

import tensor_parallel_amd as tp
from tensor_parallel_amd.config import add_lora_rules
from tensor_parallel_amd.state_actions import Scale, Split
from tensor_parallel_amd.utils import check_lora, verify_peft_version

import lora_standin


class Block(nn.Module):
    def __init__(self, lora=True):
        super().__init__()
        make = lora_standin.Linear if lora else nn.Linear
        self.up = make(16, 32)
        self.down = make(32, 16)
        self.plain = nn.Linear(16, 16)

    def forward(self, x):
        return self.plain(self.down(torch.relu(self.up(x))))


def rules(world=2):
    return tp.Config(
        state_rules={r".*up\.(weight|bias)$": Split(world, 0), r".*down\.weight$": Split(world, 1), r".*down\.bias$": Scale(world)},
        input_rules={}, output_rules={r".*down$": {0: "sum"}}, attr_rules={})


def test_detection():
    with lora_standin.installed():
        assert check_lora(lora_standin.Linear(4, 4)) and not check_lora(nn.Linear(4, 4))
    with lora_standin.installed(version="0.2.0"), pytest.raises(ImportError, match="peft>=0.3.0"):
        check_lora(lora_standin.Linear(4, 4))
    with pytest.raises(ImportError):  # no peft at all, yet a module claims to come from it
        verify_peft_version()


def test_rules_for_both_orientations():
    with lora_standin.installed():
        cfg = add_lora_rules(Block(), rules())
    state = {p.pattern: a for p, a in cfg.state_rules.items()}
    inputs = {p.pattern: a for p, a in cfg.input_rules.items()}
    outputs = {p.pattern: a for p, a in cfg.output_rules.items()}
    # column-parallel base: lora_B's weight is split like the base weight, lora_A is left whole
    lora_b = next(p for p in cfg.state_rules if "lora_B" in p.pattern)
    assert state[lora_b.pattern] is state[r".*up\.(weight|bias)$"]
    assert lora_b.search("up.lora_B.default.weight") and not lora_b.search("up.lora_A.default.weight") and not lora_b.search("xup.lora_B.default.weight")
    # row-parallel base: lora_A sees the gathered input and its output is divided by the world size
    lora_a = next(p for p in cfg.input_rules if "lora_A" in p.pattern)
    assert inputs[lora_a.pattern] == {0: "gather -1"} and outputs[lora_a.pattern] == {0: "scale"}
    assert lora_a.search("down.lora_A.default") and not lora_a.search("down.lora_A") and not lora_a.search("up.lora_A.default")
    assert sum("lora" in p for p in state) == 1 and sum("lora" in p for p in inputs) == 1


def test_no_lora_no_change_and_unsupported_actions_raise():
    cfg = rules()
    before = (dict(cfg.state_rules), dict(cfg.input_rules), dict(cfg.output_rules))
    assert add_lora_rules(Block(lora=False), cfg) is cfg
    assert (dict(cfg.state_rules), dict(cfg.input_rules), dict(cfg.output_rules)) == before
    bad = tp.Config({r".*up\.weight$": Scale(2)}, {}, {}, {})
    with lora_standin.installed(), pytest.raises(Exception, match="LoRA"):
        add_lora_rules(Block(), bad)
    bad_dim = tp.Config({r".*up\.weight$": Split(2, 2)}, {}, {}, {})
    with lora_standin.installed(), pytest.raises(Exception, match="Expected dim in"):
        add_lora_rules(Block(), bad_dim)
