"""The int8 step of the Python layer (tensor_parallel_amd.int8): the device quantiser against the closed-form definition
in oracle/quant.py bit for bit, the module against the definition evaluated in float64, and a tensor-parallel model whose
shard Linears were quantised. The reference has no int8 path: parity is against the definition."""
import math

import numpy as np
import pytest
import torch
from torch import nn

import tensor_parallel_amd as tp
from oracle import quant as oq
from tensor_parallel_amd.int8 import ShardLinearW8, quantize_linears_, quantize_rows

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)
RTOL = 2e-2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("N,K,n_out", [(64, 256, 0), (48, 512, 3), (130, 1000, 41), (5, 16, 8)])
def test_device_quantiser_equals_the_definition_bit_for_bit(dtype, N, K, n_out):
    g = torch.Generator().manual_seed(N + K)
    w = (torch.randn(N, K, generator=g) * 0.02).to(dtype)
    w[1] = 0          # a row of zeros gets scale 1
    w[2, 5] = 0.75    # one large entry sets its row's scale, unless its column is an outlier
    cols = torch.randperm(K, generator=g)[:n_out]
    wq, scale, idx, w_out = quantize_rows(w.to(DEV), cols)
    want_q, want_scale, want_out = oq.quantize_rows(w.float().numpy(), np.sort(cols.numpy()))
    assert wq.dtype == torch.int8 and scale.dtype == torch.float32 and idx.dtype == torch.int32 and w_out.dtype == dtype
    assert np.array_equal(idx.cpu().numpy(), np.sort(cols.numpy()))
    assert np.array_equal(wq.cpu().numpy(), want_q)
    assert np.array_equal(scale.cpu().numpy().view(np.uint32), want_scale.view(np.uint32))
    assert np.array_equal(w_out.float().cpu().numpy(), want_out)
    assert float(scale[1]) == 1.0


def test_quantiser_arguments():
    w = torch.randn(8, 32, dtype=torch.float16)
    with pytest.raises(tp._native.NativeLibraryError):
        quantize_rows(w)  # host tensors are refused: nothing here computes on the CPU
    with pytest.raises(ValueError, match="outlier columns"):
        quantize_rows(w.to(DEV), torch.tensor([32]))
    with pytest.raises(TypeError):
        ShardLinearW8.from_weight(torch.randn(8, 32, device=DEV))  # float32 weights stay as they are


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,N,K,n_out,bias", [(1, 64, 256, 0, False), (7, 96, 512, 9, True), (40, 256, 1024, 41, True)])
def test_module_matches_the_definition(dtype, M, N, K, n_out, bias):
    g = torch.Generator().manual_seed(3)
    lin = nn.Linear(K, N, bias=bias)
    with torch.no_grad():
        lin.weight.copy_(torch.randn(N, K, generator=g) * 0.02)
    lin = lin.to(dtype).to(DEV)
    cols = torch.randperm(K, generator=g)[:n_out]
    x = torch.randn(M, K, generator=g)
    x[:, cols] *= 20
    x = x.to(dtype)
    mod = ShardLinearW8.from_weight(lin.weight, lin.bias, cols.tolist())
    got = mod(x.to(DEV))
    wq, scale, w_out = oq.quantize_rows(lin.weight.detach().float().cpu().numpy(), np.sort(cols.numpy()))
    want = oq.linear_w8_f64(x.float().numpy(), wq, scale, np.sort(cols.numpy()), w_out)
    if bias:
        want = want + lin.bias.detach().double().cpu().numpy()
    sigma = 0.02 * math.sqrt(K + 400 * n_out)
    torch.testing.assert_close(got.double().cpu(), torch.from_numpy(want), rtol=RTOL, atol=RTOL * sigma)
    with pytest.raises(TypeError, match="quantised for"):
        mod(x.to(DEV).float())
    with torch.enable_grad(), pytest.raises(NotImplementedError):
        mod(x.to(DEV).requires_grad_()).sum().backward()


def _tiny_llama():
    import transformers as tf

    torch.manual_seed(0)
    cfg = tf.LlamaConfig(vocab_size=300, hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
                         num_key_value_heads=2, max_position_embeddings=128)
    return tf.LlamaForCausalLM(cfg).to(torch.bfloat16).eval()


def test_quantised_shards_of_a_tensor_parallel_llama():
    """Every Linear of both rank shards but the output head becomes int8 (the gated MLP blocks go back to their own
    forward, which calls the three quantised Linears); the logits stay within int8 error of the 16-bit shards' logits."""
    model = _tiny_llama()
    ids = torch.randint(0, 300, (2, 24), generator=torch.Generator().manual_seed(1))
    with torch.no_grad():
        tp_model = tp.tensor_parallel(model, [DEV, DEV])
        before = tp_model(input_ids=ids.to(DEV)).logits.float().cpu()
        n = quantize_linears_(tp_model, skip=lambda name, m: name.endswith("lm_head") or "lm_head" in name)
        assert n == 2 * 2 * 7  # ranks x layers x (q, k, v, o, gate, up, down)
        assert sum(isinstance(m, ShardLinearW8) for m in tp_model.modules()) == n
        after = tp_model(input_ids=ids.to(DEV)).logits.float().cpu()
        again = tp_model(input_ids=ids.to(DEV)).logits.float().cpu()
    assert torch.equal(after, again)
    # int8 rows with 127 levels: a few per cent of the logits' spread, and not the 16-bit result itself
    err = (after - before).abs().max().item()
    assert 0 < err < 0.1 * before.std().item(), err
    with pytest.raises(RuntimeError, match="int8"):
        with tp.save_tensor_parallel(tp_model):
            tp_model.state_dict()
    assert any(k.endswith(".wq") for k in tp_model.state_dict())  # the shards themselves can be saved


def test_outlier_columns_by_name_and_conv1d():
    """Outlier columns chosen per Linear by its name; a transformers Conv1D ([in, out] weight) is quantised along its input
    axis like a Linear."""
    from transformers.pytorch_utils import Conv1D

    class Block(nn.Module):
        def __init__(self):
            super().__init__()
            self.fc = nn.Linear(64, 96)
            self.proj = Conv1D(48, 96)  # nf = 48 outputs, nx = 96 inputs

        def forward(self, x):
            return self.proj(torch.relu(self.fc(x)))

    torch.manual_seed(2)
    block = Block().to(torch.float16).to(DEV)
    x = torch.randn(5, 64, device=DEV, dtype=torch.float16)
    with torch.no_grad():
        want = block(x).float()
        n = quantize_linears_(block, outlier_cols={"fc": [3, 17], "proj": [0]})
        got = block(x).float()
    assert n == 2 and block.fc.outlier_idx.tolist() == [3, 17] and block.proj.outlier_idx.tolist() == [0]
    assert block.proj.in_features == 96 and block.proj.out_features == 48
    torch.testing.assert_close(got, want, rtol=5e-2, atol=5e-2 * want.std().item())
