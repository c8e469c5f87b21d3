"""Transposing mover and the [in, out]-weight (Conv1D) route on the GPU: element movement bit-exact against the
oracle, the shard matmul against F.linear on the transposed weight."""
import numpy as np
import pytest
import torch

import tensor_parallel_amd as tp
from conftest import to_bits
from oracle import shard_forward as ofw
from oracle import slicing as osl
from tensor_parallel_amd import _native
from tensor_parallel_amd.slicing import BatchSlicer, is_k_major

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)


def rand_tensor(shape, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    if dtype in (torch.int8, torch.uint8, torch.int32):
        return torch.randint(-100, 100, shape, generator=g).to(dtype)
    return (torch.randn(shape, generator=g) * 0.02).to(dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16, torch.int8, torch.int32])
@pytest.mark.parametrize("shape", [(64, 64), (128, 256), (1, 1), (1, 300), (300, 1), (7, 5), (65, 63), (100, 257), (768, 2304), (1000, 129), (33, 4096)])
def test_whole_tensor_transpose_bit_exact(dtype, shape):
    t = rand_tensor(shape, dtype, 0)
    got = _native.transpose_regions(t.to(DEV), [(0, shape[1])])
    assert got.is_contiguous() and tuple(got.shape) == shape[::-1]
    assert np.array_equal(to_bits(got), osl.in_axis_fastest(to_bits(t)))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.int8])
def test_regions_with_unaligned_offsets_and_pitches(dtype):
    """Column and row ranges whose byte offsets are not multiples of 16 take the element path; aligned ones next to
    them in the same launch take the vector path."""
    t = rand_tensor((203, 331), dtype, 1)
    bits = to_bits(t)
    td = t.to(DEV)
    for rows, cols in (((0, 203), [(0, 331)]), ((3, 200), [(1, 66), (100, 101), (128, 320)]), ((64, 192), [(64, 192)]), ((5, 5), [(0, 10)]),
                       ((0, 203), [(7, 7), (8, 331)])):
        got = _native.transpose_regions(td, cols, rows)
        want = np.concatenate([bits[rows[0]:rows[1], a:b] for a, b in cols], axis=1).T
        assert np.array_equal(to_bits(got), want), (rows, cols)


def test_sixteen_jobs_per_launch_and_more():
    t = rand_tensor((96, 40 * 24), torch.bfloat16, 2)
    cols = [(i * 24, i * 24 + 24) for i in range(40)][::-1]
    got = _native.transpose_regions(t.to(DEV), cols)
    want = np.concatenate([to_bits(t)[:, a:b] for a, b in cols], axis=1).T
    assert np.array_equal(to_bits(got), want)


def test_bad_arguments_raise_before_any_launch():
    t = torch.zeros(8, 8, device=DEV)
    with pytest.raises(ValueError):
        _native.transpose_regions(t, [(0, 9)])
    with pytest.raises(ValueError):
        _native.transpose_regions(t.double(), [(0, 8)])
    with pytest.raises(ValueError):
        _native.transpose_regions(t[:, ::2], [(0, 4)])
    with pytest.raises(_native.NativeLibraryError):
        _native.transpose_regions(t.cpu(), [(0, 8)])
    with pytest.raises(ValueError, match="pitch"):
        _native.run_transpose_jobs([(t.data_ptr(), t.data_ptr() + 4096, 8, 8, 16, 32)], 4, DEV)
    with pytest.raises(ValueError, match="elem_bytes"):
        _native.run_transpose_jobs([(t.data_ptr(), t.data_ptr(), 8, 8, 32, 32)], 8, DEV)


@pytest.mark.parametrize("world", [2, 3, 4])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_gpt2_rules_slice_and_transpose_in_one_pass(world, dtype):
    """The GPT-2 table's weight rules (slicing_configs.py:192-201) on [in, out] weights of GPT-2 small, shards written
    with the `in` axis fastest by the batch slicer: same elements as the oracle's shard, stored as its transpose."""
    hidden, head = 768, 64
    cases = [((hidden, 3 * hidden), tp.SplitInGroupedChunks(world, 1, 3, head), lambda b, r: osl.split_in_grouped_chunks(b, world, 1, 3, head, r)),
             ((hidden, hidden), tp.SplitInChunks(world, 0, head), lambda b, r: osl.split_in_chunks(b, world, 0, head, r)),
             ((hidden, 4 * hidden), tp.Split(world, 1), lambda b, r: osl.split(b, world, 1, r)),
             ((4 * hidden, hidden), tp.Split(world, 0), lambda b, r: osl.split(b, world, 0, r)),
             ((50, 37), tp.Split(world, 1), lambda b, r: osl.split(b, world, 1, r)),
             ((50, 37), tp.Split(world, 0), lambda b, r: osl.split(b, world, 0, r))]
    batch = BatchSlicer(DEV)
    made = []
    for i, (shape, action, want) in enumerate(cases):
        t = rand_tensor(shape, dtype, 10 + i)
        td = t.to(DEV)
        for r in range(world):
            made.append((batch.add(td, action.spec(shape, r), k_major=True), want(to_bits(t), r), action, td))
    batch.run()
    torch.cuda.synchronize()
    batch.close()
    for shard, want, _, _ in made:
        assert tuple(shard.shape) == want.shape and is_k_major(shard)
        assert np.array_equal(to_bits(shard.t()), osl.in_axis_fastest(want))
        assert np.array_equal(to_bits(shard.contiguous()), want)
    # undo takes the shards as they are stored and gives the unsplit weight back, bit for bit
    for i in range(0, len(made), world):
        action, td = made[i][2], made[i][3]
        assert torch.equal(action.undo([m[0] for m in made[i:i + world]]), td)


@pytest.mark.parametrize("dtype,rtol", [(torch.bfloat16, 2e-2), (torch.float16, 2e-2), (torch.float32, 1e-5)])
@pytest.mark.parametrize("tokens", [1, 5, 300])
def test_shard_conv1d_forward_matches_linear_on_the_transposed_weight(dtype, rtol, tokens):
    from transformers.pytorch_utils import Conv1D

    from tensor_parallel_amd.shard_modules import install_shard_kernels

    torch.manual_seed(0)
    holder = torch.nn.Sequential(Conv1D(2304, 768), Conv1D(768, 3072))
    with torch.no_grad():
        for m in holder:
            m.weight.normal_(0, 0.02)
            m.bias.normal_(0, 0.5)
    x = [torch.randn(2, tokens, 768), torch.randn(2, tokens, 3072)]
    want = [torch.nn.functional.linear(xi.to(dtype).double(), m.weight.to(dtype).double().t(), m.bias.to(dtype).double()) for xi, m in zip(x, holder)]
    oracle = [ofw.conv1d_shard(xi.to(dtype).double(), m.weight.to(dtype).double(), m.bias.to(dtype).double()) for xi, m in zip(x, holder)]
    shard = holder.to(dtype).to(DEV)
    install_shard_kernels(shard)
    for i, m in enumerate(shard):
        assert type(m).__name__ == "ShardConv1D" and isinstance(m, Conv1D)
        with torch.no_grad():
            got = m(x[i].to(dtype).to(DEV))
        assert is_k_major(m.weight) and tuple(m.weight.shape) == tuple(holder[i].weight.shape)  # laid out at the first forward
        scale = want[i].std().item()
        torch.testing.assert_close(oracle[i], want[i], rtol=1e-12, atol=1e-12)
        torch.testing.assert_close(got.double().cpu(), want[i], rtol=rtol, atol=rtol * scale)
        with torch.no_grad():
            again = m(x[i].to(dtype).to(DEV))
        assert torch.equal(again, got)


def test_gpt2_shards_run_conv1d_on_the_kernels_and_match_the_unsplit_model():
    from transformers import GPT2Config, GPT2LMHeadModel

    torch.manual_seed(0)
    cfg = GPT2Config(n_layer=2, n_head=4, n_embd=256, vocab_size=512, n_positions=64)
    model = GPT2LMHeadModel(cfg).eval()
    ids = torch.randint(0, 512, (2, 17), generator=torch.Generator().manual_seed(1))
    with torch.no_grad():
        want = model(ids).logits
    tpm = tp.tensor_parallel(model, [DEV, DEV])
    convs = [m for shard in tpm.wrapped_model.module_shards for m in shard.modules() if type(m).__name__ == "ShardConv1D"]
    assert len(convs) == 2 * 2 * 4 and all(is_k_major(m.weight) for m in convs)
    with torch.no_grad():
        got = tpm(ids.to(DEV)).logits
    torch.testing.assert_close(got.cpu(), want, rtol=1e-4, atol=2e-4)
    # the state dict comes back in the unsplit model's layout and values
    with tp.save_tensor_parallel(tpm):
        sd = tpm.state_dict()
    ref = model.state_dict()
    assert set(sd) == set(ref)
    for name, t in ref.items():
        assert torch.equal(sd[name].cpu(), t), name
