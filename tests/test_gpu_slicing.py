"""Slicing engine on the GPU against the oracle: bit-exact."""
import numpy as np
import pytest
import torch

import tensor_parallel_amd as tp
from conftest import to_bits
from oracle import naming as onm
from oracle import slicing as osl
from tensor_parallel_amd import _native
from tensor_parallel_amd.slicing import BatchSlicer, concat_dim
from tensor_parallel_amd.slicing_configs import get_llama_config

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)


def rand_tensor(shape, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    if dtype in (torch.int8, torch.uint8, torch.int32, torch.int64):
        return torch.randint(0, 100, shape, generator=g).to(dtype)
    return (torch.randn(shape, generator=g) * 0.02).to(dtype)


def same_bits(dev_tensor, np_want):
    got = to_bits(dev_tensor)
    return got.shape == np_want.shape and np.array_equal(got, np_want)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16, torch.int8])
@pytest.mark.parametrize("shape,dim", [((64, 48), 0), ((64, 48), 1), ((10, 7), 1), ((5, 9, 6), 1), ((5, 9, 6), -1), ((33,), 0), ((3, 1000), 1), ((2, 3, 4, 10), 2)])
@pytest.mark.parametrize("world", [2, 3, 8])
def test_split_bit_exact(dtype, shape, dim, world):
    t = rand_tensor(shape, dtype, 0)
    bits = to_bits(t)
    td = t.to(DEV)
    action = tp.Split(world, dim)
    parts = [action(td, rank=r) for r in range(world)]
    for r in range(world):
        assert parts[r].is_contiguous() and parts[r].device == DEV
        assert same_bits(parts[r], osl.split(bits, world, dim, r)), (shape, dim, world, r)
    assert same_bits(action.undo(parts), bits)


@pytest.mark.parametrize("world", [1, 2, 3, 5])
def test_chunked_and_grouped_bit_exact(world):
    t = rand_tensor((24, 60), torch.bfloat16, 1)
    bits, td = to_bits(t), t.to(DEV)
    for dim, chunk in ((0, 4), (1, 5), (-1, 12), (-2, 3)):
        a = tp.SplitInChunks(world, dim, chunk)
        parts = [a(td, rank=r) for r in range(world)]
        for r in range(world):
            assert same_bits(parts[r], osl.split_in_chunks(bits, world, dim, chunk, r))
        assert same_bits(a.undo(parts), bits)
    for dim, groups, chunk in ((1, 3, 4), (1, 2, 5), (0, 3, 2), (0, 4, 1)):
        a = tp.SplitInGroupedChunks(world, dim, groups, chunk)
        parts = [a(td, rank=r) for r in range(world)]
        for r in range(world):
            assert same_bits(parts[r], osl.split_in_grouped_chunks(bits, world, dim, groups, chunk, r))
        assert same_bits(a.undo(parts), bits)


def test_docstring_vectors_on_device():
    def dev(s):
        return torch.tensor(list(s.replace(" ", "").encode()), dtype=torch.uint8, device=DEV)

    def txt(t):
        return bytes(t.cpu().tolist()).decode()

    assert [txt(tp.Split(3, 0)(dev("ABCDEFGHIJKLMNO"), rank=r)) for r in range(3)] == ["ABCDE", "FGHIJ", "KLMNO"]
    assert [txt(tp.SplitInChunks(3, 0, 3)(dev("AAABBBCCCDDDEEE"), rank=r)) for r in range(3)] == ["AAABBB", "CCCDDD", "EEE"]
    fused = dev("AABBCCDDEE AABBCCDDEE AABBCCDDEE")
    got = [tp.SplitInGroupedChunks(3, 0, 3, 2)(fused, rank=r) for r in range(3)]
    assert [txt(g) for g in got] == ["AABBAABBAABB", "CCDDCCDDCCDD", "EEEEEE"]
    assert txt(tp.SplitInGroupedChunks(3, 0, 3, 2).undo(got)) == "AABBCCDDEE" * 3


def test_empty_ragged_and_host_inputs():
    # more ranks than rows: trailing ranks get empty shards
    t = rand_tensor((3, 8), torch.float32, 2)
    parts = [tp.Split(5, 0)(t.to(DEV), rank=r) for r in range(5)]
    assert [p.shape[0] for p in parts] == [1, 1, 1, 0, 0]
    assert same_bits(tp.Split(5, 0).undo(parts), to_bits(t))
    # a host tensor is uploaded, sliced on the device, and the input is left untouched
    before = t.clone()
    out = tp.Split(2, 1)(t, rank=1)
    assert out.device.type == "cuda" and torch.equal(t, before)
    assert same_bits(out, osl.split(to_bits(t), 2, 1, 1))
    # non-contiguous input
    nc = rand_tensor((16, 12), torch.bfloat16, 3).to(DEV).t()
    assert same_bits(tp.Split(3, 0)(nc, rank=2), osl.split(to_bits(nc), 3, 0, 2))
    # zero-element tensor
    assert tp.Split(2, 0)(torch.empty(0, 4, device=DEV), rank=0).shape == (0, 4)
    # odd byte sizes exercise the 2-, 4- and 8-byte paths
    for shape, dtype in (((7, 13), torch.uint8), ((7, 13), torch.bfloat16), ((6, 10), torch.float32), ((4, 1026), torch.bfloat16)):
        x = rand_tensor(shape, dtype, 4)
        for r in range(3):
            assert same_bits(tp.Split(3, 1)(x.to(DEV), rank=r), osl.split(to_bits(x), 3, 1, r))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_scale_matches_torch_division(dtype):
    t = rand_tensor((1000,), dtype, 5) * 37
    for world in (2, 3, 7):
        got = tp.Scale(world)(t.to(DEV), rank=0).cpu()
        assert torch.equal(got, t / world)
        back = tp.Scale(world).undo([got.to(DEV)]).cpu()
        assert torch.equal(back, got * world)


def test_gather_concat_uneven_parts():
    parts = [rand_tensor((4, 6, n), torch.bfloat16, 10 + n) for n in (5, 0, 3, 8)]
    got = concat_dim([p.to(DEV) for p in parts], -1)
    assert torch.equal(got.cpu(), torch.cat(parts, dim=-1))
    got1 = concat_dim([p.to(DEV) for p in parts[:1]], 1)
    assert torch.equal(got1.cpu(), parts[0])


def _small_llama_state(hidden=128, heads=8, kv=4, ffn=344, vocab=320, layers=2, dtype=torch.bfloat16):
    hd = hidden // heads
    state, seed = {}, 0
    def add(name, shape):
        nonlocal seed
        state[name] = rand_tensor(shape, dtype, seed)
        seed += 1
    add("model.embed_tokens.weight", (vocab, hidden))
    for i in range(layers):
        p = f"model.layers.{i}."
        add(p + "self_attn.q_proj.weight", (hidden, hidden))
        add(p + "self_attn.k_proj.weight", (kv * hd, hidden))
        add(p + "self_attn.v_proj.weight", (kv * hd, hidden))
        add(p + "self_attn.o_proj.weight", (hidden, hidden))
        add(p + "mlp.gate_proj.weight", (ffn, hidden))
        add(p + "mlp.up_proj.weight", (ffn, hidden))
        add(p + "mlp.down_proj.weight", (hidden, ffn))
        add(p + "input_layernorm.weight", (hidden,))
        add(p + "post_attention_layernorm.weight", (hidden,))
    add("model.norm.weight", (hidden,))
    add("lm_head.weight", (vocab, hidden))
    return state, dict(hidden_size=hidden, num_attention_heads=heads, num_key_value_heads=kv)


@pytest.mark.parametrize("world", [2, 3, 4, 8])
def test_convert_state_dict_matches_oracle(world):
    from types import SimpleNamespace

    state, mc = _small_llama_state()
    cfg = get_llama_config(SimpleNamespace(model_type="llama", **mc), [DEV] * world)
    hd = mc["hidden_size"] // mc["num_attention_heads"]
    qpk = mc["num_attention_heads"] // mc["num_key_value_heads"]
    rules = [
        (r".*self_attn\.q_proj\.weight$", lambda a, r: osl.split_in_chunks(a, world, 0, qpk * hd, r)),
        (r".*self_attn\.k_proj\.weight$", lambda a, r: osl.split_in_chunks(a, world, 0, hd, r)),
        (r".*self_attn\.v_proj\.weight$", lambda a, r: osl.split_in_chunks(a, world, 0, hd, r)),
        (r".*self_attn\.o_proj\.weight$", lambda a, r: osl.split_in_chunks(a, world, 1, qpk * hd, r)),
        (r".*mlp\.gate_proj\.weight$", lambda a, r: osl.split(a, world, 0, r)),
        (r".*mlp\.down_proj\.weight$", lambda a, r: osl.split(a, world, 1, r)),
        (r".*mlp\.up_proj\.weight$", lambda a, r: osl.split(a, world, 0, r)),
        (r".*embed_tokens.weight$", lambda a, r: osl.split(a, world, 1, r)),
        (r".*lm_head\.weight$", lambda a, r: osl.split(a, world, 0, r)),
    ]
    patterns = [p.pattern for p in cfg.input_rules] + [p.pattern for p in cfg.output_rules]
    want = onm.convert_state_dict({k: to_bits(v) for k, v in state.items()}, rules, patterns, world)
    dev_state = {k: v.to(DEV) for k, v in state.items()}
    got = tp.convert_state_dict(dev_state, cfg, world)
    assert set(got.keys()) == set(want.keys())
    for k, w in want.items():
        assert same_bits(got[k], w), k
    for k, v in dev_state.items():  # inputs untouched
        assert torch.equal(v.cpu(), state[k])
    # host-resident input gives the same shards
    got_host = tp.convert_state_dict(state, cfg, world)
    for k, w in want.items():
        if "norm" not in k and "_sanity" not in k:
            assert got_host[k].device.type == "cuda" and same_bits(got_host[k], w), k


def test_batch_is_one_plan_and_counts_bytes():
    t = rand_tensor((256, 512), torch.bfloat16, 0).to(DEV)
    batch = BatchSlicer(DEV)
    outs = [batch.add(t, tp.Split(4, 1).spec(t.shape, r)) for r in range(4)]
    outs += [batch.add(t, tp.Split(4, 0).spec(t.shape, r)) for r in range(4)]
    moved = batch.run()
    torch.cuda.synchronize()
    assert moved == 2 * t.numel() * 2
    assert torch.equal(torch.cat(outs[:4], dim=1), t) and torch.equal(torch.cat(outs[4:], dim=0), t)
    batch.close()


def test_llama_7b_layer_full_size_round_trip():
    """One Llama-2-7B decoder layer plus embeddings at their real sizes, W = 2, 4, 8: split -> undo is the
    identity, and integer checksums of the shards add up to the checksum of the source."""
    from types import SimpleNamespace

    g = torch.Generator(device=DEV).manual_seed(0)
    def dev_rand(shape):
        return (torch.randn(shape, generator=g, device=DEV) * 0.02).to(torch.bfloat16)
    state = {
        "model.embed_tokens.weight": dev_rand((32000, 4096)),
        "model.layers.0.self_attn.q_proj.weight": dev_rand((4096, 4096)),
        "model.layers.0.self_attn.o_proj.weight": dev_rand((4096, 4096)),
        "model.layers.0.mlp.gate_proj.weight": dev_rand((11008, 4096)),
        "model.layers.0.mlp.down_proj.weight": dev_rand((4096, 11008)),
        "lm_head.weight": dev_rand((32000, 4096)),
    }
    mc = SimpleNamespace(model_type="llama", hidden_size=4096, num_attention_heads=32, num_key_value_heads=32)
    for world in (2, 4, 8):
        cfg = get_llama_config(mc, [DEV] * world)
        out = tp.convert_state_dict(state, cfg, world)
        names = tp.config.get_parameter_name_mapping(state.keys(), cfg)
        for name, full in state.items():
            shards = [out[f"module_shards.{r}.{names[name]}"] for r in range(world)]
            action = next(a for p, a in cfg.state_rules.items() if p.search(name))
            assert torch.equal(action.undo(shards), full), (name, world)
            total = sum(int(s.view(torch.int16).to(torch.int64).sum()) for s in shards)
            assert total == int(full.view(torch.int16).to(torch.int64).sum())
        assert out[f"module_shards.{world - 1}.{names['model.layers.0.mlp.down_proj.weight']}"].shape == (4096, 11008 // world)


@pytest.mark.parametrize("rows,row_bytes,src_pitch,dst_pitch", [
    (1, 1 << 20, 0, 0),            # contiguous, many tiles
    (3, 70001, 70001, 70001),      # contiguous by pitch, odd byte count (1-byte units)
    (5, 200000, 262144, 200000),   # long rows: several tiles per row
    (1000, 48, 96, 48),            # short rows: many rows per tile
    (7, 6, 10, 8),                 # 2-byte units
    (0, 16, 16, 16),               # empty
])
def test_planless_jobs_match_plan(rows, row_bytes, src_pitch, dst_pitch):
    """tpamd_copy_jobs_run derives its tiles on the device; the plan derives them on the host. Same bytes."""
    span_s = max(rows * max(src_pitch, row_bytes), 16)
    span_d = max(rows * max(dst_pitch, row_bytes), 16)
    g = torch.Generator().manual_seed(rows + row_bytes)
    src = torch.randint(0, 256, (span_s,), generator=g, dtype=torch.uint8).to(DEV)
    a = torch.full((span_d,), 0xEE, dtype=torch.uint8, device=DEV)
    b = a.clone()
    job = lambda dst: (src.data_ptr(), dst.data_ptr(), rows, row_bytes, src_pitch, dst_pitch)
    plan = _native.CopyPlan([job(a)], DEV)
    plan.run()
    torch.cuda.synchronize()
    plan.close()
    _native.run_copy_jobs([job(b)], DEV)
    torch.cuda.synchronize()
    assert torch.equal(a, b)
    want = np.full(span_d, 0xEE, dtype=np.uint8)
    s = src.cpu().numpy()
    for r in range(rows):
        want[r * dst_pitch: r * dst_pitch + row_bytes] = s[r * src_pitch: r * src_pitch + row_bytes]
    assert np.array_equal(b.cpu().numpy(), want)


def test_planless_many_jobs_and_limit():
    src = torch.arange(16 * 64, dtype=torch.int32, device=DEV)
    dst = torch.zeros_like(src)
    jobs = [(src.data_ptr() + 256 * i, dst.data_ptr() + 256 * (15 - i), 1, 256, 0, 0) for i in range(16)]
    _native.run_copy_jobs(jobs, DEV)
    torch.cuda.synchronize()
    assert torch.equal(dst.view(16, 64), src.view(16, 64).flip(0))
    arr = (_native.CopyJob * 17)(*[_native.CopyJob(*jobs[0]) for _ in range(17)])
    assert _native.lib().tpamd_copy_jobs_run(arr, 17, None) == -1
    assert b"at most" in _native.lib().tpamd_last_error()
    # the Python helper falls back to a plan beyond the limit
    dst.zero_()
    _native.run_copy_jobs(jobs + [(src.data_ptr(), dst.data_ptr(), 0, 0, 0, 0)], DEV)
    torch.cuda.synchronize()
    assert torch.equal(dst.view(16, 64), src.view(16, 64).flip(0))
