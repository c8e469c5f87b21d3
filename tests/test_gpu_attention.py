"""Rank-local attention core on the GPU against the oracle (float64 on the CPU): rtol 2e-2 on 16-bit inputs, plus an
absolute floor of 2e-2 standard deviations of the expected output (outputs are convex combinations of v rows: over
2048 keys with N(0,1) values their spread is 0.03-0.04, so a floor in units of the values would hide a lost key tile)."""
import numpy as np
import pytest
import torch

from oracle import attention as oat
from tensor_parallel_amd import _native

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)
RTOL = 2e-2


def make(B, Hq, Hkv, Sq, Skv, D, dtype, seed=0):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, Hq, Sq, D, generator=g).to(dtype)
    k = torch.randn(B, Hkv, Skv, D, generator=g).to(dtype)
    v = torch.randn(B, Hkv, Skv, D, generator=g).to(dtype)
    return q, k, v


def close(got, want):
    want = torch.from_numpy(want)
    torch.testing.assert_close(got.double().cpu(), want, rtol=RTOL, atol=RTOL * want.std().item())


def check(q, k, v, causal, scale=None):
    D = q.shape[-1]
    scale = D ** -0.5 if scale is None else scale
    got = _native.attention(q.to(DEV), k.to(DEV), v.to(DEV), scale=scale, causal=causal)
    assert got.shape == (q.shape[0], q.shape[2], q.shape[1], D) and got.dtype == q.dtype
    want = oat.attention_f64(q.float().numpy(), k.float().numpy(), v.float().numpy(), scale, causal)
    close(got, want)
    return got


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("B,Hq,Hkv,Sq,Skv,D", [
    (2, 4, 4, 64, 64, 64),      # one tile of rows per head, equal heads
    (1, 16, 2, 1, 300, 64),     # decode: a group of 8 heads in one MFMA tile, ragged key count
    (2, 8, 2, 3, 200, 64),      # a few new positions on a cache
    (1, 2, 1, 70, 70, 64),      # row tiles that straddle heads, ragged
    (1, 4, 2, 130, 130, 128),   # head_dim 128
    (3, 6, 3, 1, 17, 128),      # fewer keys than a tile
    (2, 8, 2, 256, 256, 64),    # several position tiles per head and several (batch, kv head) pairs: the causal block order
])
def test_attention_matches_oracle(dtype, causal, B, Hq, Hkv, Sq, Skv, D):
    check(*make(B, Hq, Hkv, Sq, Skv, D, dtype), causal)


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("Skv", [64, 65, 127, 128, 129, 192, 200, 256, 321])
@pytest.mark.parametrize("Sq", [1, 40, 130])
def test_key_counts_around_the_tile_size(Sq, Skv, causal):
    """1 to 6 key tiles of 64, full and ragged: the tiles alternate between two LDS buffers and the tile after next is
    prefetched, so every count of tiles ends the pipeline differently."""
    if causal and Sq > Skv:
        pytest.skip("more new positions than keys")
    check(*make(2, 4, 2, Sq, Skv, 64, torch.bfloat16, seed=Sq * 1000 + Skv), causal)


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("Skv", [1, 63, 64, 65, 128, 200, 256, 257, 320, 449, 512, 577, 640, 1100])
@pytest.mark.parametrize("Sq", [1, 40])
def test_key_counts_with_several_tiles_in_flight(tune, Sq, Skv, D, causal):
    """The kernel that keeps 4 (head_dim 64) or 2 (128) key tiles requested per block, forced onto short ranges too: 1 to
    18 tiles, so that the rounds of 4 / 2 end after every possible number of tiles, with full and ragged last tiles."""
    if causal and Sq > Skv:
        pytest.skip("more new positions than keys")
    tune("TPAMD_ATTN_RING", 1)
    check(*make(2, 4, 2, Sq, Skv, D, torch.float16 if Skv % 2 else torch.bfloat16, seed=Sq * 1000 + Skv), causal)


@pytest.mark.parametrize("ring", [0, 1])
@pytest.mark.parametrize("splits", [1, 3, 8])
def test_both_few_row_kernels_on_split_key_ranges(tune, ring, splits):
    """Decode on 2100 keys cut into 1, 3 and 8 ranges (the last one ragged), by the kernel with one tile in flight and by
    the one with several: the default choice between them depends on the range length, here both take every length."""
    tune("TPAMD_ATTN_SPLITS", splits)
    tune("TPAMD_ATTN_RING", ring)
    check(*make(2, 16, 2, 1, 2100, 64, torch.bfloat16, seed=11), True)
    check(*make(1, 8, 2, 3, 2100, 128, torch.float16, seed=12), True)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("Sq,causal", [(1, False), (96, False), (96, True)])
def test_reference_maximum_moves_along_the_keys(dtype, Sq, causal):
    """Scores that grow along the keys, in steps larger and smaller than the 2^6 the running reference tolerates, then
    fall again: the accumulators are rescaled several times and most tiles take the path without any rescaling."""
    B, Hq, Hkv, Skv, D = 1, 4, 2, 640, 64
    g = torch.Generator().manual_seed(5)
    q = torch.randn(B, Hq, Sq, D, generator=g)
    k = torch.randn(B, Hkv, Skv, D, generator=g) * 0.05
    v = torch.randn(B, Hkv, Skv, D, generator=g)
    # keys aligned with the mean query direction get a score that depends on their position
    direction = q.mean(dim=(0, 1, 2))
    direction = direction / direction.norm()
    level = torch.zeros(Skv)
    level[64:128] = 2.0      # a small step: inside the tolerance
    level[128:320] = 12.0    # a large one
    level[320:384] = 40.0    # larger still, for one tile
    level[384:] = 11.0       # and back
    k = k + level[None, None, :, None] * direction[None, None, None, :]
    q = q + 3.0 * direction  # every query has a clearly positive component along it
    check(q.to(dtype), k.to(dtype), v.to(dtype), causal, scale=1.0)


@pytest.mark.parametrize("Sq", [1, 200])
def test_output_rows_on_8_byte_boundaries_only(Sq):
    """The output may be a view whose rows start on 8-byte boundaries (the ABI asks for no more), with other data between
    the rows."""
    B, Hq, Hkv, Skv, D = 2, 4, 2, 200, 64
    q, k, v = make(B, Hq, Hkv, Sq, Skv, D, torch.bfloat16, seed=11)
    want = _native.attention(q.to(DEV), k.to(DEV), v.to(DEV), causal=True)
    store = torch.full((B, Sq, Hq, D + 4), 7.0, dtype=torch.bfloat16, device=DEV)
    out = store[..., 4:]  # rows at byte offsets 8, 144, ...: 8-byte but not 16-byte aligned
    assert out.data_ptr() % 16 == 8
    got = _native.attention(q.to(DEV), k.to(DEV), v.to(DEV), causal=True, out=out)
    assert got.data_ptr() == out.data_ptr()
    torch.testing.assert_close(got, want, rtol=0, atol=0)
    assert bool((store[..., :4] == 7.0).all())


def test_strided_inputs_as_projection_outputs_produce_them():
    """q / k / v as views of [B, S, H, D] projection outputs (what the attention modules pass), sliced cache."""
    B, Hq, Hkv, S, D = 2, 8, 2, 96, 64
    g = torch.Generator().manual_seed(3)
    qkv = torch.randn(B, S, (Hq + 2 * Hkv) * D, generator=g).to(torch.bfloat16).to(DEV)
    q = qkv[..., : Hq * D].view(B, S, Hq, D).transpose(1, 2)
    k = qkv[..., Hq * D: (Hq + Hkv) * D].view(B, S, Hkv, D).transpose(1, 2)
    v = qkv[..., (Hq + Hkv) * D:].view(B, S, Hkv, D).transpose(1, 2)
    assert not q.is_contiguous()
    got = _native.attention(q, k, v, causal=True)
    want = oat.attention_f64(q.float().cpu().numpy(), k.float().cpu().numpy(), v.float().cpu().numpy(), D ** -0.5, True)
    close(got, want)
    assert torch.equal(got, _native.attention(q.contiguous(), k.contiguous(), v.contiguous(), causal=True))


def test_falcon_40b_rank_shard_decode_and_prefill():
    """BASELINE config 4 at W = 2: 64 query heads and 4 key/value heads per rank, head_dim 64; decode batch 8 on 2048
    cached keys (split over the keys), prefill of 1024 positions (sampled rows against the oracle)."""
    q, k, v = make(8, 64, 4, 1, 2048, 64, torch.bfloat16, seed=1)
    check(q, k, v, True)
    q, k, v = make(1, 64, 4, 1024, 1024, 64, torch.bfloat16, seed=2)
    got = _native.attention(q.to(DEV), k.to(DEV), v.to(DEV), causal=True)
    assert torch.isfinite(got.float()).all()
    heads = [0, 17, 63]
    want = oat.attention_f64(q[:, heads].float().numpy(), k[:, [0, 1, 3]].float().numpy(), v[:, [0, 1, 3]].float().numpy(), 64 ** -0.5, True)
    close(got[:, :, heads], want)


@pytest.mark.parametrize("causal", [True, False])
def test_falcon_40b_rank_shard_prefill_at_batch_8(causal):
    """The benchmark's prefill shape (8 x 1024 positions, 64 query heads on 4 key/value heads, 16 key tiles and 8 row
    tiles per head), sampled (batch, head) pairs against the oracle: first, middle and last of both axes, so that a
    block order or a row-to-wavefront mapping that goes wrong late in the grid shows."""
    B = 8
    q, k, v = make(B, 64, 4, 1024, 1024, 64, torch.bfloat16, seed=6)
    got = _native.attention(q.to(DEV), k.to(DEV), v.to(DEV), causal=causal)
    assert torch.isfinite(got.float()).all()
    for b, heads in [(0, [0, 15, 16, 63]), (3, [31, 47]), (7, [0, 33, 63])]:
        for h in heads:
            want = oat.attention_f64(q[b:b + 1, h:h + 1].float().numpy(), k[b:b + 1, h // 16:h // 16 + 1].float().numpy(),
                                     v[b:b + 1, h // 16:h // 16 + 1].float().numpy(), 64 ** -0.5, causal)
            close(got[b:b + 1, :, h:h + 1], want)


def test_split_and_unsplit_key_ranges_agree():
    """The same decode rows with many keys (split over blocks, merged by the second kernel) and as part of a batch
    large enough not to be split."""
    q, k, v = make(1, 16, 1, 1, 4096, 64, torch.float16, seed=4)
    one = _native.attention(q.to(DEV), k.to(DEV), v.to(DEV), causal=False)
    B = 300
    many = _native.attention(q.expand(B, -1, -1, -1).contiguous().to(DEV), k.expand(B, -1, -1, -1).contiguous().to(DEV),
                             v.expand(B, -1, -1, -1).contiguous().to(DEV), causal=False)
    torch.testing.assert_close(many[7].float(), one[0].float(), rtol=2e-3, atol=2e-3)


def test_argument_errors():
    q, k, v = make(1, 4, 3, 2, 2, 64, torch.float16)
    with pytest.raises(ValueError):
        _native.attention(q.to(DEV), k.to(DEV), v.to(DEV))  # 4 query heads over 3 key/value heads
    q, k, v = make(1, 2, 2, 5, 3, 64, torch.float16)
    with pytest.raises(ValueError):
        _native.attention(q.to(DEV), k.to(DEV), v.to(DEV), causal=True)  # more queries than keys
    q, k, v = make(1, 2, 2, 4, 4, 32, torch.float16)
    with pytest.raises(RuntimeError):
        _native.attention(q.to(DEV), k.to(DEV), v.to(DEV))  # head_dim 32: no kernel
    with pytest.raises(TypeError):
        _native.attention(q.float().to(DEV), k.float().to(DEV), v.float().to(DEV))


def test_llama_with_the_registered_attention_implementation():
    """A small Llama (grouped-query, head_dim 64) with attn_implementation "tpamd" against the same weights with
    transformers' eager attention: prefill logits and one decode step on the cache, unsplit and through
    tp.tensor_parallel on two ranks sharing the device."""
    from copy import deepcopy

    from transformers import LlamaConfig, LlamaForCausalLM

    import tensor_parallel_amd as tp

    name = tp.attention.register()
    torch.manual_seed(0)
    cfg = LlamaConfig(vocab_size=512, hidden_size=512, intermediate_size=1024, num_hidden_layers=2, num_attention_heads=8,
                      num_key_value_heads=2, max_position_embeddings=256, attn_implementation="eager")
    model = LlamaForCausalLM(cfg).to(torch.bfloat16).to(DEV).eval()
    ids = torch.randint(0, 512, (2, 48), generator=torch.Generator().manual_seed(1)).to(DEV)
    nxt = torch.randint(0, 512, (2, 1), generator=torch.Generator().manual_seed(2)).to(DEV)
    with torch.no_grad():
        ref = model(input_ids=ids, use_cache=True)
        ref_step = model(input_ids=nxt, past_key_values=ref.past_key_values, use_cache=True).logits
    fast = deepcopy(model)
    fast.config._attn_implementation = name
    with torch.no_grad():
        out = fast(input_ids=ids, use_cache=True)
        step = fast(input_ids=nxt, past_key_values=out.past_key_values, use_cache=True).logits
    scale = ref.logits.float().std().item()
    torch.testing.assert_close(out.logits.float(), ref.logits.float(), rtol=RTOL, atol=3 * RTOL * scale)
    torch.testing.assert_close(step.float(), ref_step.float(), rtol=RTOL, atol=3 * RTOL * scale)
    model_tp = tp.tensor_parallel(deepcopy(fast), [DEV, DEV])
    with torch.no_grad():
        tp_logits = model_tp(input_ids=ids, use_cache=False).logits
    torch.testing.assert_close(tp_logits.float(), ref.logits.float(), rtol=RTOL, atol=3 * RTOL * scale)
