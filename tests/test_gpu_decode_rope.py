"""Decode step with the rotary embedding folded into the attention call (`tpamd_attention_decode_rope`) against the oracle's
two steps (oracle/rope.py, then oracle/attention.py in float64): the cache rows of the new position bit for bit, the
attention output to rtol 2e-2 with a floor of 2e-2 standard deviations; and against the two-call sequence on the device."""
import pytest
import torch

from oracle import attention as oat
from oracle import rope as orp
from tensor_parallel_amd import _native

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)
RTOL = 2e-2


def case(B, Hkv, per, D, pos0, L, dtype, seed, shared_angles=True):
    g = torch.Generator().manual_seed(seed)
    fused = torch.randn(B, 1, Hkv, per + 2, D, generator=g).to(dtype)  # a fused QKV projection output
    kc = torch.randn(B, Hkv, L, D, generator=g).to(dtype)
    vc = torch.randn(B, Hkv, L, D, generator=g).to(dtype)
    if shared_angles:
        cos, sin = orp.angles(torch.tensor([pos0]), D, dtype=dtype)  # [1, D]
        cos, sin = cos[None], sin[None]                              # [1, 1, D]
    else:  # every sequence at an angle of its own (left-padded batches)
        cs = [orp.angles(torch.tensor([pos0 + 3 * b]), D, dtype=dtype) for b in range(B)]
        cos, sin = torch.stack([c for c, _ in cs]), torch.stack([s for _, s in cs])  # [B, 1, D]
    return fused, kc, vc, cos, sin


def expected(fused, kc, vc, cos, sin, pos0, scale):
    B, _, Hkv, per2, D = fused.shape
    per = per2 - 2
    q = fused[:, :, :, :per].reshape(B, 1, Hkv * per, D)
    q_rot, kc2, vc2 = orp.rope_append(q, fused[:, :, :, per], fused[:, :, :, per + 1], cos, sin, kc.clone(), vc.clone(), pos0)
    want = oat.attention_f64(q_rot.float().numpy(), kc2[:, :, :pos0 + 1].float().numpy(), vc2[:, :, :pos0 + 1].float().numpy(), scale, True)
    return torch.from_numpy(want), kc2, vc2


def bits(t):
    return t.detach().cpu().contiguous().view(torch.int16)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,Hkv,per,D,pos0,L", [
    (8, 4, 16, 64, 2047, 2048),   # the Falcon-40B rank shard's decode step
    (2, 2, 8, 128, 300, 512),     # head_dim 128, ragged key count
    (3, 3, 1, 64, 0, 16),         # empty cache: the new position alone
    (2, 1, 4, 64, 1, 8),          # one cached key
    (1, 2, 16, 64, 63, 128), (1, 2, 16, 64, 64, 128), (1, 2, 16, 64, 65, 128),  # around a key tile
    (1, 4, 16, 64, 8191, 8200),   # long ranges: the kernel with several tiles in flight
    (40, 8, 2, 128, 777, 800),    # enough (batch, kv head) pairs that the keys are not split: the partials are still merged
])
def test_fused_decode_matches_the_oracle(dtype, B, Hkv, per, D, pos0, L):
    fused, kc, vc, cos, sin = case(B, Hkv, per, D, pos0, L, dtype, seed=pos0 + B)
    scale = D ** -0.5
    want, want_kc, want_vc = expected(fused, kc, vc, cos, sin, pos0, scale)
    fd, kcd, vcd = fused.to(DEV), kc.to(DEV), vc.to(DEV)
    got = _native.attention_decode_rope(fd[:, :, :, :per], fd[:, :, :, per], fd[:, :, :, per + 1], cos.to(DEV), sin.to(DEV), kcd, vcd, pos0)
    assert got.shape == (B, 1, Hkv * per, D) and got.dtype == dtype
    assert torch.equal(bits(kcd), bits(want_kc)) and torch.equal(bits(vcd), bits(want_vc))
    torch.testing.assert_close(got.double().cpu(), want, rtol=RTOL, atol=RTOL * want.std().item())


def test_fused_decode_against_the_two_calls_and_per_sequence_angles():
    """The same step as rope_append + attention on the device: the caches identical, the outputs apart by the rounding of
    one probability; cos / sin per sequence; a plain [B, 1, Hq, D] query view; a scale of the caller's."""
    B, Hkv, per, D, pos0, L = 4, 2, 8, 64, 1000, 1024
    fused, kc, vc, cos, sin = case(B, Hkv, per, D, pos0, L, torch.bfloat16, seed=5, shared_angles=False)
    fd = fused.to(DEV)
    q_plain = fd[:, :, :, :per].reshape(B, 1, Hkv * per, D)
    kc1, vc1, kc2, vc2 = kc.to(DEV), vc.to(DEV), kc.to(DEV), vc.to(DEV)
    got = _native.attention_decode_rope(q_plain, fd[:, :, :, per], fd[:, :, :, per + 1], cos.to(DEV), sin.to(DEV), kc1, vc1, pos0, scale=0.2)
    q_rot = _native.rope_append(q_plain, fd[:, :, :, per], fd[:, :, :, per + 1], cos.to(DEV), sin.to(DEV), kc2, vc2, pos0)
    two = _native.attention(q_rot, kc2[:, :, :pos0 + 1], vc2[:, :, :pos0 + 1], scale=0.2, causal=True)
    assert torch.equal(bits(kc1), bits(kc2)) and torch.equal(bits(vc1), bits(vc2))
    torch.testing.assert_close(got.float(), two.float(), rtol=RTOL, atol=RTOL * two.float().std().item())
    want, _, _ = expected(fused, kc, vc, cos, sin, pos0, 0.2)
    torch.testing.assert_close(got.double().cpu(), want, rtol=RTOL, atol=RTOL * want.std().item())


def test_fused_decode_steps_in_a_row_fill_the_cache():
    """Five decode steps: each sees what the steps before it appended."""
    B, Hkv, per, D, L = 2, 2, 4, 64, 16
    g = torch.Generator().manual_seed(9)
    kc, vc = torch.zeros(B, Hkv, L, D, dtype=torch.float16), torch.zeros(B, Hkv, L, D, dtype=torch.float16)
    kcd, vcd = kc.to(DEV), vc.to(DEV)
    for pos in range(5):
        fused = torch.randn(B, 1, Hkv, per + 2, D, generator=g).to(torch.float16)
        cos, sin = orp.angles(torch.tensor([pos]), D, dtype=torch.float16)
        want, kc, vc = expected(fused, kc, vc, cos[None], sin[None], pos, D ** -0.5)
        fd = fused.to(DEV)
        got = _native.attention_decode_rope(fd[:, :, :, :per], fd[:, :, :, per], fd[:, :, :, per + 1], cos.to(DEV), sin.to(DEV), kcd, vcd, pos)
        assert torch.equal(bits(kcd), bits(kc)) and torch.equal(bits(vcd), bits(vc))
        torch.testing.assert_close(got.double().cpu(), want, rtol=RTOL, atol=RTOL * want.std().item())


def test_fused_decode_argument_errors():
    fused, kc, vc, cos, sin = (t.to(DEV) for t in case(1, 2, 2, 64, 3, 8, torch.float16, seed=1))
    q, k, v = fused[:, :, :, :2], fused[:, :, :, 2], fused[:, :, :, 3]
    with pytest.raises(ValueError, match="does not fit a cache"):
        _native.attention_decode_rope(q, k, v, cos, sin, kc, vc, 8)
    with pytest.raises(ValueError, match="one new position"):
        _native.attention_decode_rope(q.expand(1, 2, 2, 2, 64), k.expand(1, 2, 2, 64), v.expand(1, 2, 2, 64), cos, sin, kc, vc, 3)
    with pytest.raises(TypeError):
        _native.attention_decode_rope(q.float(), k.float(), v.float(), cos.float(), sin.float(), kc.float(), vc.float(), 3)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,Hkv,per,D,pos0,L", [
    (8, 4, 16, 64, 2047, 2048),   # the last position of a full cache
    (8, 4, 16, 64, 100, 2048),    # few keys in caches laid out for many: most key splits are empty
    (2, 2, 8, 128, 300, 512),
    (3, 3, 1, 64, 0, 16),         # nothing cached yet
    (1, 2, 16, 64, 63, 128), (1, 2, 16, 64, 64, 128), (1, 2, 16, 64, 65, 128),
    (1, 4, 16, 64, 5000, 8200),   # the kernel with several tiles in flight, on a range shorter than its launch was laid out for
    (40, 8, 2, 128, 777, 800),
])
def test_position_read_on_the_device_matches_the_oracle(dtype, B, Hkv, per, D, pos0, L):
    """`pos0` as an int64 tensor on the device (`tpamd_attention_decode_rope_devpos`): the same step, laid out for the capacity."""
    fused, kc, vc, cos, sin = case(B, Hkv, per, D, pos0, L, dtype, seed=pos0 + B + 1)
    scale = D ** -0.5
    want, want_kc, want_vc = expected(fused, kc, vc, cos, sin, pos0, scale)
    fd, kcd, vcd = fused.to(DEV), kc.to(DEV), vc.to(DEV)
    pos = torch.tensor(pos0, dtype=torch.int64, device=DEV)
    got = _native.attention_decode_rope(fd[:, :, :, :per], fd[:, :, :, per], fd[:, :, :, per + 1], cos.to(DEV), sin.to(DEV), kcd, vcd, pos)
    assert torch.equal(bits(kcd), bits(want_kc)) and torch.equal(bits(vcd), bits(want_vc))
    torch.testing.assert_close(got.double().cpu(), want, rtol=RTOL, atol=RTOL * want.std().item())
    assert int(pos) == pos0  # the caller advances the count


def test_one_graph_serves_every_decode_step():
    """The call recorded once in a HIP graph; every replay reads the count anew. Eager work and synchronisations sit between
    the replays, and every replay is checked against the oracle."""
    B, Hkv, per, D, L = 2, 2, 8, 64, 256
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(11)
    kc, vc = torch.zeros(B, Hkv, L, D, dtype=dtype), torch.zeros(B, Hkv, L, D, dtype=dtype)
    kcd, vcd = kc.to(DEV), vc.to(DEV)
    pos = torch.zeros((), dtype=torch.int64, device=DEV)
    fd = torch.zeros(B, 1, Hkv, per + 2, D, dtype=dtype, device=DEV)
    cosd, sind = torch.zeros(1, 1, D, dtype=dtype, device=DEV), torch.zeros(1, 1, D, dtype=dtype, device=DEV)
    out = torch.empty(B, 1, Hkv * per, D, dtype=dtype, device=DEV)

    def step():
        _native.attention_decode_rope(fd[:, :, :, :per], fd[:, :, :, per], fd[:, :, :, per + 1], cosd, sind, kcd, vcd, pos, out=out)
        pos.add_(1)

    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        step()  # the stream's scratch buffer is made outside the capture
    torch.cuda.current_stream().wait_stream(stream)
    torch.cuda.synchronize()
    kcd.zero_(), vcd.zero_(), pos.zero_()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        step()
    kcd.zero_(), vcd.zero_(), pos.zero_()
    for p in range(70):  # past a tile of 64 keys
        fused = torch.randn(B, 1, Hkv, per + 2, D, generator=g).to(dtype)
        cos, sin = orp.angles(torch.tensor([p]), D, dtype=dtype)
        want, kc, vc = expected(fused, kc, vc, cos[None], sin[None], p, D ** -0.5)
        fd.copy_(fused.to(DEV)), cosd.copy_(cos[None].to(DEV)), sind.copy_(sin[None].to(DEV))
        graph.replay()
        torch.cuda.synchronize()
        assert int(pos) == p + 1
        assert torch.equal(bits(kcd), bits(kc)) and torch.equal(bits(vcd), bits(vc)), f"caches after step {p}"
        torch.testing.assert_close(out.double().cpu(), want, rtol=RTOL, atol=RTOL * want.std().item(), msg=lambda m: f"step {p}: {m}")


def test_count_past_the_capacity_leaves_the_caches_alone():
    B, Hkv, per, D, L = 1, 2, 2, 64, 8
    fused, kc, vc, cos, sin = (t.to(DEV) for t in case(B, Hkv, per, D, 3, L, torch.float16, seed=2))
    before_k, before_v = kc.clone(), vc.clone()
    pos = torch.tensor(L, dtype=torch.int64, device=DEV)
    out = _native.attention_decode_rope(fused[:, :, :, :per], fused[:, :, :, per], fused[:, :, :, per + 1], cos, sin, kc, vc, pos)
    torch.cuda.synchronize()
    assert torch.equal(kc, before_k) and torch.equal(vc, before_v) and torch.isfinite(out.float()).all()
    with pytest.raises(ValueError, match="one int64 element"):
        _native.attention_decode_rope(fused[:, :, :, :per], fused[:, :, :, per], fused[:, :, :, per + 1], cos, sin, kc, vc, pos.to(torch.int32))
