"""Host-side logic of the product, checked without a GPU: slice specs and copy-job tables against the oracle,
renaming against the golden vectors, rule matching, meta-device model building, and the C ABI's exports."""
import ctypes
import json
import re
import threading
from pathlib import Path
from types import SimpleNamespace

import numpy as np
import pytest
import torch
from torch import nn

import tensor_parallel_amd as tp
from conftest import run_jobs_on_host
from oracle import slicing as osl
from tensor_parallel_amd import _native
from tensor_parallel_amd.aux_actions import split_inner_dim, split_num_heads
from tensor_parallel_amd.collectives import CollectiveOperation
from tensor_parallel_amd.config import get_parameter_name_mapping
from tensor_parallel_amd.shard import find_matching_actions
from tensor_parallel_amd.slicing import SliceSpec, copy_jobs, tensor_split_range
from tensor_parallel_amd.slicing_configs import get_gpt2_config, get_llama_config, get_refined_web_config

ROOT = Path(__file__).resolve().parent.parent
GOLDEN = json.loads((Path(__file__).parent / "golden" / "naming.json").read_text())


# ---------------------------------------------------------------------------------------- C ABI
def test_library_loads_and_exports_every_declared_symbol():
    assert _native.available(), _native.load_error()
    header = (ROOT / "include" / "tpamd.h").read_text()
    declared = set(re.findall(r"\b(tpamd_[a-z0-9_]+)\s*\(", header))
    assert declared == set(_native.EXPORTS)
    lib = ctypes.CDLL(str(_native.LIB_PATH))
    for name in declared:
        assert getattr(lib, name) is not None
    assert lib.tpamd_abi_version() == _native.ABI_VERSION


def test_compute_refuses_host_tensors():
    with pytest.raises(_native.NativeLibraryError):
        _native.linear(torch.zeros(2, 8), torch.zeros(4, 8))
    with pytest.raises(_native.NativeLibraryError):
        _native.reduce_partials([torch.zeros(4), torch.zeros(4)])
    if not torch.cuda.is_available():
        with pytest.raises(_native.NativeLibraryError):
            tp.Split(2, 0)(torch.zeros(4, 4), rank=0)
        with pytest.raises(_native.NativeLibraryError):
            tp.TensorParallel(nn.Sequential(nn.Linear(4, 4)), ["cpu", "cpu"])


# ---------------------------------------------------------------------------------------- specs and job tables
def _run_spec_on_host(a: np.ndarray, spec: SliceSpec) -> np.ndarray:
    src = np.ascontiguousarray(a).view(np.uint8).reshape(-1).copy()
    out = np.zeros(int(np.prod(spec.out_shape)) * a.itemsize, dtype=np.uint8)
    SRC, DST = 1 << 20, 1 << 30
    run_jobs_on_host(copy_jobs(spec, a.itemsize, SRC, DST), {SRC: src, DST: out})
    return out.view(a.dtype).reshape(spec.out_shape)


@pytest.mark.parametrize("n", [0, 1, 5, 10, 71])
@pytest.mark.parametrize("world", [1, 2, 3, 8])
def test_tensor_split_range_closed_form(n, world):
    parts = torch.tensor_split(torch.arange(n), world)
    for r in range(world):
        start, length = tensor_split_range(n, world, r)
        assert length == parts[r].numel()
        if length:
            assert start == parts[r][0].item()


@pytest.mark.parametrize("shape,dim", [((10, 6), 0), ((10, 6), 1), ((4, 9, 5), 1), ((4, 9, 5), -1), ((7,), 0), ((3, 1, 8), 2)])
@pytest.mark.parametrize("world", [1, 2, 3, 4])
@pytest.mark.parametrize("dtype", [np.uint8, np.uint16, np.float32])
def test_split_jobs_match_oracle(shape, dim, world, dtype):
    rng = np.random.default_rng(0)
    a = rng.integers(0, 200, size=shape).astype(dtype)
    action = tp.Split(world, dim)
    for r in range(world):
        got = _run_spec_on_host(a, action.spec(shape, r))
        assert np.array_equal(got, osl.split(a, world, dim, r))


@pytest.mark.parametrize("world", [1, 2, 3, 5])
def test_chunk_and_grouped_jobs_match_oracle(world):
    rng = np.random.default_rng(1)
    a = rng.integers(0, 60000, size=(12, 30)).astype(np.uint16)
    for r in range(world):
        for dim, chunk in ((0, 3), (1, 5), (-1, 2), (-2, 4)):
            spec = tp.SplitInChunks(world, dim, chunk).spec(a.shape, r)
            assert np.array_equal(_run_spec_on_host(a, spec), osl.split_in_chunks(a, world, dim, chunk, r))
        for dim, groups, chunk in ((1, 3, 2), (1, 2, 5), (0, 3, 1), (0, 2, 3)):
            spec = tp.SplitInGroupedChunks(world, dim, groups, chunk).spec(a.shape, r)
            assert np.array_equal(_run_spec_on_host(a, spec), osl.split_in_grouped_chunks(a, world, dim, groups, chunk, r))


def test_undo_jobs_restore_the_tensor():
    rng = np.random.default_rng(2)
    a = rng.integers(0, 255, size=(6, 18)).astype(np.uint8)
    for action in (tp.Split(4, 1), tp.SplitInChunks(3, 0, 2), tp.SplitInGroupedChunks(2, 1, 3, 3)):
        world = action.world_size
        parts = [_run_spec_on_host(a, action.spec(a.shape, r)) for r in range(world)]
        full = np.zeros(a.size, dtype=np.uint8)
        FULL = 1 << 30
        bufs = {FULL: full}
        jobs = []
        for r, p in enumerate(parts):
            base = (r + 1) << 20
            bufs[base] = p.reshape(-1).copy()
            jobs += copy_jobs(action.spec(a.shape, r), 1, FULL, base, scatter=True)
        run_jobs_on_host(jobs, bufs)
        assert np.array_equal(full.reshape(a.shape), a)


def test_action_errors():
    with pytest.raises(AssertionError):
        tp.SplitInChunks(2, 0, 4).spec((10, 3), 0)  # 10 % 4 != 0, state_actions.py:80
    with pytest.raises(ValueError):
        tp.SplitInGroupedChunks(2, -1, 3, 2)
    assert tp.SplitInChunks(2, 0, 4, optional=True)(None, rank=0) is None
    with pytest.raises(IndexError):
        tp.Split(2, 3).spec((4, 4), 0)


def test_meta_tensors_pass_through_as_shapes():
    t = torch.empty(11008, 4096, device="meta", dtype=torch.bfloat16)
    assert tp.Split(2, 0)(t, rank=1).shape == (5504, 4096)
    assert tp.Split(8, 1)(t, rank=7).shape == (11008, 512)
    qkv = torch.empty(9216, 8192, device="meta")
    assert tp.SplitInChunks(2, 0, 1152)(qkv, rank=0).shape == (4608, 8192)
    parts = [tp.SplitInGroupedChunks(3, 1, 3, 64)(torch.empty(768, 2304, device="meta"), rank=r) for r in range(3)]
    assert [p.shape for p in parts] == [(768, 768)] * 3
    assert tp.SplitInGroupedChunks(3, 1, 3, 64).undo(parts).shape == (768, 2304)
    assert tp.Scale(4)(t, rank=0).shape == t.shape


def test_attr_math_matches_oracle():
    for heads, world in ((8, 3), (2, 4), (128, 2), (32, 8)):
        for r in range(world):
            assert split_num_heads(heads, rank=r, world_size=world) == osl.split_num_heads(heads, r, world)
            assert split_inner_dim(heads * 64, rank=r, num_heads=heads, world_size=world) == osl.split_inner_dim(heads * 64, r, heads, world)


# ---------------------------------------------------------------------------------------- names and rules
@pytest.mark.parametrize("case", GOLDEN["name_mapping"], ids=lambda c: c["label"])
def test_name_mapping_golden(case):
    half = len(case["module_patterns"])  # inputs first, then outputs; the split point does not matter
    cfg = tp.Config({}, {}, {}, {})
    cfg.input_rules = {re.compile(p): {} for p in case["module_patterns"][:half]}
    assert dict(get_parameter_name_mapping(case["names"], cfg)) == case["mapping"]


@pytest.mark.parametrize("case", GOLDEN["convert_state_dict"], ids=lambda c: f"W{c['world_size']}-pre{int(c['for_pretrained'])}")
def test_convert_state_dict_names_and_shapes_golden(case):
    world = case["world_size"]
    cfg = get_llama_config(SimpleNamespace(model_type="llama", hidden_size=64, num_attention_heads=8, num_key_value_heads=4),
                           [torch.device("cuda", 0)] * world)
    state = {k: torch.empty(shape, device="meta") for k, shape in case["input"].items()}
    out = tp.convert_state_dict(state, cfg, world, for_pretrained=case["for_pretrained"])
    assert set(out.keys()) == set(case["output"].keys())
    for k, shape in case["output"].items():
        assert list(out[k].shape) == shape, k
    # unmatched tensors are the same object for every rank (dispatch.py:110)
    pre = "wrapped_model." if case["for_pretrained"] else ""
    assert out[pre + "module_shards.0.model.norm.weight"] is state["model.norm.weight"]


def test_llama_7b_and_falcon_40b_tables_give_the_baseline_shapes():
    llama = SimpleNamespace(model_type="llama", hidden_size=4096, num_attention_heads=32, num_key_value_heads=32)
    state = {
        "model.layers.0.self_attn.q_proj.weight": (4096, 4096), "model.layers.0.self_attn.k_proj.weight": (4096, 4096),
        "model.layers.0.self_attn.v_proj.weight": (4096, 4096), "model.layers.0.self_attn.o_proj.weight": (4096, 4096),
        "model.layers.0.mlp.gate_proj.weight": (11008, 4096), "model.layers.0.mlp.up_proj.weight": (11008, 4096),
        "model.layers.0.mlp.down_proj.weight": (4096, 11008), "model.embed_tokens.weight": (32000, 4096),
        "lm_head.weight": (32000, 4096), "model.norm.weight": (4096,),
    }
    want = {2: [(2048, 4096)] * 3 + [(4096, 2048), (5504, 4096), (5504, 4096), (4096, 5504), (32000, 2048), (16000, 4096), (4096,)],
            8: [(512, 4096)] * 3 + [(4096, 512), (1376, 4096), (1376, 4096), (4096, 1376), (32000, 512), (4000, 4096), (4096,)]}
    for world, shapes in want.items():
        cfg = get_llama_config(llama, [torch.device("cuda", 0)] * world)
        meta = {k: torch.empty(s, device="meta", dtype=torch.bfloat16) for k, s in state.items()}
        out = tp.convert_state_dict(meta, cfg, world)
        names = get_parameter_name_mapping(state.keys(), cfg)
        assert [tuple(out[f"module_shards.0.{names[k]}"].shape) for k in state] == shapes
    falcon = SimpleNamespace(model_type="RefinedWeb", hidden_size=8192, n_head=128, n_head_kv=8, num_attention_heads=128, bias=False, alibi=False)
    cfg = get_refined_web_config(falcon, [torch.device("cuda", 0)] * 2)
    meta = {"transformer.h.0.self_attention.query_key_value.weight": torch.empty(9216, 8192, device="meta"),
            "transformer.h.0.self_attention.dense.weight": torch.empty(8192, 8192, device="meta")}
    out = tp.convert_state_dict(meta, cfg, 2)
    assert out["module_shards.0.transformer.h.0.self_attention.tp_wrapped_module.query_key_value.weight"].shape == (4608, 8192)
    assert out["module_shards.1.transformer.h.0.self_attention.tp_wrapped_module.dense.weight"].shape == (8192, 4096)
    attn = cfg.attr_rules[next(iter(cfg.attr_rules))]
    assert attn["num_kv"](8, rank=0) == 4 and attn["num_heads"](128, rank=0) == 64


def test_state_rules_first_match_wins_and_module_rules_merge():
    cfg = tp.Config(
        state_rules={r"w$": tp.Split(2, 0), r"\.w$": tp.Split(2, 1)},
        input_rules={r"^a$": {0: "split -1"}, r"a": {"0": "split -1", "x": "scale"}},
        output_rules={r"^a$": {0: "sum"}, r"^a": {0: "gather -1"}},
        attr_rules={},
    )
    out = tp.convert_state_dict({"m.w": torch.empty(4, 6, device="meta")}, cfg, 2)
    assert out["module_shards.0.m.w"].shape == (2, 6)
    assert find_matching_actions("input", "a", cfg.input_rules) == {0: "split -1", "x": "scale"}  # "0" canonicalised to 0
    with pytest.raises(ValueError):
        find_matching_actions("output", "a", cfg.output_rules)


def test_legacy_state_rules_are_accepted():
    fn = lambda t, rank: torch.tensor_split(t, 2, dim=0)[rank]  # noqa: E731
    undo = lambda ts: torch.cat(list(ts), dim=0)  # noqa: E731
    cfg = tp.Config({r"w$": fn, r"v$": (fn, undo)}, {}, {}, {})
    acts = list(cfg.state_rules.values())
    assert all(isinstance(a, tp.StateAction) for a in acts)
    t = torch.arange(8.0).reshape(4, 2)
    assert torch.equal(acts[0](t, rank=1), t[2:])
    assert torch.equal(acts[1].undo([t[:2], t[2:]]), t)
    with pytest.raises(Exception):
        acts[0].undo([t])
    with pytest.raises(Exception):
        tp.Config({r"w$": 3}, {}, {}, {})


def test_gpt2_table_uses_grouped_split():
    cfg = get_gpt2_config(SimpleNamespace(num_attention_heads=12, hidden_size=768), [torch.device("cuda", 0)] * 2)
    out = tp.convert_state_dict({"h.0.attn.c_attn.weight": torch.empty(768, 2304, device="meta"),
                                 "h.0.attn.c_attn.bias": torch.empty(2304, device="meta")}, cfg, 2)
    assert out["module_shards.1.h.0.attn.tp_wrapped_module.c_attn.weight"].shape == (768, 1152)
    assert out["module_shards.1.h.0.attn.tp_wrapped_module.c_attn.bias"].shape == (1152,)


# ---------------------------------------------------------------------------------------- model building on meta
def _toy(device="meta"):
    return nn.Sequential(nn.Embedding(1337, 64, device=device), nn.LayerNorm(64, device=device), nn.Linear(64, 128, device=device),
                         nn.ReLU(), nn.Linear(128, 10, device=device))


@pytest.mark.parametrize("world", [2, 3])
def test_meta_model_linear_attributes_follow_weights(world):
    # tests/test_basic.py:12-29 of the reference, on meta tensors
    model_tp = tp.TensorParallel(_toy(), ["cuda:0"] * world, sharded=False)
    assert len(model_tp.module_shards) == world
    seen = 0
    for name, module in model_tp.named_modules():
        if isinstance(module, nn.Linear):
            assert module.weight.shape == (module.out_features, module.in_features), name
            seen += 1
    assert seen == 2 * world
    shard0 = model_tp.module_shards[0]
    assert shard0[0].tp_wrapped_module.weight.shape == (1337, 64 // world + (64 % world > 0))
    total = sum(p.numel() for p in _toy().parameters())
    assert sum(p.numel() for p in model_tp.parameters()) >= total
    # names of the sharded model are what convert_state_dict produces (tests/test_saving.py:139-169 of the reference)
    conv = tp.convert_state_dict(_toy().state_dict(), model_tp.tensor_parallel_config, world)
    assert set(conv.keys()) == set(model_tp.state_dict().keys())
    for k, v in model_tp.state_dict().items():
        assert conv[k].shape == v.shape, k


def test_factory_and_single_device_passthrough():
    m = _toy()
    one = tp.tensor_parallel(m, ["meta"]) if False else tp.TensorParallel(m, [], sharded=False)
    assert len(one.module_shards) == 1 and one.module_shards[0] is m
    two = tp.tensor_parallel(_toy(), ["cuda:0", "cuda:0"])
    assert isinstance(two, tp.TensorParallel) and two.sharding_manager is None
    with pytest.raises(NotImplementedError):
        tp.tensor_parallel(_toy(), ["cuda:0"], distributed=True)
    with pytest.raises(AssertionError):
        tp.TensorParallel(nn.Linear(4, 4, device="meta"), ["cuda:0", "cuda:0"])  # not a container, shard.py:31-33


def test_unshard_state_dict_names_on_meta():
    model_tp = tp.TensorParallel(_toy(), ["cuda:0"] * 2, sharded=False)
    with tp.save_tensor_parallel(model_tp):
        sd = model_tp.state_dict()
    ref = _toy().state_dict()
    assert set(sd.keys()) == set(ref.keys())
    for k in ref:
        assert sd[k].shape == ref[k].shape, k
    assert any(k.startswith("module_shards.1.") for k in model_tp.state_dict())


# ---------------------------------------------------------------------------------------- failure handling
def test_collective_operation_fans_errors_out_and_recovers():
    world = 3

    def func(*xs):
        if any(x == "boom" for x in xs):
            raise RuntimeError("rank 0 failed")
        return [sum(xs)] * world

    op = CollectiveOperation(world, func, timeout=30)
    results = [None] * world

    def run(rank, value):
        try:
            results[rank] = op(value, rank)
        except Exception as e:  # noqa: BLE001
            results[rank] = e

    for values in (["boom", 1, 2], [1, 2, 3]):
        ts = [threading.Thread(target=run, args=(r, values[r])) for r in range(world)]
        [t.start() for t in ts]
        [t.join(60) for t in ts]
        if values[0] == "boom":
            assert all(isinstance(r, RuntimeError) for r in results)
        else:
            assert results == [6, 6, 6]


def test_rendezvous_timeout_does_not_hang():
    op = CollectiveOperation(2, lambda *xs: list(xs), timeout=0.2)
    with pytest.raises(threading.BrokenBarrierError):
        op(1, 0)  # the peer never arrives


def test_rank_threads_take_turns_between_rendezvous():
    """With a turn published, only one rank runs host code at a time; the turn is given up while a rank waits inside a
    collective (otherwise the next rank could never arrive) and is free again afterwards."""
    import threading
    import time

    from tensor_parallel_amd.collectives import CollectiveOperation, Turn, set_turn_lock

    world = 3
    op = CollectiveOperation(world, lambda *xs: [sum(xs)] * world, timeout=20.0)
    turn = Turn()
    running, overlaps, results = [0], [0], {}

    def critical():
        running[0] += 1
        if running[0] > 1:
            overlaps[0] += 1
        time.sleep(0.002)
        running[0] -= 1

    def worker(rank):
        turn.lock.acquire()
        set_turn_lock(turn)
        try:
            total = 0
            for step in range(5):
                critical()
                total += op(rank + step, rank)
            results[rank] = total
        finally:
            set_turn_lock(None)
            turn.lock.release()

    threads = [threading.Thread(target=worker, args=(r,)) for r in range(world)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(30)
    assert not any(t.is_alive() for t in threads)
    assert overlaps[0] == 0
    want = sum(sum(r + step for r in range(world)) for step in range(5))
    assert results == {r: want for r in range(world)}
    assert turn.lock.acquire(blocking=False)


def test_a_failing_rank_wakes_the_ranks_that_wait_in_turns():
    """Two ranks wait inside a collective; the third fails before it arrives and says so on the turn: the waiting ranks
    leave with BrokenBarrierError, and the op is usable for the next forward (a fresh turn)."""
    import threading

    from tensor_parallel_amd.collectives import CollectiveOperation, Turn, set_turn_lock

    world = 3
    op = CollectiveOperation(world, lambda *xs: [sum(xs)] * world, timeout=20.0)

    def run(fail_rank):
        turn, outcome = Turn(), {}

        def worker(rank):
            turn.lock.acquire()
            set_turn_lock(turn)
            try:
                if rank == fail_rank:
                    turn.fail()
                    outcome[rank] = "failed"
                    return
                outcome[rank] = op(rank, rank)
            except threading.BrokenBarrierError:
                outcome[rank] = "broken"
            finally:
                set_turn_lock(None)
                turn.lock.release()

        threads = [threading.Thread(target=worker, args=(r,)) for r in range(world)]
        for t in threads:
            t.start()
        for t in threads:
            t.join(10)
        assert not any(t.is_alive() for t in threads)
        return outcome

    assert run(fail_rank=2) == {0: "broken", 1: "broken", 2: "failed"}
    assert run(fail_rank=None) == {0: 3, 1: 3, 2: 3}


class _Steps(torch.nn.Module):
    """A rank's module for the greenlet tests: `steps` collectives, host work between them recorded in `log`."""

    def __init__(self, op, rank, steps, log, fail_at=None, leave_at=None):
        super().__init__()
        self.op, self.rank, self.steps, self.log, self.fail_at, self.leave_at = op, rank, steps, log, fail_at, leave_at

    def forward(self, x):
        from tensor_parallel_amd.collectives import current_sum_context, pop_sum_context, push_sum_context

        push_sum_context(("ctx", self.rank))  # the stack of contexts is a rank's own
        try:
            for step in range(self.steps):
                self.log.append((self.rank, step))
                if step == self.fail_at:
                    raise ValueError(f"rank {self.rank} fails")
                if step == self.leave_at:
                    return x
                x = x + self.op(self.rank + step, self.rank)
                assert current_sum_context() == ("ctx", self.rank)
            return x
        finally:
            pop_sum_context()


greenlets = pytest.mark.skipif(not __import__("tensor_parallel_amd.tensor_parallel", fromlist=["x"]).RANK_GREENLETS,
                               reason="the greenlet package is not there: the ranks of a device are threads")


@greenlets
def test_ranks_as_greenlets_take_turns_and_meet_in_collectives():
    from tensor_parallel_amd.collectives import CollectiveOperation, current_turn
    from tensor_parallel_amd.tensor_parallel import _apply_in_greenlets

    world, steps, log = 3, 4, []
    op = CollectiveOperation(world, lambda *xs: [sum(xs)] * world, timeout=5.0)
    mods = [_Steps(op, r, steps, log) for r in range(world)]
    for _ in range(2):  # the op is ready for the next forward
        out = _apply_in_greenlets(mods, [(10 * r,) for r in range(world)], [{}] * world, torch.device("cpu"))
        want = sum(sum(r + step for r in range(world)) for step in range(steps))
        assert out == [10 * r + want for r in range(world)]
    # a rank runs until its next collective, then the next one gets the turn: every step is entered by all ranks before
    # any rank enters the step after it
    first = log[:world * steps]
    assert [step for _, step in first] == sorted(step for _, step in first)
    assert current_turn() is None  # nothing leaks into the caller's context


@greenlets
def test_a_failing_greenlet_rank_frees_its_peers_and_the_next_forward_works():
    import threading

    from tensor_parallel_amd.collectives import CollectiveOperation
    from tensor_parallel_amd.tensor_parallel import _apply_in_greenlets

    world, log = 3, []
    op = CollectiveOperation(world, lambda *xs: [sum(xs)] * world, timeout=5.0)
    bad = [_Steps(op, r, 3, log, fail_at=1 if r == 1 else None) for r in range(world)]
    with pytest.raises(ValueError, match="rank 1 fails"):
        _apply_in_greenlets(bad, [(0,)] * world, [{}] * world, torch.device("cpu"))
    good = [_Steps(op, r, 3, log) for r in range(world)]
    assert _apply_in_greenlets(good, [(0,)] * world, [{}] * world, torch.device("cpu")) == [18] * world
    # a rank that returns without taking part in a collective its peers wait in: they are told to give up at once
    early = [_Steps(op, r, 3, log, leave_at=2 if r == 0 else None) for r in range(world)]
    with pytest.raises(threading.BrokenBarrierError):
        _apply_in_greenlets(early, [(0,)] * world, [{}] * world, torch.device("cpu"))
    assert _apply_in_greenlets(good, [(0,)] * world, [{}] * world, torch.device("cpu")) == [18] * world


@greenlets
def test_a_collective_whose_function_raises_raises_on_every_greenlet_rank():
    from tensor_parallel_amd.collectives import CollectiveOperation
    from tensor_parallel_amd.tensor_parallel import _apply_in_greenlets

    def boom(*xs):
        raise KeyError("bad values")

    op = CollectiveOperation(2, boom, timeout=5.0)
    with pytest.raises(KeyError, match="bad values"):
        _apply_in_greenlets([_Steps(op, r, 1, []) for r in range(2)], [(0,)] * 2, [{}] * 2, torch.device("cpu"))


def test_a_collective_whose_function_raises_raises_on_every_rank_in_turns():
    import threading

    from tensor_parallel_amd.collectives import CollectiveOperation, Turn, set_turn_lock

    def boom(*xs):
        raise ValueError("bad values")

    op, turn, seen = CollectiveOperation(2, boom, timeout=5.0), Turn(), {}

    def worker(rank):
        turn.lock.acquire()
        set_turn_lock(turn)
        try:
            op(rank, rank)
        except ValueError as e:
            seen[rank] = str(e)
        finally:
            set_turn_lock(None)
            turn.lock.release()

    threads = [threading.Thread(target=worker, args=(r,)) for r in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(10)
    assert seen == {0: "bad values", 1: "bad values"}


# ---------------------------------------------------------------------------------------- wrapper protocol
class _Recorder(torch.nn.Module):
    def forward(self, *args, **kwargs):
        self.seen = (args, kwargs)
        return self.result


def test_wrapper_routes_rules_by_position_and_name():
    """Input rules address positions and keyword names, output rules positions / keys / 0 for a bare tensor; a keyword
    the caller left out reaches its action as None (reference wrapper.py:31-48)."""
    from tensor_parallel_amd.wrapper import TensorParallelWrapper, apply_action, process_input, process_output

    calls = []

    def tag(label):
        def act(value, rank):
            calls.append((label, value, rank))
            return (label, value)
        return act

    args, kwargs = process_input({0: tag("a"), "mask": tag("m"), "absent": tag("n"), 5: tag("never")}, 1, 2, "x0", "x1", mask="M")
    assert args == [("a", "x0"), "x1"] and kwargs == {"mask": ("m", "M"), "absent": ("n", None)}
    assert ("never", None, 1) not in calls and all(rank == 1 for _, _, rank in calls)
    # (split, undo) pairs act with their first half
    assert apply_action("v", (tag("first"), tag("second")), rank=0, world_size=2) == ("first", "v")
    with pytest.raises(Exception, match="unexpected action"):
        apply_action(torch.zeros(2), "transpose 0", rank=0, world_size=2)

    t = torch.zeros(1)
    assert process_output(t, {0: tag("o")}, rank=0, world_size=2) == ("o", t)
    assert process_output(t, {}, rank=0, world_size=2) is t
    out = process_output((1, 2, 3), {1: tag("o")}, rank=0, world_size=2)
    assert out == (1, ("o", 2), 3) and isinstance(out, tuple)
    assert process_output([1, 2], {0: tag("o")}, rank=0, world_size=2) == [("o", 1), 2]
    d = {"logits": 7, "other": 8}
    assert process_output(d, {"logits": tag("o")}, rank=0, world_size=2) is d and d["logits"] == ("o", 7)

    inner = _Recorder()
    inner.result = (10, 20)
    inner.hidden_size = 64
    w = TensorParallelWrapper(inner, {0: tag("in")}, {0: tag("out")}, rank=1, world_size=2)
    assert w("p", q="r") == (("out", 10), 20)
    assert inner.seen == ((("in", "p"),), {"q": "r"})
    # attributes of the wrapped module are reachable through the wrapper, its own come first
    assert w.hidden_size == 64 and w.rank == 1 and w.tp_wrapped_module is inner
    with pytest.raises(AttributeError):
        w.no_such_attribute
    assert [n for n, _ in w.named_modules()] == ["", "tp_wrapped_module"]


def test_legacy_tuple_kv_cache_is_refused_for_several_ranks():
    """A tuple of key/value tensors holds one rank's heads; handing it to every rank would be silently wrong."""
    from tensor_parallel_amd.tensor_parallel import TensorParallel

    tp_model = TensorParallel.__new__(TensorParallel)
    torch.nn.Module.__init__(tp_model)
    tp_model.devices = (torch.device("cuda", 0), torch.device("cuda", 0))
    legacy = ((torch.zeros(1, 2, 3, 4), torch.zeros(1, 2, 3, 4)),)
    for name in ("past_key_values", "past_key_value", "layer_past"):
        with pytest.raises(NotImplementedError, match="Cache object"):
            tp_model.prepare_args_kwargs_for_forward(torch.zeros(1), **{name: legacy})
    tp_model.devices = (torch.device("cpu"),)
    tp_model.prepare_args_kwargs_for_forward(torch.zeros(1), past_key_values=legacy)  # one rank: nothing to split


def test_delay_init_and_output_device_arguments():
    from tensor_parallel_amd.tensor_parallel import TensorParallel

    lin = torch.nn.Linear(4, 4)
    one = TensorParallel(lin, device_ids=["cpu"], delay_init=True)
    assert one.need_delayed_init and one.module_shards[0] is lin and one.output_device_index == 0
    with pytest.raises(AssertionError):
        TensorParallel(lin, device_ids=["cpu"], output_device="cpu", output_device_index=0)
    with pytest.raises(AssertionError):
        TensorParallel(lin, device_ids=["cpu"], output_device="cuda:0")


def test_native_wrappers_validate_operands_before_any_launch():
    """Shapes, dtypes and devices the C ABI cannot see are checked in Python: a wrong operand raises instead of being
    dereferenced by a kernel. Runs without a GPU: every check fires before the library is reached."""
    meta = torch.device("meta")
    x = torch.empty(4, 64, dtype=torch.float16, device=meta)

    class OnGpu(torch.Tensor):
        """A tensor that claims to live on cuda:0, for the device checks."""

    def fake(shape, dtype, device="cuda:0"):
        t = torch.empty(shape, dtype=dtype, device=meta)
        t.__class__ = OnGpu
        OnGpu.device = property(lambda self: self._dev)
        t._dev = torch.device(device)
        return t

    xg = fake((4, 64), torch.float16)
    wq = fake((32, 64), torch.int8)
    sc = fake((32,), torch.float32)
    with pytest.raises(_native.NativeLibraryError):
        _native.linear_w8(x, wq, sc, None, None)  # x not on a HIP device
    with pytest.raises(ValueError, match="input features"):
        _native.linear_w8(xg, fake((32, 48), torch.int8), sc, None, None)
    with pytest.raises(ValueError, match="scale must have shape"):
        _native.linear_w8(xg, wq, fake((16,), torch.float32), None, None)
    with pytest.raises(ValueError, match="wq on"):
        _native.linear_w8(xg, fake((32, 64), torch.int8, "cuda:1"), sc, None, None)
    with pytest.raises(ValueError, match="bias must have shape"):
        _native.linear_w8(xg, wq, sc, None, None, bias=fake((31,), torch.float16))
    with pytest.raises(ValueError, match="bias on"):
        _native.linear_w8(xg, wq, sc, None, None, bias=fake((32,), torch.float16, "cuda:1"))
    with pytest.raises(TypeError):
        _native.linear_w8(fake((4, 64), torch.float32), wq, sc, None, None)
    w = fake((32, 64), torch.float16)
    with pytest.raises(ValueError, match="w on"):
        _native.linear(xg, fake((32, 64), torch.float16, "cuda:1"))
    with pytest.raises(ValueError, match="bias"):
        _native.linear(xg, w, bias=fake((32,), torch.float16, "cuda:1"))
    with pytest.raises(ValueError, match="wu on"):
        _native.swiglu_up(xg, w, fake((32, 64), torch.float16, "cuda:1"))
    q = fake((1, 2, 3, 64), torch.float16)
    with pytest.raises(ValueError, match="k on"):
        _native.attention(q, fake((1, 2, 3, 64), torch.float16, "cuda:1"), fake((1, 2, 3, 64), torch.float16))


def test_infer_sharded_device_map_names_and_devices():
    """Every parameter, buffer and tied alias of a tensor-parallel model maps to the device of the rank whose index its
    name carries (reference dispatch.py:35-72)."""
    from tensor_parallel_amd.dispatch import infer_sharded_data_device_id, infer_sharded_device_map

    assert infer_sharded_data_device_id("wrapped_model.module_shards.3.model.layers.0.mlp.tp_wrapped_module.up_proj.weight") == 3
    assert infer_sharded_data_device_id("_sanity_check_params.1") == 1
    assert infer_sharded_data_device_id("wrapped_model.sharding_manager.flat_shards.2") == 2
    assert infer_sharded_data_device_id("module_shards.10.bias") == 10
    with pytest.raises(KeyError):
        infer_sharded_data_device_id("model.layers.0.weight")

    class Shard(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.emb = torch.nn.Embedding(8, 4)
            self.head = torch.nn.Linear(4, 8, bias=False)
            self.head.weight = self.emb.weight  # tied
            self.register_buffer("steps", torch.zeros(1))

    class Model(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.module_shards = torch.nn.ModuleList([Shard(), Shard()])
            self._sanity_check_params = torch.nn.ParameterList([torch.nn.Parameter(torch.empty(0)) for _ in range(2)])
            self.devices = (torch.device("cuda", 0), torch.device("cuda", 1))

    dm = infer_sharded_device_map(Model())
    want = {}
    for r in range(2):
        dev = torch.device("cuda", r)
        want.update({f"module_shards.{r}.emb.weight": dev, f"module_shards.{r}.head.weight": dev,
                     f"module_shards.{r}.steps": dev, f"_sanity_check_params.{r}": dev})
    assert dm == want


def test_reference_import_name_serves_the_same_objects():
    """`import tensor_parallel as tp`, the reference's import name, and its submodule paths."""
    import tensor_parallel as ref_name
    from tensor_parallel.slicing_configs import get_llama_config as by_ref_path
    from tensor_parallel.state_actions import Split as split_by_ref_path

    for name in ("Config", "TensorParallel", "tensor_parallel", "convert_state_dict", "infer_sharded_device_map",
                 "save_tensor_parallel", "Sharded", "StateAction"):
        assert getattr(ref_name, name) is getattr(tp, name)
    assert by_ref_path is get_llama_config and split_by_ref_path is tp.Split
    assert ref_name.tensor_parallel.__module__ == "tensor_parallel_amd.factory"


def test_convolution_layers_get_no_rule_and_a_warning(caplog):
    """The automatic config leaves convolution layers whole on every rank (the reference's conv rules,
    autoconfig.py:40-78, are not carried) instead of refusing the model."""
    import logging

    from tensor_parallel_amd.autoconfig import get_default_config

    model = nn.Sequential(nn.Conv1d(4, 8, 3), nn.Flatten(), nn.Linear(16, 6))
    with caplog.at_level(logging.WARNING):
        cfg = get_default_config(model, [torch.device("cuda", 0)] * 2)
    assert any("convolution" in r.getMessage() for r in caplog.records)
    patterns = [p.pattern for p in cfg.state_rules]
    assert any(p.startswith("^2.") for p in patterns) and not any(p.startswith("^0.") for p in patterns)


# ---------------------------------------------------------------------------------------- the sum folded into a Linear
def test_sum_op_hands_out_only_running_sums_in_rank_order(monkeypatch):
    """What a rank's last Linear may add in its epilogue: with two ranks whatever the other rank has handed in; with more,
    the running sum over ranks 0 .. r-1 and nothing else, so that the result stays the rank-ordered stepwise sum. The
    reduction then adds only what the widest value lacks."""
    from tensor_parallel_amd import _native, collectives
    from tensor_parallel_amd.collectives import DeviceAllReduce, Turn, set_turn_lock

    summed = []

    def host_sum(parts, accum=0, out=None):
        summed.append([float(p[0]) for p in parts])
        total = parts[0].clone()
        for p in parts[1:]:
            total = total + p
        return total

    monkeypatch.setattr(_native, "reduce_partials", host_sum)
    monkeypatch.setattr(collectives, "FUSE_SUM", True)
    t = [torch.full((2,), float(10 ** r)) for r in range(4)]  # 1, 10, 100, 1000: a sum shows which ranks it covers
    op = DeviceAllReduce(3)
    assert op.addend_for(1) is None  # no turn: ranks are not taking turns on one device
    set_turn_lock(Turn())
    try:
        assert op.addend_for(1) is None  # nothing has been handed in
        op._inputs, op._masks = [t[0], None, None], [0b001, 0, 0]
        got = op.addend_for(1)
        assert got is not None and got[0] is t[0] and got[1] == 0b001
        assert op.addend_for(2) is None  # rank 1 has not arrived
        s01 = t[0] + t[1]
        op._inputs, op._masks = [t[0], s01, None], [0b001, 0b011, 0]
        got = op.addend_for(2)
        assert got[0] is s01 and got[1] == 0b011
        # rank 1 arrived first: neither rank 0 (nothing below it) nor rank 2 (rank 1's value is not a sum from rank 0 on)
        op._inputs, op._masks = [None, t[1], None], [0, 0b010, 0]
        assert op.addend_for(0) is None and op.addend_for(2) is None
        # the reduction: a value that covers ranks 0 and 1 and rank 2's own partial -> only those two are added, in order
        op._masks = [0b001, 0b011, 0b100]
        out = op._reduce(t[0], s01, t[2])
        assert summed[-1] == [11.0, 100.0] and float(out[0][0]) == 111.0 and len(out) == 3
        # a value that covers every rank: nothing is launched
        s012 = s01 + t[2]
        op._masks = [0b001, 0b011, 0b111]
        n = len(summed)
        out = op._reduce(t[0], s01, s012)
        assert len(summed) == n and float(out[1][0]) == 111.0
        # nobody folded anything: the plain rank-ordered sum
        op._masks = [0b001, 0b010, 0b100]
        op._reduce(t[0], t[1], t[2])
        assert summed[-1] == [1.0, 10.0, 100.0]
        # two ranks: either order
        two = DeviceAllReduce(2)
        two._inputs, two._masks = [None, t[1]], [0, 0b10]
        got = two.addend_for(0)
        assert got[0] is t[1] and got[1] == 0b10
        two._masks = [0b11, 0b10]
        n = len(summed)
        out = two._reduce(t[0] + t[1], t[1])
        assert len(summed) == n and float(out[0][0]) == 11.0
        # F32 accumulation is another arithmetic: never folded
        assert DeviceAllReduce(2, accum=_native.ACCUM_F32).fusable is False
    finally:
        set_turn_lock(None)


def test_int8_step_refuses_host_tensors_and_leaves_host_modules_alone():
    """The quantiser computes on the device only; Linears whose weights live on the host are not touched."""
    from tensor_parallel_amd import _native
    from tensor_parallel_amd.int8 import ShardLinearW8, quantize_linears_, quantize_rows

    with pytest.raises(_native.NativeLibraryError):
        quantize_rows(torch.randn(4, 16, dtype=torch.float16))
    block = nn.Sequential(nn.Linear(16, 8), nn.ReLU(), nn.Linear(8, 4)).to(torch.float16)
    assert quantize_linears_(block) == 0
    assert not any(isinstance(m, ShardLinearW8) for m in block.modules())
    with pytest.raises(TypeError):
        ShardLinearW8(torch.zeros(4, 16, dtype=torch.int8), torch.ones(4), torch.zeros(0, dtype=torch.int32),
                      torch.zeros(4, 0), None, torch.float32)


def test_bench_refuses_more_than_one_gpu():
    """The benchmark measures one GPU's share: asking for more exits with a message that says so, before anything is
    imported or measured."""
    import subprocess
    import sys

    root = Path(__file__).resolve().parents[1]
    res = subprocess.run([sys.executable, str(root / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert res.returncode == 2 and res.stdout == ""
    assert "--gpus above 1 is not supported" in res.stderr


def test_graph_capture_needs_a_hip_device():
    """`tp.graphs.capture` records kernels of one HIP device: a host module is refused before anything runs."""
    module = torch.nn.Linear(8, 8)
    with pytest.raises(ValueError, match="one HIP device"):
        tp.graphs.capture(module, torch.zeros(2, 8))
