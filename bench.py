"""Benchmark of the per-rank hot path on one MI355X.

Workload (BASELINE.json configs[1]): the rank-0 shard at W = 2 of a Llama-7B MLP, d = 4096, shard width 5504,
bf16, M = 4096 tokens. One step = fused gate/up GEMM + SiLU gate, then the down-projection GEMM (the row-parallel
partial) whose epilogue adds the other rank's partial (the on-device 2-partial sum). Prints ONE JSON line.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

D_MODEL, FFN_SHARD = 4096, 5504
PEAK_BF16_TFLOPS = 2500.0
PEAK_HBM_GBS = 8000.0
# Fabric bytes per launch of the fused gate/up GEMM at M = 4096 come from two rocprofv3 --pmc runs of this script
# (FETCH_SIZE, WRITE_SIZE, each scaled by what the same counter reads for the slicing kernel's known 13.476 GB); a
# counter cannot be read from inside the script, so the figure is taken from the committed summary of those runs.
PMC_SUMMARY = ROOT / "profiles" / "pmc_fetch_write_bench_kernels.txt"
PMC_ROW = "gate/up M=4096"


def measured_traffic_bytes():
    """fetch + write MB per launch of the row `PMC_ROW` of the PMC summary, in bytes; None when there is no such row."""
    try:
        for line in PMC_SUMMARY.read_text().splitlines():
            if PMC_ROW in line and line.lstrip().startswith("gemm_"):
                cols = line.split(PMC_ROW)[1].split()
                return (float(cols[1]) + float(cols[2])) * 1e6  # n, fetch MB, write MB, ...
    except (OSError, ValueError, IndexError):
        pass
    return None


def cpu_baseline(tokens: int = 4096, seconds_budget: float = 12.0) -> dict:
    """The reference path on the host, restated by the oracle, on bounded samples of the same workloads:
    `value`: both rank shards of the MLP on two threads at the benchmark's token count, torch CPU ops in bf16, then the
             sum (device_ids=['cpu','cpu'] in the reference: tensor_parallel.py:237-287);
    `decode_m1`: the same step on one token;
    `slicing`: state actions + the copy that installs the shard (shard.py:160) over the seven split tensors of one
             Llama-2-7B decoder layer, every rank at W = 2, in GB/s read + written (32 such layers and the two
             embedding-sized matrices make up the dict the GPU figure is quoted on)."""
    import numpy as np
    import torch

    from oracle import shard_forward as ofw
    from oracle import slicing as osl

    g = torch.Generator().manual_seed(0)
    shards = []
    for _ in range(2):
        wg, wu = ((torch.randn(FFN_SHARD, D_MODEL, generator=g) * 0.02).bfloat16() for _ in range(2))
        wd = (torch.randn(D_MODEL, FFN_SHARD, generator=g) * 0.02).bfloat16()
        shards.append((wg, wu, wd))

    def timed(m, budget):
        x = torch.randn(m, D_MODEL, generator=torch.Generator().manual_seed(1)).bfloat16()
        ofw.run_mlp_shards(x, shards, threads=True)  # warm
        reps, t0 = 0, time.perf_counter()
        while True:
            ofw.run_mlp_shards(x, shards, threads=True)
            reps += 1
            dt = time.perf_counter() - t0
            if dt > budget:
                return reps, dt

    reps, dt = timed(tokens, seconds_budget)
    d_reps, d_dt = timed(1, 3.0)

    # slicing: one decoder layer, both ranks
    rng = np.random.default_rng(0)
    layer = {name: rng.integers(0, 1 << 16, size=shape, dtype=np.uint16)
             for name, shape in (("q", (4096, 4096)), ("k", (4096, 4096)), ("v", (4096, 4096)), ("o", (4096, 4096)),
                                 ("gate", (11008, 4096)), ("up", (11008, 4096)), ("down", (4096, 11008)))}
    world = 2

    def slice_layer():
        moved = 0
        for r in range(world):
            for name, t in layer.items():
                if name in ("q", "k", "v"):
                    out = osl.split_in_chunks(t, world, 0, 128, r)
                elif name == "o":
                    out = osl.split_in_chunks(t, world, 1, 128, r)
                elif name == "down":
                    out = osl.split(t, world, 1, r)
                else:
                    out = osl.split(t, world, 0, r)
                moved += 2 * out.nbytes
        return moved

    slice_layer()
    s_reps, s_bytes, t0 = 0, 0, time.perf_counter()
    while time.perf_counter() - t0 < 4.0:
        s_bytes += slice_layer()
        s_reps += 1
    s_dt = time.perf_counter() - t0
    return {
        "value": tokens * reps / dt,
        "unit": "tokens/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"{reps} forwards of {tokens} tokens through both W=2 shards (2 threads) + sum, bf16 on host, {dt:.1f} s",
        "host_cpus": os.cpu_count(),
        "torch": torch.__version__,
        "decode_m1": {"value": d_reps / d_dt, "unit": "tokens/s", "us_per_step": d_dt / d_reps * 1e6,
                      "sample": f"{d_reps} forwards of 1 token, same shards and threads, {d_dt:.1f} s"},
        "slicing": {"value": s_bytes / s_dt / 1e9, "unit": "GB/s read + written", "cores": 1,
                    "sample": f"{s_reps} passes over the 7 split tensors of one Llama-2-7B decoder layer (404.8 MB), both ranks at W=2: "
                              f"state action + contiguous copy in numpy, {s_dt:.1f} s; the full dict is 32 such layers + 2 x 262 MB"},
    }


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--tokens", type=int, default=4096)
    ap.add_argument("--settle", type=int, default=240, help="untimed steps before the counted warm-up (clock settling)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra", action="store_true")
    ap.add_argument("--no-model-graphs", action="store_true",
                    help="leave out the two figures that replay a whole model forward as a HIP graph (counter-collecting profiler runs)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU's share of the tensor-parallel layer; --gpus above 1 is not supported "
              "(this package has no inter-GPU collective).", file=sys.stderr)
        return 2

    import torch

    from tensor_parallel_amd import _native

    if not _native.available():
        print(f"HIP library missing: {_native.load_error()}", file=sys.stderr)
        return 1
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    M = args.tokens
    g = torch.Generator(device=dev).manual_seed(0)

    def w(shape):
        return (torch.randn(shape, generator=g, device=dev) * 0.02).to(torch.bfloat16)

    n_sets = 3  # weight sets rotated so that HBM-bound shapes are not served from the 256 MB Infinity Cache
    sets = [(w((FFN_SHARD, D_MODEL)), w((FFN_SHARD, D_MODEL)), w((D_MODEL, FFN_SHARD))) for _ in range(n_sets)]
    x = torch.randn(M, D_MODEL, generator=torch.Generator(device=dev).manual_seed(1), device=dev).to(torch.bfloat16)
    other = torch.randn(M, D_MODEL, generator=g, device=dev).to(torch.bfloat16)  # the other rank's partial

    out_buf = torch.empty(M, D_MODEL, device=dev, dtype=torch.bfloat16)

    def step(i, ev=None):
        wg, wu, wd = sets[i % n_sets]
        if ev is not None:
            ev[0].record()
        h = _native.swiglu_up(x, wg, wu)
        if ev is not None:
            ev[1].record()
        # the down projection adds the other rank's partial in its epilogue: product rounded to bf16, fp32 add, rounded
        # again, i.e. the 2-partial `sum` of the reference in the same launch
        return _native.linear(h, wd, addend=other, out=out_buf)

    # Settling run, outside the counted warm-up: the part's power management needs about a hundred launches (50 ms) of
    # this load before its clock stops moving (the first launches run at boost clock, the next ones over-correct), and
    # every rotated weight set has to have been touched. Without it a short run times the transient, not the kernel.
    for i in range(args.settle):
        step(i)
    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(i, events[i])
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt / args.steps * 1e3
    tokens_per_s = M * args.steps / dt

    # dominant kernel: the fused gate/up GEMM (two thirds of the FLOPs). Events sit on the stream the kernels
    # are launched on (torch's current stream is handed to the library).
    up_ms = sum(a.elapsed_time(b) for a, b in events) / len(events)
    up_flops = 4.0 * M * D_MODEL * FFN_SHARD
    mfma_bound = M >= 256
    if mfma_bound:
        achieved = up_flops / (up_ms * 1e-3) / 1e12
        roofline = {"bound": "mfma", "achieved": achieved, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                    "frac": achieved / PEAK_BF16_TFLOPS, "traffic": measured_traffic_bytes() if M == 4096 else None,
                    "traffic_unit": "bytes per launch (L2<->fabric, rocprofv3 --pmc, read from profiles/pmc_fetch_write_bench_kernels.txt; algorithmic 168.8e6)",
                    "kernel": "gemm_direct4_kernel<bf16, swiglu> (tpamd_swiglu_up)", "avg_launch_ms": up_ms,
                    "algorithmic_flops_per_launch": up_flops}
    else:
        up_bytes = 2.0 * FFN_SHARD * D_MODEL * 2 + M * D_MODEL * 2 + M * FFN_SHARD * 2
        achieved = up_bytes / (up_ms * 1e-3) / 1e9
        roofline = {"bound": "hbm", "achieved": achieved, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                    "frac": achieved / PEAK_HBM_GBS, "traffic": None,
                    "kernel": "skinny_kernel<bf16, swiglu> (tpamd_swiglu_up)", "avg_launch_ms": up_ms,
                    "algorithmic_bytes_per_launch": up_bytes}

    out = {
        "metric": "rank-0 shard tokens/s + % MFMA/HBM roofline, Llama-7B-shape layer W=2",
        "value": tokens_per_s,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": f"llama7b_mlp_rank0_shard_w2_m{M}_bf16", "d_model": D_MODEL, "ffn_shard": FFN_SHARD,
                   "tokens": M, "step": "swiglu_up + down projection with the 2-partial sum in its epilogue", "settle_steps": args.settle, "weights": "N(0,0.02) seed 0", "weight_sets_rotated": n_sets},
        "roofline": roofline,
    }
    if not args.no_extra:
        out["extra"] = extra_measurements(torch, _native, dev, sets, other, model_graphs=not args.no_model_graphs)
        out["extra"]["copy_bandwidth"] = copy_bandwidth(torch, _native, dev)
        add_copy_fractions(out["extra"], out["extra"]["copy_bandwidth"]["GBps"])
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(M)
    print(json.dumps(out), flush=True)
    return 0


def copy_bandwidth(torch, _native, dev) -> dict:
    """What a plain copy reaches on this part, as the second yardstick beside the published 8 TB/s: 1 GiB moved to another
    1 GiB buffer (bytes read + written per second) by torch's `copy_` and by the library's region mover as one job of
    8192 rows; `GBps` is the better of the two."""
    n = 1 << 30
    src = torch.empty(n, dtype=torch.uint8, device=dev).random_()
    dst = torch.empty_like(src)
    t_torch = _time_us(torch, lambda i: dst.copy_(src), 3, 10)
    job = [(src.data_ptr(), dst.data_ptr(), 8192, n // 8192, n // 8192, n // 8192)]
    t_lib = _time_us(torch, lambda i: _native.run_copy_jobs(job, dev), 3, 10)
    torch.cuda.synchronize()
    assert torch.equal(src[-4096:], dst[-4096:])
    both = {"torch_copy_GBps": 2.0 * n / t_torch / 1e3, "region_mover_GBps": 2.0 * n / t_lib / 1e3}
    return {**both, "GBps": max(both.values()), "bytes_each_way": n}


def add_copy_fractions(tree, copy_gbps: float) -> None:
    """Beside every `hbm_frac` (of the published 8 TB/s) the same figure as a fraction of the measured copy bandwidth."""
    if isinstance(tree, dict):
        if "hbm_frac" in tree and "GBps" in tree:
            tree["copy_frac"] = tree["GBps"] / copy_gbps
        for value in tree.values():
            add_copy_fractions(value, copy_gbps)


def _graph_us(torch, fn, per=30, reps=10):
    """Average time of one fn(i) inside a HIP graph of `per` calls (captured on the stream that ran the warm-up calls)."""
    global _SIDE_STREAM
    if _SIDE_STREAM is None:  # one capture stream for the whole run: the library keeps a scratch buffer per stream
        _SIDE_STREAM = torch.cuda.Stream()
    side = _SIDE_STREAM
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for i in range(3):
            fn(i)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        for i in range(per):
            fn(i)
    return _time_us(torch, lambda i: graph.replay(), 3, reps) / per


_SIDE_STREAM = None


def _time_us(torch, fn, warm, iters):
    for i in range(warm):
        fn(i)
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for i in range(iters):
        fn(i)
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / iters * 1e3


def extra_measurements(torch, _native, dev, sets, other, model_graphs: bool = True) -> dict:
    """The other two targets of the same path, reported beside the headline: decode (M = 1, HBM-bound) and
    state-dict slicing (every split tensor of a Llama-2-7B-shaped dict, all ranks' shards, W = 2, HBM-bound)."""
    extra = {}
    n_sets = len(sets)
    for m in (1, 4, 16, 64):
        x = torch.randn(m, D_MODEL, device=dev).to(torch.bfloat16)

        def fn(i):
            wg, wu, wd = sets[i % n_sets]
            return _native.linear(_native.swiglu_up(x, wg, wu), wd)

        by = 3.0 * FFN_SHARD * D_MODEL * 2 + 38400.0 * m
        us = _time_us(torch, fn, 10, 100)
        entry = {"us_per_step": us, "tokens_per_s": m / us * 1e6, "GBps": by / us / 1e3,
                 "hbm_frac": by / us / 1e3 / PEAK_HBM_GBS, "algorithmic_bytes": by, "launch": "eager (one C-ABI call per kernel)"}
        # the same step captured in a HIP graph (30 steps per graph, weight sets rotated inside it): what a serving
        # loop that replays graphs sees, without the host's per-launch cost
        try:
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for i in range(3):
                    fn(i)
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            graph, per = torch.cuda.CUDAGraph(), 30
            with torch.cuda.graph(graph, stream=side):  # the stream that ran the warm-up calls
                for i in range(per):
                    fn(i)
            gus = _time_us(torch, lambda i: graph.replay(), 3, 10) / per
            entry["graph"] = {"us_per_step": gus, "tokens_per_s": m / gus * 1e6, "GBps": by / gus / 1e3,
                              "hbm_frac": by / gus / 1e3 / PEAK_HBM_GBS}
            del graph
        except Exception as e:  # noqa: BLE001 - the eager figure stands on its own
            entry["graph"] = {"error": str(e)[:200]}
        extra[f"decode_m{m}"] = entry
    # the same shard at M = 512 (the prefill size of the configuration list between decode and the headline)
    x512 = torch.randn(512, D_MODEL, device=dev).to(torch.bfloat16)

    def fn512(i):
        wg, wu, wd = sets[i % n_sets]
        return _native.linear(_native.swiglu_up(x512, wg, wu), wd)

    us = _time_us(torch, fn512, 10, 50)
    flops = 6.0 * 512 * D_MODEL * FFN_SHARD
    extra["prefill_m512"] = {"us_per_step": us, "tokens_per_s": 512 / us * 1e6, "TFLOPs": flops / us / 1e6,
                             "mfma_frac": flops / us / 1e6 / PEAK_BF16_TFLOPS, "algorithmic_flops": flops,
                             "step": "swiglu_up + down (tiling and K split chosen by the library: 256x256 / 2 and 128x128 / 4)"}
    for m in (1, 16, 32, 64):
        extra[f"w8_decode_m{m}"] = w8_decode(torch, _native, dev, m)
    extra["w8_prefill_m1024"] = w8_decode(torch, _native, dev, 1024, graph=False)
    extra["reduce_2partials_m4096"] = reduce_extra(torch, _native, dev, other)
    extra["attention_falcon40b_shard"] = attention_extra(torch, _native, dev)
    extra["c4_decode_step"] = falcon_attention_decode_step(torch, _native, dev)
    extra["c4_prefill_step"] = falcon_attention_prefill_step(torch, _native, dev)
    extra.update(api_level_extras(torch, dev, model_graphs))

    from types import SimpleNamespace

    from tensor_parallel_amd.slicing import BatchSlicer
    from tensor_parallel_amd.slicing_configs import get_llama_config

    layers = 32
    state = {}
    for layer in range(layers):
        p = f"model.layers.{layer}."
        for name, shape in (("self_attn.q_proj", (4096, 4096)), ("self_attn.k_proj", (4096, 4096)), ("self_attn.v_proj", (4096, 4096)),
                            ("self_attn.o_proj", (4096, 4096)), ("mlp.gate_proj", (11008, 4096)), ("mlp.up_proj", (11008, 4096)),
                            ("mlp.down_proj", (4096, 11008))):
            state[p + name + ".weight"] = torch.empty(shape, device=dev, dtype=torch.bfloat16).normal_(0, 0.02)
    state["model.embed_tokens.weight"] = torch.empty((32000, 4096), device=dev, dtype=torch.bfloat16).normal_(0, 0.02)
    state["lm_head.weight"] = torch.empty((32000, 4096), device=dev, dtype=torch.bfloat16).normal_(0, 0.02)
    for world in (2, 4, 8):
        cfg = get_llama_config(SimpleNamespace(model_type="llama", hidden_size=4096, num_attention_heads=32, num_key_value_heads=32), [dev] * world)
        batch = BatchSlicer(dev)
        keep = []
        for r in range(world):
            for name, t in state.items():
                action = next(a for p, a in cfg.state_rules.items() if p.search(name))
                keep.append(batch.add(t, action.spec(tuple(t.shape), r)))
        plan = batch.build()
        us = _time_us(torch, lambda i: plan.run(), 2, 10)
        moved = 2.0 * plan.nbytes
        extra[f"slicing_w{world}"] = {"tensors": len(state), "shards": len(keep), "bytes_read_plus_written": moved, "us_per_launch": us,
                                      "GBps": moved / us / 1e3, "hbm_frac": moved / us / 1e3 / PEAK_HBM_GBS}
        torch.cuda.synchronize()
        if world == 2:
            # the way back (what TensorParallel.state_dict does per tensor): action.undo on the two rank shards of every
            # split tensor, one launch of the region mover each, host time of the 226 calls included
            plan.run()
            torch.cuda.synchronize()
            names = list(state)
            actions = [next(a for p, a in cfg.state_rules.items() if p.search(name)) for name in names]

            def unshard(i):
                for j, action in enumerate(actions):
                    action.undo([keep[j], keep[len(names) + j]])

            us_u = _time_us(torch, unshard, 1, 3)
            extra["unshard_w2"] = {"tensors": len(names), "bytes_read_plus_written": moved, "us_per_dict": us_u, "GBps": moved / us_u / 1e3,
                                   "hbm_frac": moved / us_u / 1e3 / PEAK_HBM_GBS,
                                   "what": "StateAction.undo over the W=2 shards of every split tensor of the same dict (one launch per tensor)"}
        batch.close()
        del keep, plan, batch
    # the "gather -1" rule of the output head at BASELINE config 1: two ranks' halves of [2, 64, 50272] fp32 logits, every
    # rank handed its own copy of the whole, one launch
    from tensor_parallel_amd.slicing import concat_dim

    halves = [torch.randn(2, 64, 25136, device=dev) for _ in range(2)]
    us = _time_us(torch, lambda i: concat_dim(halves, -1, copies=2), 5, 30)
    moved = float(2 * 2 * halves[0].numel() * 4 + 2 * 2 * halves[0].numel() * 4)  # both halves read for each copy, two whole copies written
    extra["gather_c1_logits_w2"] = {"us_per_call": us, "bytes_read_plus_written": moved, "GBps": moved / us / 1e3,
                                    "hbm_frac": moved / us / 1e3 / PEAK_HBM_GBS,
                                    "what": "DeviceAllGather's concatenation for two ranks (2 x [2, 64, 25136] fp32 -> two copies of [2, 64, 50272]), host call included"}
    return extra


def attention_extra(torch, _native, dev) -> dict:
    """Rank-local attention core at the shape of a Falcon-40B rank shard at W = 2 (64 query heads, 4 key/value heads,
    head_dim 64): decode batch 8 on 2048 and on 8192 cached keys (bound by reading K and V once) and causal prefill of
    1024 positions at batch 8 (bound by the matrix pipe; flops counted for the visible half of the score matrix)."""
    g = torch.Generator(device=dev).manual_seed(0)
    out = {}
    q = torch.randn(8, 64, 1, 64, device=dev, generator=g).to(torch.bfloat16)

    def decode(keys, n_caches):
        # more caches than the 256 MB of last-level cache hold, taken in turn
        caches = [(torch.randn(8, 4, keys, 64, device=dev, generator=g).to(torch.bfloat16),
                   torch.randn(8, 4, keys, 64, device=dev, generator=g).to(torch.bfloat16)) for _ in range(n_caches)]

        def dec(i):
            k, v = caches[i % len(caches)]
            return _native.attention(q, k, v, causal=True)

        by = 2.0 * 8 * 4 * keys * 64 * 2
        us = _time_us(torch, dec, 10, 100)
        entry = {"us_per_call": us, "GBps": by / us / 1e3, "hbm_frac": by / us / 1e3 / PEAK_HBM_GBS, "algorithmic_bytes": by, "launch": "eager"}
        try:
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for i in range(3):
                    dec(i)
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            graph, per = torch.cuda.CUDAGraph(), 32
            with torch.cuda.graph(graph, stream=side):  # the stream that ran the warm-up calls
                for i in range(per):
                    dec(i)
            gus = _time_us(torch, lambda i: graph.replay(), 3, 10) / per
            entry["graph"] = {"us_per_call": gus, "GBps": by / gus / 1e3, "hbm_frac": by / gus / 1e3 / PEAK_HBM_GBS}
            del graph
        except Exception as e:  # noqa: BLE001
            entry["graph"] = {"error": str(e)[:200]}
        return entry

    out["decode_b8_kv2048"] = decode(2048, 8)
    out["decode_b8_kv8192"] = decode(8192, 6)
    q = torch.randn(8, 64, 1024, 64, device=dev, generator=g).to(torch.bfloat16)
    k = torch.randn(8, 4, 1024, 64, device=dev, generator=g).to(torch.bfloat16)
    v = torch.randn(8, 4, 1024, 64, device=dev, generator=g).to(torch.bfloat16)
    us = _time_us(torch, lambda i: _native.attention(q, k, v, causal=True), 5, 30)
    flops = 4.0 * 8 * 64 * 1024 * 1024 * 64 * 0.5
    out["prefill_b8_s1024"] = {"us_per_call": us, "TFLOPs": flops / us / 1e6, "mfma_frac": flops / us / 1e6 / PEAK_BF16_TFLOPS,
                               "algorithmic_flops": flops}
    return out


def falcon_attention_decode_step(torch, _native, dev) -> dict:
    """BASELINE config 4, decode, as one step of the rank-0 attention shard of a Falcon-40B-shape layer at W = 2: fused
    QKV projection [4608 x 8192] on 8 new tokens, rotary embedding + hand-over to the rank-local cache (position 2047 of
    2048), attention core over the 2048 cached positions (64 query heads on 4 key/value heads of 64), dense projection
    [8192 x 4096] (the row-parallel partial). Algorithmic bytes: both weights and the key/value cache once; three weight
    and cache sets are rotated."""
    B, L, Hq, Hkv, D, d_model = 8, 2048, 64, 4, 64, 8192
    per = Hq // Hkv
    g = torch.Generator(device=dev).manual_seed(0)
    n_sets = 3
    sets = []
    for _ in range(n_sets):
        wqkv = (torch.randn((Hq + 2 * Hkv) * D, d_model, device=dev, generator=g) * 0.02).to(torch.bfloat16)
        wdense = (torch.randn(d_model, Hq * D, device=dev, generator=g) * 0.02).to(torch.bfloat16)
        kc = torch.randn(B, Hkv, L, D, device=dev, generator=g).to(torch.bfloat16)
        vc = torch.randn(B, Hkv, L, D, device=dev, generator=g).to(torch.bfloat16)
        sets.append((wqkv, wdense, kc, vc))
    x = torch.randn(B, 1, d_model, device=dev, generator=g).to(torch.bfloat16)
    inv = 1.0 / (10000.0 ** (torch.arange(0, D, 2, device=dev, dtype=torch.float32) / D))
    ang = torch.cat([(L - 1) * inv, (L - 1) * inv])[None, None, :]
    cos, sin = ang.cos().to(torch.bfloat16), ang.sin().to(torch.bfloat16)
    q_rot = torch.empty(B, Hq, 1, D, device=dev, dtype=torch.bfloat16)
    attn = torch.empty(B, 1, Hq, D, device=dev, dtype=torch.bfloat16)

    def separate(i):
        wqkv, wdense, kc, vc = sets[i % n_sets]
        fused = _native.linear(x, wqkv).view(B, 1, Hkv, per + 2, D)
        _native.rope_append(fused[:, :, :, :per], fused[:, :, :, per], fused[:, :, :, per + 1], cos, sin, kc, vc, L - 1, q_out=q_rot)
        _native.attention(q_rot, kc, vc, causal=True, out=attn)
        return _native.linear(attn.view(B, Hq * D), wdense)

    def folded(i):
        wqkv, wdense, kc, vc = sets[i % n_sets]
        fused = _native.linear(x, wqkv).view(B, 1, Hkv, per + 2, D)
        _native.attention_decode_rope(fused[:, :, :, :per], fused[:, :, :, per], fused[:, :, :, per + 1], cos, sin, kc, vc, L - 1, out=attn)
        return _native.linear(attn.view(B, Hq * D), wdense)

    by = 2.0 * ((Hq + 2 * Hkv) * D * d_model + d_model * Hq * D) + 2.0 * B * Hkv * L * D * 2

    def measure(fn, step):
        us = _time_us(torch, fn, 10, 100)
        entry = {"us_per_step": us, "tokens_per_s": B / us * 1e6, "GBps": by / us / 1e3, "hbm_frac": by / us / 1e3 / PEAK_HBM_GBS,
                 "algorithmic_bytes": by, "launch": "eager (one C-ABI call per kernel or pair of kernels)", "step": step}
        try:
            gus = _graph_us(torch, fn, per=24)
            entry["graph"] = {"us_per_step": gus, "tokens_per_s": B / gus * 1e6, "GBps": by / gus / 1e3, "hbm_frac": by / gus / 1e3 / PEAK_HBM_GBS}
        except Exception as e:  # noqa: BLE001 - the eager figure stands on its own
            entry["graph"] = {"error": str(e)[:200]}
        return entry

    _native.attention(q_rot, sets[0][2], sets[0][3], causal=True, out=attn)  # the stream's scratch buffer exists before any capture
    entry = measure(folded, "qkv projection + attention core with the rotary embedding and the cache append folded in "
                            "(tpamd_attention_decode_rope: 2 launches) + dense projection")
    entry["separate_calls"] = measure(separate, "qkv projection + rotary/cache append + attention core (keys split, 2 launches) + dense projection")
    return entry


def falcon_attention_prefill_step(torch, _native, dev) -> dict:
    """BASELINE config 4, prefill: the same shard on 1024 new tokens of one sequence (empty cache): QKV projection, rotary +
    cache fill, causal attention over the 1024 positions, dense projection. FLOPs: both projections and the visible half
    of the score and value products."""
    S, Hq, Hkv, D, d_model = 1024, 64, 4, 64, 8192
    per = Hq // Hkv
    g = torch.Generator(device=dev).manual_seed(0)
    wqkv = (torch.randn((Hq + 2 * Hkv) * D, d_model, device=dev, generator=g) * 0.02).to(torch.bfloat16)
    wdense = (torch.randn(d_model, Hq * D, device=dev, generator=g) * 0.02).to(torch.bfloat16)
    kc = torch.zeros(1, Hkv, S, D, device=dev, dtype=torch.bfloat16)
    vc = torch.zeros(1, Hkv, S, D, device=dev, dtype=torch.bfloat16)
    x = torch.randn(1, S, d_model, device=dev, generator=g).to(torch.bfloat16)
    inv = 1.0 / (10000.0 ** (torch.arange(0, D, 2, device=dev, dtype=torch.float32) / D))
    ang = torch.arange(S, device=dev, dtype=torch.float32)[:, None] * inv[None, :]
    ang = torch.cat([ang, ang], dim=-1)[None]
    cos, sin = ang.cos().to(torch.bfloat16), ang.sin().to(torch.bfloat16)

    def fn(i):
        fused = _native.linear(x, wqkv).view(1, S, Hkv, per + 2, D)
        q_rot = _native.rope_append(fused[:, :, :, :per], fused[:, :, :, per], fused[:, :, :, per + 1], cos, sin, kc, vc, 0)
        attn = _native.attention(q_rot, kc, vc, causal=True)
        return _native.linear(attn.view(S, Hq * D), wdense)

    us = _time_us(torch, fn, 10, 50)
    flops = 2.0 * S * d_model * (Hq + 2 * Hkv) * D + 2.0 * S * Hq * D * d_model + 4.0 * Hq * S * S * D * 0.5
    return {"us_per_step": us, "tokens_per_s": S / us * 1e6, "TFLOPs": flops / us / 1e6, "mfma_frac": flops / us / 1e6 / PEAK_BF16_TFLOPS,
            "algorithmic_flops": flops, "step": "qkv projection + rotary/cache fill + causal attention core + dense projection, eager"}


def api_level_extras(torch, dev, model_graphs: bool = True) -> dict:
    """Two figures through the package's Python surface (tp.TensorParallel / tp.tensor_parallel), host orchestration
    included, with BOTH rank shards on this one GPU:
    c2_tp_module_m4096: the Llama-7B MLP (d 4096, ffn 11008, bf16) split by the Llama rules at W = 2, 4096 tokens per
        forward: each rank's fused gate/up GEMM and down projection, the second rank's down projection adding the first
        rank's partial in its epilogue (no reduction launch), and the copy that gives each rank its own result;
    c1_opt125m: BASELINE config 1, OPT-125m architecture in fp32 with N(0, 0.02) weights, batch 2 x 64 tokens, W = 2
        through tp.tensor_parallel: tokens/s = 128 / forward latency (for information; the step is launch-bound)."""
    from types import SimpleNamespace

    from torch import nn

    import tensor_parallel_amd as tp
    from tensor_parallel_amd.slicing_configs import get_llama_config

    out = {}

    class MLP(nn.Module):
        def __init__(self, d, f):
            super().__init__()
            self.gate_proj, self.up_proj, self.down_proj = nn.Linear(d, f, bias=False), nn.Linear(d, f, bias=False), nn.Linear(f, d, bias=False)
            self.act_fn = nn.SiLU()

        def forward(self, x):
            return self.down_proj(self.act_fn(self.gate_proj(x)) * self.up_proj(x))

    class Block(nn.Module):
        def __init__(self, d, f):
            super().__init__()
            self.mlp = MLP(d, f)

        def forward(self, x):
            return self.mlp(x)

    with torch.no_grad():
        with torch.device(dev):
            block = Block(D_MODEL, 2 * FFN_SHARD).to(torch.bfloat16)
        for p in block.parameters():
            p.normal_(0.0, 0.02)
        cfg = get_llama_config(SimpleNamespace(model_type="llama", hidden_size=D_MODEL, num_attention_heads=32, num_key_value_heads=32), [dev, dev])
        model_tp = tp.TensorParallel(block, [dev, dev], tensor_parallel_config=cfg, sharded=False)
        del block
        x = torch.randn(4096, D_MODEL, device=dev).to(torch.bfloat16)
        us = _time_us(torch, lambda i: model_tp(x), 20, 30)
        flops = 2 * 6.0 * 4096 * D_MODEL * FFN_SHARD
        out["c2_tp_module_m4096"] = {"us_per_forward": us, "tokens_per_s": 4096 / us * 1e6, "TFLOPs": flops / us / 1e6,
                                     "mfma_frac": flops / us / 1e6 / PEAK_BF16_TFLOPS, "algorithmic_flops": flops,
                                     "what": "tp.TensorParallel forward, both W=2 rank shards on this GPU (the ranks take turns on the host), sum folded into the second rank's down projection"}
        del model_tp, x

        from transformers import OPTConfig, OPTForCausalLM

        torch.manual_seed(0)
        model = OPTForCausalLM(OPTConfig()).eval()
        for p in model.parameters():
            p.normal_(0.0, 0.02)
        opt_tp = tp.tensor_parallel(model, [dev, dev])
        ids = torch.randint(0, 50272, (2, 64), generator=torch.Generator().manual_seed(1)).to(dev)
        us = _time_us(torch, lambda i: opt_tp(input_ids=ids, use_cache=False).logits, 5, 20)
        out["c1_opt125m"] = {"us_per_forward": us, "tokens_per_s": 128 / us * 1e6, "dtype": "f32",
                             "what": "tp.tensor_parallel(OPT-125m, W=2) forward of 2 x 64 tokens, both rank shards on this GPU, host orchestration included"}
        if model_graphs:
            graphed = tp.graphs.capture(opt_tp, input_ids=ids, use_cache=False)
            us_g = _time_us(torch, lambda i: graphed.replay().logits, 5, 20)
            out["c1_opt125m"]["graph"] = {"us_per_forward": us_g, "tokens_per_s": 128 / us_g * 1e6,
                                          "what": "the same forward recorded once with tp.graphs.capture and replayed as a HIP graph"}
            del graphed
        del opt_tp, model
        out["llama_layer_decode_tp"] = llama_layer_decode(torch, dev, model_graphs)
    return out


def llama_layer_decode(torch, dev, model_graphs: bool = True) -> dict:
    """One decode step of a Llama-2-7B-shaped decoder (2 layers: d 4096, 32 heads of 128, ffn 11008, bf16) through
    tp.tensor_parallel at W = 2 with both rank shards on this GPU, batch 8 on 2048 cached positions, host orchestration
    included: the wrapped attention modules with their own forward (torch rotary embedding and cache update, the library's
    attention core) and with tp.attention.fuse_rotary_ (rotary embedding, cache append and attention core in the library's
    decode call). Every step appends a position, so the cache is cropped back between steps."""
    from copy import deepcopy

    from transformers import DynamicCache, LlamaConfig, LlamaModel

    import tensor_parallel_amd as tp

    name = tp.attention.register()
    torch.manual_seed(0)
    cfg = LlamaConfig(vocab_size=1024, hidden_size=D_MODEL, intermediate_size=2 * FFN_SHARD, num_hidden_layers=2, num_attention_heads=32,
                      num_key_value_heads=32, max_position_embeddings=4096, attn_implementation="eager")
    with torch.device(dev):
        model = LlamaModel(cfg).to(torch.bfloat16).eval()
    for p in model.parameters():
        p.normal_(0.0, 0.02)
    model.config._attn_implementation = name
    B, L = 8, 2048
    prompt = torch.randint(0, 1024, (B, L), generator=torch.Generator().manual_seed(1)).to(dev)
    tok = torch.randint(0, 1024, (B, 1), generator=torch.Generator().manual_seed(2)).to(dev)
    res = {}
    for label in ("own_forward", "fuse_rotary"):
        m = tp.tensor_parallel(deepcopy(model), [dev, dev])
        if label == "fuse_rotary":
            tp.attention.fuse_rotary_(m)
        cache = DynamicCache()
        m(input_ids=prompt, past_key_values=cache, use_cache=True)

        def step(i, m=m, cache=cache):
            m(input_ids=tok, past_key_values=cache, use_cache=True)
            cache.crop(-1)

        us = _time_us(torch, step, 5, 30)
        res[label] = {"us_per_step": us, "tokens_per_s": B / us * 1e6}
        del m, cache
    res["what"] = ("tp.tensor_parallel(2-layer Llama-2-7B-shaped decoder, W=2) decode step, batch 8 on 2048 cached positions, both rank "
                   "shards on this GPU, host orchestration and the cache crop included")
    if not model_graphs:
        return res
    # the same step on a static cache (the count of cached positions stays on the device), recorded once as a HIP graph
    from transformers import StaticCache

    m = tp.tensor_parallel(deepcopy(model), [dev, dev])
    tp.attention.fuse_rotary_(m, assume_no_padding=True)
    cache = StaticCache(config=cfg, max_cache_len=L + 64)
    m(input_ids=prompt, past_key_values=cache, use_cache=True)
    graphed = tp.graphs.capture(m, input_ids=tok, past_key_values=cache, use_cache=True)
    counts = [layer.cumulative_length for c in [cache] + cache.__dict__["_tp_rank_siblings"] for layer in c.layers]

    def replay(i):
        graphed.replay()
        for count in counts:  # back to 2048 cached positions (the counterpart of the crop above)
            count.sub_(1)

    us = _time_us(torch, replay, 5, 30)
    res["fuse_rotary_static_cache_graph"] = {"us_per_step": us, "tokens_per_s": B / us * 1e6}
    del m, cache, graphed
    res["what"] = ("tp.tensor_parallel(2-layer Llama-2-7B-shaped decoder, W=2) decode step, batch 8 on 2048 cached positions, both rank "
                   "shards on this GPU, host orchestration and the cache crop included; the last entry: transformers' StaticCache, "
                   "fuse_rotary_(assume_no_padding=True), the whole step replayed as one HIP graph (tp.graphs.capture)")
    res["generate"] = llama_generate(torch, dev, cfg, model, prompt)
    return res


def llama_generate(torch, dev, cfg, decoder, prompt) -> dict:
    """`generate` of the same decoder under a language-model head (greedy, batch 8, 2048 prompt positions): time per new token
    = (a call for 33 new tokens - a call for 1) / 32, so the prefill and the set-up of a call drop out. Three ways: the
    wrapped modules' own forward on a growing cache; fuse_rotary_ on a growing cache; fuse_rotary_(assume_no_padding=True) with
    cache_implementation="static", where the wrapper records the decode step as a HIP graph at its first use in a call
    (the recording is inside the timed call) and replays it for every further token."""
    import time
    from copy import deepcopy

    from transformers import LlamaForCausalLM

    import tensor_parallel_amd as tp

    with torch.device(dev):
        lm = LlamaForCausalLM(cfg).to(torch.bfloat16).eval()
    lm.model.load_state_dict(decoder.state_dict())
    lm.lm_head.weight.data.normal_(0.0, 0.02)
    lm.config._attn_implementation = decoder.config._attn_implementation
    lm.generation_config.pad_token_id = 0
    out = {}
    for label in ("own_forward", "fuse_rotary", "fuse_rotary_static_cache_graph"):
        m = tp.tensor_parallel(deepcopy(lm), [dev, dev])
        kwargs = {}
        if label == "fuse_rotary":
            tp.attention.fuse_rotary_(m)
        elif label != "own_forward":
            tp.attention.fuse_rotary_(m, assume_no_padding=True)
            kwargs["cache_implementation"] = "static"

        def run(n):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            m.generate(prompt, max_new_tokens=n, min_new_tokens=n, do_sample=False, **kwargs)
            torch.cuda.synchronize()
            return time.perf_counter() - t0

        run(3)  # first uses
        one = min(run(1) for _ in range(2))
        many = min(run(33) for _ in range(2))
        ms = (many - one) / 32 * 1e3
        out[label] = {"ms_per_new_token_step": ms, "tokens_per_s": prompt.shape[0] / ms * 1e3}
        del m
    out["what"] = "tp.tensor_parallel(LlamaForCausalLM over the same 2 layers, W=2).generate, greedy, batch 8 on a 2048-token prompt, (33 new tokens - 1 new token) / 32"
    return out


def reduce_extra(torch, _native, dev, other) -> dict:
    """The "sum" rule on its own: two rank partials [4096 x 4096] bf16 added by tpamd_reduce_partials (what runs when the sum
    is not folded into the down projection's epilogue). Bytes: two partials read, one result written."""
    parts = [[torch.randn_like(other), torch.randn_like(other)] for _ in range(4)]
    out = torch.empty_like(other)
    us = _time_us(torch, lambda i: _native.reduce_partials(parts[i % 4], out=out), 10, 100)
    by = 3.0 * other.numel() * 2
    return {"us_per_call": us, "GBps": by / us / 1e3, "hbm_frac": by / us / 1e3 / PEAK_HBM_GBS, "algorithmic_bytes": by}


def w8_decode(torch, _native, dev, m=1, graph=True) -> dict:
    """BASELINE config 5 at batch m: int8 weight-only rank-0 shard of a Falcon-40B-shape MLP (up [16384 x 8192] + GELU,
    down [8192 x 16384], per-row scales, 41 / 82 outlier columns in fp16), fp16 activations. HBM-bound."""
    d, f, n_sets = 8192, 16384, 3
    g = torch.Generator(device=dev).manual_seed(0)

    def make(n, k, n_out):
        wq = torch.randint(-127, 128, (n, k), device=dev, dtype=torch.int8, generator=g)
        scale = torch.rand(n, device=dev, generator=g) * 1e-3
        idx = torch.randperm(k, device=dev, generator=g)[:n_out].sort().values.int()
        w_out = (torch.randn(n, n_out, device=dev, generator=g) * 0.02).half()
        return wq, scale, idx, w_out

    ups = [make(f, d, 41) for _ in range(n_sets)]
    downs = [make(d, f, 82) for _ in range(n_sets)]
    x = torch.randn(m, d, device=dev, generator=g).half()

    def fn(i):
        u, dn = ups[i % n_sets], downs[i % n_sets]
        h = _native.linear_w8(x, u[0], u[1], u[2], u[3], act=_native.ACT_GELU)
        return _native.linear_w8(h, dn[0], dn[1], dn[2], dn[3])

    us = _time_us(torch, fn, 10, 100)
    by = 2.0 * f * d + (f * 41 + d * 82) * 2.0 + (f + d) * 4.0
    entry = {"us_per_step": us, "tokens_per_s": m * 1e6 / us, "GBps": by / us / 1e3, "hbm_frac": by / us / 1e3 / PEAK_HBM_GBS,
             "algorithmic_bytes": by, "launch": "eager"}
    if not graph:  # prefill-sized: bound by the matrix pipe, not by the weight bytes
        flops = 4.0 * m * d * f
        return {"us_per_step": us, "tokens_per_s": m * 1e6 / us, "TFLOPs": flops / us / 1e6, "mfma_frac": flops / us / 1e6 / PEAK_BF16_TFLOPS,
                "algorithmic_flops": flops, "step": "int8 up + GELU + down of the Falcon-40B MLP shard, weights dequantised on their way into LDS"}
    try:
        gus = _graph_us(torch, fn, per=12)
        entry["graph"] = {"us_per_step": gus, "tokens_per_s": m * 1e6 / gus, "GBps": by / gus / 1e3, "hbm_frac": by / gus / 1e3 / PEAK_HBM_GBS}
    except Exception as e:  # noqa: BLE001 - the eager figure stands on its own
        entry["graph"] = {"error": str(e)[:200]}
    return entry


if __name__ == "__main__":
    sys.exit(main())
