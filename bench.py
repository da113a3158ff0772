#!/usr/bin/env python3
"""Benchmark of the quantized-linear hot path on one MI355X.

Workload (default): the headline configuration, "random-init Llama-2-7B-architecture model with int4 g128 weight-only
linears, batch 32, prompt 256, 512 greedy-decoded tokens, bf16 KV cache".  One step = one decode step of the whole
batch (129 dequant-GEMV launches -- w1 and w3 of a block share one gated launch -- plus decode attention, norms,
RoPE), replayed from a HIP graph.  The timed steps sit at cache positions spread evenly over the whole decode, so
`value` -- decoded tokens per second = batch * steps / time, everything resident in HBM -- is the configuration's
average whatever --steps is (--full-decode runs every position once as a check).

Extra objects on the JSON line:
  roofline      the dequant-GEMV kernels of one decode step launched back to back (all of them, each on its
                own weights, 3.5 GB working set per pass so no cache holds it), timed with events on the
                launch stream: algorithmic bytes / average launch duration against 8 TB/s.
  cpu_baseline  the reference CPU path (dequantize + F.linear, torch CPU ops) on the host cores for one
                transformer layer + LM head at the same batch, extrapolated to a full decode step (every other mode
                -- --per-shape, --reward, --model 34B, --mode int8 -- carries its own CPU leg).
"""

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0

# HBM bytes per dequant-GEMV launch (fetched + written) from rocprofv3 FETCH_SIZE / WRITE_SIZE runs of
# `bench.py --gemv-only`, scaled by a 256 MiB copy; the summary with the commands is in
# profiles/int4_staged_mm_7b_decode_bs32.md (int4_skinny_mm_7b_decode_bs32.md for the row-major kernels).  Counters cannot be read from inside this process, so the figure is
# recorded here for the configuration and kernel set it was measured on and reported as null for any other.
MEASURED_TRAFFIC_BYTES = {("7B", "int4", 128, 32, "int4_skinny_mm_kernel"): 33_440_000,
                          ("7B", "int4", 128, 32, "int4_staged_mm_kernel"): 32_370_000}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--model", default="7B", help="7B (headline) | 34B | tiny-test")
    ap.add_argument("--mode", default="int4", choices=["int4", "int8"])
    ap.add_argument("--groupsize", type=int, default=128)
    ap.add_argument("--batch", type=int, default=32)
    ap.add_argument("--prompt", type=int, default=256)
    ap.add_argument("--max-new", type=int, default=512)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--seed-on", default="auto", choices=["auto", "cpu", "device"],
                    help="where the random weights are drawn: a CPU generator with seed 1234 (identical values on every machine; "
                         "about 8 s per billion parameters) or the GPU's generator; auto = cpu up to 8 billion parameters")
    ap.add_argument("--gemv-reps", type=int, default=20)
    ap.add_argument("--reward", action="store_true",
                    help="reward-model scoring workload instead of decode: one fully causal pass over --batch x --prompt "
                         "tokens per step (use --mode int8 --batch 64 --prompt 768 for the reference's scoring configuration)")
    ap.add_argument("--per-shape", default="",
                    help="comma-separated row counts M: time every distinct quantized-linear shape of the model at each M "
                         "(all layers' instances back to back, so the weights rotate) and print one JSON line")
    ap.add_argument("--stock", action="store_true",
                    help="with --per-shape (int4): time PyTorch-ROCm's own aten._weight_int4pack_mm on the same codes instead "
                         "of this library's kernel, and report the largest difference between the two results")
    ap.add_argument("--stock-step", action="store_true",
                    help="comparator run of the decode benchmark: the same model and HIP-graph replayed step, but every int4 "
                         "linear goes through PyTorch-ROCm's aten._weight_int4pack_mm and everything around the linears through "
                         "stock torch ops (what the reference's model code executes, without inductor); prints its own JSON line")
    ap.add_argument("--model-switch", action="append", default=[], metavar="NAME=0|1",
                    help="set a fusion switch of easy_to_hard_amd.model (FUSE_GATE, FUSE_ROPE_PROJECTION, DEFER_SPLIT_K, STAGED_DECODE, STAGED_HEAD, FUSE_HEAD_ARGMAX) for a comparison run")
    ap.add_argument("--option", action="append", default=[], metavar="NAME=VALUE",
                    help="launch-geometry override passed to e2h_set_option (experiments)")
    ap.add_argument("--full-decode", action="store_true",
                    help="run the whole decode of the configuration (every position once) and print its tok/s, as a check of "
                         "the default mode's evenly spread sample of positions")
    ap.add_argument("--floor", action="store_true",
                    help="launch floor of this machine for the step's dequant-GEMV launches: a kernel of the library that only reads "
                         "(e2h_stream_read_probe) is launched once per quantized-linear launch of a decode step on as many bytes as that "
                         "launch has to read, from a HIP graph over a rotating region; prints the time per launch size and their sum")
    ap.add_argument("--gemv-only", action="store_true",
                    help="only the back-to-back dequant-GEMV pass plus a 256 MiB calibration copy (for counter runs)")
    return ap.parse_args()


def spread_positions(t_prompt, n_new, steps):
    """Cache positions of the timed decode steps: `steps` positions spread evenly over t_prompt .. t_prompt + n_new - 1
    (both ends included; a single step sits in the middle), so that their mean is the mean position of the decode."""
    if steps <= 1:
        return [t_prompt + (n_new - 1) // 2] * max(steps, 0)
    return [t_prompt + round(i * (n_new - 1) / (steps - 1)) for i in range(steps)]


def quantized_linears(model):
    import easy_to_hard_amd as e2h

    return [(n, m) for n, m in model.named_modules() if isinstance(m, (e2h.WeightOnlyInt4Linear, e2h.WeightOnlyInt8Linear))]


def algorithmic_bytes(mod, m):
    """HBM bytes one launch has to move: weights + qparams + activations in + out (bf16)."""
    import easy_to_hard_amd as e2h

    n, k = mod.out_features, mod.in_features
    if isinstance(mod, e2h.WeightOnlyInt4Linear):
        return n * k // 2 + (k // mod.groupsize) * n * 4 + m * k * 2 + m * n * 2
    return n * k + 2 * n + 2 * m * k + 2 * m * n


def measure_gemv_roofline(model, batch, reps, traffic_key=None):
    """All quantized-linear launches of one decode step, back to back from one HIP graph: the same kernel instantiations
    and epilogues the decode step runs (for an int4 model the staged decode-batch kernels with the RoPE + cache write,
    gated and K-slice epilogues), each launch on its own layer's weights."""
    import torch

    dev = torch.device("cuda", 0)
    lins = quantized_linears(model)
    xs = {}
    for _, mod in lins:
        if mod.in_features not in xs:
            xs[mod.in_features] = torch.randn((batch, mod.in_features), device=dev, dtype=torch.float32).to(torch.bfloat16)

    from easy_to_hard_amd import model as e2h_model
    from easy_to_hard_amd import ops

    calls, by_name, bytes_pass = [], dict(lins), 0
    kernel_set = None
    if not model.kv_cache_enabled:
        model.setup_caches(batch, 768)
    if model.staged_step_supported(batch):
        kernel_set = "int4_staged_mm_kernel"
        staged = {k: ops.stage_x(v) for k, v in xs.items()}
        pos = torch.tensor([model.max_seq_length // 2], device=dev, dtype=torch.int64)
        for blk in model.layers:
            att, ff = blk.attention, blk.feed_forward
            w, wo, w1, w3, w2 = att.wqkv, att.wo, ff.w1, ff.w3, ff.w2
            calls.append(lambda a=att, w=w, s=staged[w.in_features]: ops.int4_mm_staged_rope_kv(
                s, w.weight, w.scales_and_zeros, w.groupsize, a.freqs_table, a.kv_cache.k_cache, a.kv_cache.v_cache, pos, a.n_head,
                a.n_local_heads, a.head_dim))
            calls.append(lambda l=wo, s=staged[wo.in_features], n=ops.int4_staged_partial_slices(batch, wo): ops.int4_mm_staged_partials(
                s, l.weight, l.groupsize, l.scales_and_zeros, n))
            calls.append(lambda g=w1, u=w3, s=staged[w1.in_features]: ops.int4_mm_staged_silu_gate(
                s, g.weight, g.scales_and_zeros, u.weight, u.scales_and_zeros, g.groupsize))
            calls.append(lambda l=w2, s=staged[w2.in_features], n=ops.int4_staged_partial_slices(batch, w2): ops.int4_mm_staged_partials(
                s, l.weight, l.groupsize, l.scales_and_zeros, n))
            bytes_pass += algorithmic_bytes(w, batch) + algorithmic_bytes(wo, batch) + algorithmic_bytes(w2, batch)
            # two weight matrices, but x is read once and one [batch, n] result is written
            bytes_pass += algorithmic_bytes(w1, batch) + algorithmic_bytes(w3, batch) - batch * 2 * (w1.in_features + w1.out_features)
        out = model.output
        if e2h_model.STAGED_HEAD and ops.int4_staged_supported(batch, out, ops.STAGED_PLAIN):
            calls.append(lambda l=out, s=staged[out.in_features]: ops.int4_mm_staged(s, l.weight, l.groupsize, l.scales_and_zeros))
        else:
            calls.append(lambda l=out, x=xs[out.in_features]: l(x))
        bytes_pass += algorithmic_bytes(out, batch)
        lins = []
    # otherwise the launches of the row-major path: a feed-forward block's w1 and w3 go out as one gated launch where the
    # model does so too; every other quantized linear is one launch
    for name, mod in lins:
        parent_name, _, leaf = name.rpartition(".")
        parent = model.get_submodule(parent_name) if parent_name else model
        x = xs[mod.in_features]
        fused8 = isinstance(parent, e2h_model.FeedForward) and parent._gate_fusable_int8(x)
        fused = fused8 or (isinstance(parent, e2h_model.FeedForward) and parent._gate_fusable(x))
        if fused and leaf == "w3":
            continue
        if fused and leaf == "w1":
            up = by_name[parent_name + ".w3"]
            if fused8:
                calls.append(lambda x=x, g=mod, u=up: ops.int8_mm_silu_gate(x, g.weight, g.scales, u.weight, u.scales))
            else:
                calls.append(lambda x=x, g=mod, u=up: ops.int4_mm_silu_gate(
                    x, g.weight, g.scales_and_zeros, u.weight, u.scales_and_zeros, g.groupsize))
            # two weight matrices, but x is read once and one [batch, n] result is written
            bytes_pass += algorithmic_bytes(mod, batch) + algorithmic_bytes(up, batch) - batch * 2 * (mod.in_features + mod.out_features)
        else:
            calls.append(lambda x=x, m=mod: m(x))
            bytes_pass += algorithmic_bytes(mod, batch)
    if kernel_set is None:
        kernel_set = "int4_skinny_mm_kernel" if "Int4" in type(by_name[next(iter(by_name))]).__name__ else "int8_stream_mm_kernel"

    def one_pass():
        out = None
        for call in calls:
            out = call()
        return out

    side = torch.cuda.Stream(device=dev)
    side.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(side):
        one_pass()
    torch.cuda.current_stream(dev).wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        one_pass()
    for _ in range(3):
        graph.replay()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(reps):
        graph.replay()
    stop.record()
    torch.cuda.synchronize()
    total_s = start.elapsed_time(stop) * 1e-3
    launches = len(calls) * reps
    avg_launch_s = total_s / launches
    achieved = bytes_pass * reps / total_s / 1e9
    return {
        "bound": "hbm",
        "achieved": round(achieved, 1),
        "peak": HBM_PEAK_GBPS,
        "unit": "GB/s",
        "frac": round(achieved / HBM_PEAK_GBPS, 4),
        "traffic": MEASURED_TRAFFIC_BYTES.get(tuple(traffic_key or ()) + (kernel_set,)),
        "kernel": kernel_set,
        "launches_per_step": len(calls),
        "algorithmic_bytes_per_launch": bytes_pass // len(calls),
        "avg_launch_us": round(avg_launch_s * 1e6, 3),
        "gemv_ms_per_step": round(total_s / reps * 1e3, 4),
    }


def measure_launch_floor(model, batch, reps):
    """What the step's quantized-linear launches would cost if each did nothing but read its weights and qparams: the
    library's streaming-read kernel on the same byte counts, one launch per linear launch, replayed from a HIP graph.
    The read regions rotate through a buffer larger than every cache."""
    import ctypes

    import torch

    from easy_to_hard_amd import _lib

    dev = torch.device("cuda", 0)
    lib = _lib.load()
    sizes = []  # (name, weight + qparam bytes, activation bytes) of every launch of a step (w1 and w3 share a launch)
    for blk in model.layers:
        att, ff = blk.attention, blk.feed_forward
        wb = lambda m: algorithmic_bytes(m, 0)
        xb = lambda m: batch * m.in_features * 2
        sizes += [("wqkv", wb(att.wqkv), xb(att.wqkv)), ("wo", wb(att.wo), xb(att.wo)), ("w1+w3", wb(ff.w1) + wb(ff.w3), xb(ff.w1)),
                  ("w2", wb(ff.w2), xb(ff.w2))]
    sizes.append(("output", algorithmic_bytes(model.output, 0), batch * model.output.in_features * 2))
    region = torch.empty(3 << 30, dtype=torch.uint8, device=dev).fill_(3)
    shared = torch.empty(max(x for _, _, x in sizes) + 16, dtype=torch.uint8, device=dev).fill_(5)
    stream = lambda: ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)

    def timed(launches):
        """launches: list of (weight bytes, shared activation bytes); returns the average microseconds per launch"""
        def one_pass():
            off = 0
            for nbytes, xbytes in launches:
                nbytes -= nbytes % 16
                xbytes -= xbytes % 16
                if off + nbytes > region.numel():
                    off = 0
                rc = lib.e2h_stream_read_probe(ctypes.c_void_p(region.data_ptr() + off), nbytes, ctypes.c_void_p(shared.data_ptr()), xbytes,
                                               None, stream())
                assert rc == 0, rc
                off += (nbytes + 4095) // 4096 * 4096
        side = torch.cuda.Stream(device=dev)
        side.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(side):
            one_pass()
        torch.cuda.current_stream(dev).wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            one_pass()
        graph.replay()
        torch.cuda.synchronize()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(reps):
            graph.replay()
        stop.record()
        torch.cuda.synchronize()
        return start.elapsed_time(stop) * 1e3 / (reps * len(launches))

    per_size = {}
    for name, nbytes, xbytes in sizes:
        if name not in per_size:
            per_size[name] = {"bytes": nbytes, "us": round(timed([(nbytes, 0)] * 64), 2), "activation_bytes": xbytes,
                              "us_with_activations_read_by_every_workgroup": round(timed([(nbytes, xbytes)] * 64), 2)}
    empty_us = round(timed([(0, 0)] * 256), 2)
    step_us = timed([(b, 0) for _, b, _ in sizes]) * len(sizes)
    step_x_us = timed([(b, x) for _, b, x in sizes]) * len(sizes)
    total_bytes = sum(b for _, b, _ in sizes)
    return {"empty_launch_us": empty_us, "per_launch": per_size, "launches_per_step": len(sizes),
            "read_only_ms_per_step": round(step_us * 1e-3, 4), "weight_bytes_per_step": total_bytes,
            "hbm_frac_of_a_read_only_step": round(total_bytes / (step_us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
            "read_only_ms_per_step_with_activations": round(step_x_us * 1e-3, 4),
            "hbm_frac_of_a_read_only_step_with_activations": round(total_bytes / (step_x_us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
            "note": "a launch-per-linear decode step cannot spend less time in its quantized linears than read_only_ms_per_step; "
                    "with_activations: every workgroup of the read-only launch also reads the batch's activations (from L2), as every CU of "
                    "a decode-batch matmul must"}


def stock_int4_operands(mod):
    """The same codes and (scale, zero) pairs in the form PyTorch-ROCm's own aten._weight_int4pack_mm takes (its packing
    differs from the checkpoint layout): codes two per byte, even k in the high nibble, through its own packer."""
    import torch

    from easy_to_hard_amd import ops

    codes = ops.int4_unpack(mod.weight)
    two_per_byte = ((codes[:, ::2] << 4) | codes[:, 1::2]).to(torch.uint8)
    return torch.ops.aten._convert_weight_to_int4pack(two_per_byte, mod.inner_k_tiles), mod.scales_and_zeros


def measure_per_shape(model, rows_list, reps=6, stock=False, cpu=True):
    """Average launch duration of each distinct quantized-linear shape, replayed from a HIP graph and timed with events on
    the launch stream; the instances of a shape in different layers have different weights, so nothing stays cached."""
    import torch

    import easy_to_hard_amd as e2h

    dev = torch.device("cuda", 0)
    groups = {}
    for name, mod in quantized_linears(model):
        groups.setdefault((name.rpartition(".")[2], mod.out_features, mod.in_features), []).append(mod)
    out = []
    for (leaf, n, k), mods in groups.items():
        for m in rows_list:
            x = torch.randn((m, k), device=dev, dtype=torch.float32).to(torch.bfloat16)

            stock_ops = [stock_int4_operands(mod) for mod in mods] if stock else None

            def one_pass():
                if stock_ops is not None:
                    for (w_stock, sz), mod in zip(stock_ops, mods):
                        torch.ops.aten._weight_int4pack_mm(x, w_stock, mod.groupsize, sz)
                    return
                for mod in mods:
                    mod(x)

            if stock_ops is not None:  # same codes, so the two kernels must agree to bf16 rounding
                y_stock = torch.ops.aten._weight_int4pack_mm(x, stock_ops[0][0], mods[0].groupsize, stock_ops[0][1]).float()
                y_ours = mods[0](x).float()
                stock_err = float((y_stock - y_ours).abs().max() / y_ours.abs().max())
            side = torch.cuda.Stream(device=dev)
            side.wait_stream(torch.cuda.current_stream(dev))
            with torch.cuda.stream(side):
                one_pass()
            torch.cuda.current_stream(dev).wait_stream(side)
            graph = torch.cuda.CUDAGraph()  # replayed: host launch cost would otherwise hide the short kernels
            with torch.cuda.graph(graph):
                one_pass()
            graph.replay()
            torch.cuda.synchronize()
            start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            for _ in range(reps):
                graph.replay()
            stop.record()
            torch.cuda.synchronize()
            del graph
            us = start.elapsed_time(stop) * 1e3 / (reps * len(mods))
            nbytes = algorithmic_bytes(mods[0], m)
            int4 = isinstance(mods[0], e2h.WeightOnlyInt4Linear)
            out.append({"linear": leaf, "n": n, "k": k, "m": m, "instances": len(mods), "us": round(us, 2),
                        "GBps": round(nbytes / us / 1e3, 1), "hbm_frac": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4),
                        "TFLOPs": round(2.0 * m * n * k / us / 1e6, 1), "kind": "int4" if int4 else "int8"})
            if stock_ops is not None:
                out[-1]["kernel"] = "aten._weight_int4pack_mm"
                out[-1]["max_diff_vs_e2h"] = round(stock_err, 5)
            if cpu:
                # reference CPU path on the same shape: timed fully up to 64 rows, on a 512-row sample beyond
                threads, _ = _cpu_threads()
                torch.set_num_threads(threads)
                rows = m if m <= 64 else min(m, 512)
                cpu_s = _time_cpu(_cpu_case(mods[0], rows, torch.Generator().manual_seed(1234)), 1.0, max_runs=20) * (m / rows)
                out[-1]["cpu_us"] = round(cpu_s * 1e6, 1)
                out[-1]["cpu_threads"] = threads
                out[-1]["cpu_rows_timed"] = rows
    return out


def _cpu_threads():
    """Threads for the CPU baseline: the box's CPU share (OMP_NUM_THREADS where the scheduler sets it), else every
    physical core.  Returns (threads used, physical cores of the host) -- both are reported."""
    try:
        import psutil

        physical = psutil.cpu_count(logical=False) or os.cpu_count() or 1
    except Exception:
        physical = os.cpu_count() or 1
    share = os.environ.get("OMP_NUM_THREADS")
    threads = max(1, min(int(share), os.cpu_count() or 1)) if share and share.isdigit() else physical
    return threads, physical


def _time_cpu(fn, budget_s, max_runs=20):
    """Median wall time of fn() after one warm-up run, repeated until the budget is used (at least twice)."""
    fn()
    times = []
    t_end = time.perf_counter() + budget_s
    while len(times) < 2 or (time.perf_counter() < t_end and len(times) < max_runs):
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
    times.sort()
    return times[len(times) // 2]


def _cpu_case(mod, rows, gen):
    """Closure running the reference CPU path (dequantize + F.linear, oracle/reference_path.py) of one quantized linear
    on `rows` rows of N(0, 1) bfloat16 activations."""
    import torch

    import easy_to_hard_amd as e2h
    from easy_to_hard_amd import ops
    from oracle import reference_path as rp

    x = torch.randn((rows, mod.in_features), generator=gen).to(torch.bfloat16)
    if isinstance(mod, e2h.WeightOnlyInt4Linear):
        codes = ops.int4_unpack(mod.weight).cpu()
        sz = mod.scales_and_zeros.cpu()
        g = mod.groupsize
        return lambda: rp.int4_linear_cpu(x, codes, sz, g)
    q, s = mod.weight.cpu(), mod.scales.cpu()
    return lambda: rp.int8_linear_cpu(x, q, s)


def measure_cpu_baseline(model, batch, groupsize, unit_rows=None, budget_s=2.5):
    """Reference CPU path on the host cores: the quantized linears of one layer + the head at `batch` rows (decode), or at
    a bounded sample of `unit_rows` rows (many-row passes), extrapolated to the whole step."""
    import torch

    threads, physical = _cpu_threads()
    torch.set_num_threads(threads)
    backbone = model.backbone if hasattr(model, "backbone") else model
    layer = backbone.layers[0]
    sample = [layer.attention.wqkv, layer.attention.wo, layer.feed_forward.w1, layer.feed_forward.w3, layer.feed_forward.w2]
    head = backbone.output
    gen = torch.Generator().manual_seed(1234)
    rows = batch if unit_rows is None else min(unit_rows, batch)
    layer_s = sum(_time_cpu(_cpu_case(m, rows, gen), budget_s) for m in sample)
    head_s = _time_cpu(_cpu_case(head, rows, gen), budget_s)
    n_layer = len(backbone.layers)
    step_s = (layer_s * n_layer + head_s) * (batch / rows)
    return {
        "value": round(batch / step_s, 3),
        "unit": "tok/s",
        "cores": threads,
        "kind": "port",
        "sample": f"quantized linears of 1 of {n_layer} layers + head at {rows} rows"
                  + (f" (a sample of the step's {batch} rows, scaled by {batch // rows})" if rows != batch else "")
                  + f" (dequantize + F.linear, torch CPU bf16, {threads} threads; host has {physical} physical cores), "
                  f"median of repeated runs; layer {layer_s * 1e3:.1f} ms, head {head_s * 1e3:.1f} ms; extrapolated to the whole "
                  "step (linears only, attention excluded)",
    }


def run_reward_scoring(args, cfg, dev):
    """Scoring pass of a RewardModel (2-row head, mean over its rows): every linear sees batch * prompt rows, so the
    quantized linears are MFMA-bound.  One step = one pass over the whole batch; value = scored tokens per second."""
    import torch

    from easy_to_hard_amd.generate import model_score
    from easy_to_hard_amd.model import random_quantized_transformer

    model = random_quantized_transformer(cfg, args.mode, args.groupsize, device=dev, seed=1234, reward_head_rows=2,
                                         seed_on="device" if args.seed_on == "device" else "cpu")
    batch, t = args.batch, args.prompt
    ids = torch.randint(0, cfg.vocab_size, (batch, t), generator=torch.Generator().manual_seed(1234)).to(dev)
    steps, warmup = min(args.steps, 8), min(args.warmup, 2)
    for _ in range(max(warmup, 1)):
        rewards = model_score(model, ids)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        rewards = model_score(model, ids)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    lins = quantized_linears(model)
    flops = sum(2.0 * batch * t * m.out_features * m.in_features for _, m in lins)
    print(json.dumps({
        "metric": "reward-model scoring tokens/s (Llama-7B shape, weight-only quantized linears)",
        "value": round(batch * t * steps / elapsed, 1), "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(elapsed / steps * 1e3, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"random-init Llama {args.model}-shaped reward model, {args.mode} weight-only linears, "
                               f"fully causal scoring pass, batch {batch} x {t} tokens", "batch": batch, "tokens": t},
        "roofline": {"bound": "mfma", "achieved": round(flops * steps / elapsed / 1e12, 1), "peak": 2500.0, "unit": "TFLOP/s",
                     "frac": round(flops * steps / elapsed / 1e12 / 2500.0, 4), "traffic": None,
                     "note": "linear-layer flops over the whole step time (attention, norms and elementwise kernels included in the time)"},
        "cpu_baseline": None if args.no_cpu_baseline else measure_cpu_baseline(model, batch * t, args.groupsize, unit_rows=2048, budget_s=1.0),
        "finite": bool(torch.isfinite(rewards.float()).all()),
    }))


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    import torch

    from easy_to_hard_amd import _lib
    from easy_to_hard_amd.generate import GraphedDecodeStep, prefill
    from easy_to_hard_amd.model import ModelArgs, random_quantized_transformer

    _lib.load()  # no fallback: fail here if the HIP library is not built
    for item in args.option:
        name, _, value = item.partition("=")
        _lib.set_option(name, int(value))
    for item in args.model_switch:
        import easy_to_hard_amd.model as model_mod

        name, _, value = item.partition("=")
        assert name in ("FUSE_GATE", "FUSE_ROPE_PROJECTION", "DEFER_SPLIT_K", "STAGED_DECODE", "STAGED_HEAD", "FUSE_HEAD_ARGMAX"), name
        setattr(model_mod, name, bool(int(value)))
    assert torch.cuda.is_available(), "bench.py needs the GPU"
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    cfg = ModelArgs.from_name(args.model)
    if args.reward:
        if args.mode != "int8":
            # the 2-row score head cannot be an int4 linear (out_features % 8 != 0 asserts, as in the reference)
            print("bench.py --reward runs the int8 configuration only (use --mode int8)", file=sys.stderr)
            sys.exit(2)
        run_reward_scoring(args, cfg, dev)
        return
    t0 = time.time()
    n_params = cfg.n_layer * (cfg.dim * (cfg.n_head + 2 * cfg.n_local_heads) * cfg.head_dim + cfg.dim * cfg.dim
                              + 3 * cfg.dim * cfg.intermediate_size) + 2 * cfg.vocab_size * cfg.dim
    seed_on = args.seed_on if args.seed_on != "auto" else ("cpu" if n_params <= 8e9 else "device")
    model = random_quantized_transformer(cfg, args.mode, args.groupsize, device=dev, seed=1234, seed_on=seed_on)
    torch.cuda.synchronize()
    build_s = time.time() - t0

    batch, t_prompt = args.batch, args.prompt
    if args.per_shape:
        rows_list = [int(v) for v in args.per_shape.split(",") if v]
        rows_out = measure_per_shape(model, rows_list, stock=args.stock, cpu=not args.no_cpu_baseline)
        cpu = None
        if not args.no_cpu_baseline:
            cpu = {"value": round(sum(r["cpu_us"] for r in rows_out), 1), "unit": "us (sum over the listed shapes and row counts)",
                   "cores": rows_out[0]["cpu_threads"], "kind": "port",
                   "sample": "dequantize + F.linear (torch CPU bf16) of every listed shape, median of repeated runs; row counts up to "
                             "64 timed fully, larger ones on 512 rows and scaled (see cpu_rows_timed)"}
        print(json.dumps({"per_shape": rows_out, "model": args.model, "mode": args.mode,
                          "groupsize": args.groupsize if args.mode == "int4" else None, "cpu_baseline": cpu}))
        return
    if args.floor:
        print(json.dumps({"floor": measure_launch_floor(model, batch, args.gemv_reps), "model": args.model, "mode": args.mode,
                          "groupsize": args.groupsize if args.mode == "int4" else None, "batch": batch}))
        return
    if args.gemv_only:
        # counter-collection mode: the GEMV pass and a plain copy of known size (its FETCH_SIZE / WRITE_SIZE
        # readings calibrate the counters: 256 MiB read, 256 MiB written per copy)
        roofline = measure_gemv_roofline(model, batch, args.gemv_reps, (args.model, args.mode, args.groupsize, batch))
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"roofline": roofline, "calibration_copy_bytes": src.numel()}))
        return
    if args.stock_step:
        import easy_to_hard_amd as e2h
        import easy_to_hard_amd.model as model_mod

        assert args.mode == "int4", "--stock-step compares the int4 path"
        model_mod.FUSED_DECODE = False
        for _, mod in quantized_linears(model):
            if isinstance(mod, e2h.WeightOnlyInt4Linear):
                w_stock, sz = stock_int4_operands(mod)
                mod.forward = (lambda x, w=w_stock, q=sz, g=mod.groupsize, n=mod.out_features:
                               torch.ops.aten._weight_int4pack_mm(x.reshape(-1, x.shape[-1]), w, g, q).reshape(*x.shape[:-1], n))
    max_seq = min(t_prompt + args.max_new, cfg.block_size)
    n_new = max_seq - t_prompt
    assert n_new >= 2, "the decode budget needs at least two new tokens"
    model.setup_caches(batch, max_seq)
    prompt = torch.randint(0, cfg.vocab_size, (batch, t_prompt), generator=torch.Generator().manual_seed(1234)).to(dev)
    input_pos = torch.arange(0, t_prompt, device=dev)
    t0 = time.time()
    cur = prefill(model, prompt, input_pos)
    torch.cuda.synchronize()
    prefill_s = time.time() - t0
    stepper = GraphedDecodeStep(model, batch, dev)
    cur = prefill(model, prompt, input_pos)  # the capture warm-up wrote cache row 0

    if args.full_decode:
        # the whole decode of the configuration, every position once, timed as the reference does
        # (inference_generate.py:484-486: decoded tokens / wall time of decode_n_tokens)
        pos = torch.tensor([t_prompt], device=dev, dtype=torch.int64)
        for _ in range(args.warmup):
            stepper.step(cur, pos)
            pos += 1  # also loads the kernel of this update, whose first use costs tens of milliseconds
        pos.fill_(t_prompt)
        cur = prefill(model, prompt, input_pos)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n_new - 1):
            cur = stepper.step(cur, pos)
            pos += 1
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
        print(json.dumps({"full_decode": True, "value": round(batch * (n_new - 1) / elapsed, 2), "unit": "tok/s",
                          "ms_per_step": round(elapsed / (n_new - 1) * 1e3, 4), "steps": n_new - 1, "batch": batch,
                          "prompt_len": t_prompt, "model": args.model, "mode": args.mode}))
        return

    # The timed steps sit at positions spread evenly over the whole decode (prompt .. prompt + new - 1), so that their
    # average is the average step of the configuration whatever --steps is: decode attention reads every live cache
    # position, so a step late in the decode costs more than one right after the prompt.  The graph reads the position
    # from device memory; cache rows beyond the prompt hold N(0, 1) values standing in for the keys and values that the
    # skipped steps would have written.
    gen_dev = torch.Generator(device=dev).manual_seed(1234)
    for blk in model.layers:
        kv = blk.attention.kv_cache
        for cache in (kv.k_cache, kv.v_cache):
            cache[:, :, t_prompt:] = torch.randn(cache[:, :, t_prompt:].shape, generator=gen_dev, device=dev, dtype=torch.float32).to(cache.dtype)
    steps = args.steps
    positions = spread_positions(t_prompt, n_new, steps)
    pos_tensors = [torch.tensor([p], device=dev, dtype=torch.int64) for p in positions]
    warm_pos = torch.tensor([t_prompt + (n_new - 1) // 2], device=dev, dtype=torch.int64)
    for _ in range(args.warmup):
        cur = stepper.step(cur, warm_pos).clone()
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        marks[i].record()
        cur = stepper.step(cur, pos_tensors[i])
    marks[steps].record()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    tok_s = batch * steps / elapsed
    step_ms = [marks[i].elapsed_time(marks[i + 1]) for i in range(steps)]

    if args.stock_step:
        print(json.dumps({"comparator": "stock torch ops + aten._weight_int4pack_mm, HIP-graph replayed decode step",
                          "value": round(tok_s, 2), "unit": "tok/s", "ms_per_step": round(elapsed / args.steps * 1e3, 4),
                          "steps": args.steps, "warmup": args.warmup, "batch": batch, "prompt_len": t_prompt, "model": args.model,
                          "groupsize": args.groupsize}))
        return
    roofline = measure_gemv_roofline(model, batch, args.gemv_reps, (args.model, args.mode, args.groupsize, batch))
    cpu = None if args.no_cpu_baseline else measure_cpu_baseline(model, batch, args.groupsize)

    line = {
        "metric": "batched int4 decode tok/s (Llama-7B shape, bs32); dequant-GEMV HBM GB/s % of peak",
        "value": round(tok_s, 2),
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(elapsed / args.steps * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": f"random-init Llama {args.model}-shaped model, {args.mode}"
                        + (f" g{args.groupsize}" if args.mode == "int4" else "")
                        + f" weight-only linears, greedy decode, batch {batch}, prompt {t_prompt}, bf16 KV cache of {max_seq} positions, HIP-graph replayed decode step",
            "batch": batch,
            "prompt_len": t_prompt,
            "new_tokens": n_new,
            "timed_positions": f"{steps} steps at cache positions {positions[0]} .. {positions[-1]}, evenly spread over the decode",
            "step_ms_first_mid_last": [round(step_ms[0], 4), round(step_ms[steps // 2], 4), round(step_ms[-1], 4)],
            "quantized_linears_per_step": roofline["launches_per_step"],
            "weights_seeded_on": seed_on,
            "model_build_s": round(build_s, 2),
            "prefill_s": round(prefill_s, 3),
        },
        "roofline": roofline,
        "cpu_baseline": cpu,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
