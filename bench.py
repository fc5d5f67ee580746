#!/usr/bin/env python3
"""Benchmark of the duo-causal attention hot path on one MI355X.

A step is one duo-causal prefill forward (both iteration streams, one launch) over
the BASELINE.json configs[1] workload: batch 4, seq 4096, 16 query heads, 8 kv
heads, head_dim 128, bf16, 6 % hard tokens, inputs resident in HBM.  The single
JSON line reports algorithmic TFLOP/s (4*D*Hq*visible_pairs per forward), the
MFMA roofline fraction of the dominant kernel, and the reference formulation
(dense additive mask + SDPA, fp32, torch) timed on the host CPU on a bounded
sample as a baseline.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA, vendor figure
PEAK_HBM_GBS = 8000.0


def measured_traffic(leg: str):
    """HBM bytes per launch (per step for the forward+backward legs) of a default workload, as the rocprofv3 --pmc
    FETCH_SIZE / WRITE_SIZE runs measured them: profiles/traffic.json holds the figures (fetched + written, each
    scaled by what the same counter reads for a plain copy of known size) next to the summary file they come from.
    None for a leg the file does not list."""
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            entry = json.load(f)["legs"].get(leg)
    except (OSError, ValueError, KeyError):
        return None
    return None if entry is None else float(entry["fetch_bytes"]) + float(entry["write_bytes"])



def visible_pairs(case):
    from oracle.duo_oracle import visible_pairs as vp
    return vp(case["cu_q1"], case["cu_k1"], case["pos_q2"], case["pos_k2"], case["cu_q2"], case["cu_k2"])


def cpu_baseline(seed: int, T: int, p: float, reps: int = 3):
    """Reference formulation on the host: dense mask + GQA expansion + softmax(QK^T s + M)V, fp32."""
    import torch

    from oracle import duo_oracle as O
    from tests.cases import dense_to_varlen, make_dense_case

    c = make_dense_case(seed, B=1, T=T, p_hard=p)
    for k in ("q1", "k1", "v1", "q2", "k2", "v2"):
        c[k] = c[k] * 0.5
    pairs = visible_pairs(dense_to_varlen(c))
    flops = 4.0 * 128 * 16 * pairs
    ts = []
    with torch.no_grad():
        for _ in range(reps + 1):
            t0 = time.perf_counter()
            O.duo_prefill_dense(c["q1"], c["k1"], c["v1"], c["q2"], c["k2"], c["v2"], c["hard"], c["scale"])
            ts.append(time.perf_counter() - t0)
    t = sorted(ts[1:])[len(ts[1:]) // 2]
    # BASELINE configs[0] exactly as stated: B=1, T=512, fp32, N(0,1) inputs, Bernoulli(0.06) hard tokens
    c0 = make_dense_case(1234, B=1, T=512, p_hard=0.06)
    f0 = 4.0 * 128 * 16 * visible_pairs(dense_to_varlen(c0))
    t0s = []
    with torch.no_grad():
        for _ in range(11):
            t0 = time.perf_counter()
            O.duo_prefill_dense(c0["q1"], c0["k1"], c0["v1"], c0["q2"], c0["k2"], c0["v2"], c0["hard"], c0["scale"])
            t0s.append(time.perf_counter() - t0)
    tc0 = sorted(t0s[1:])[5]
    # configs[2], the reference's way: per sequence one Tq = 1 SDPA call over the repeated-head cache with a
    # (1, 1, 1, L) additive mask, fp32; sample: the first 8 of the 64 sequences (same seeded context lengths)
    g = torch.Generator().manual_seed(1236)
    lens = torch.randint(1024, 16385, (64,), generator=g).tolist()[:8]
    dec_in = [(torch.randn(1, 16, 1, 128, generator=g), torch.randn(1, 8, L, 128, generator=g), torch.randn(1, 8, L, 128, generator=g),
               torch.zeros(1, 1, 1, L)) for L in lens]
    tds = []
    with torch.no_grad():
        for _ in range(4):
            t0 = time.perf_counter()
            for q, k, v, m in dec_in:
                O.sdpa_dense(q, k, v, m, 128 ** -0.5)
            tds.append(time.perf_counter() - t0)
    td = sorted(tds[1:])[1]
    dec_bytes = sum(lens) * 2 * 8 * 128 * 2  # the bytes the metric counts for these rows (bf16 K and V)
    del dec_in
    # configs[3], down-scaled: one document of 1024 tokens (the shortest of the four), p = 0.10, forward + backward
    # through torch autograd over the same dense formulation
    c3 = make_dense_case(1237, B=1, T=1024, p_hard=0.10)
    f3 = 3.5 * 4.0 * 128 * 16 * visible_pairs(dense_to_varlen(c3))
    leaves = {k: (c3[k] * 0.5).requires_grad_(True) for k in ("q1", "k1", "v1", "q2", "k2", "v2")}
    t3s = []
    for _ in range(4):
        t0 = time.perf_counter()
        o1, o2, _ = O.duo_prefill_dense(leaves["q1"], leaves["k1"], leaves["v1"], leaves["q2"], leaves["k2"], leaves["v2"],
                                        c3["hard"], c3["scale"])
        (o1.sum() + o2.sum()).backward()
        t3s.append(time.perf_counter() - t0)
        for t_ in leaves.values():
            t_.grad = None
    t3 = sorted(t3s[1:])[1]
    return {
        "value": flops / t / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
        "sample": f"1 of 4 sequences (B=1, T={T}, p={p}), fp32 dense mask + SDPA restatement, median of {reps}, "
                  f"{t * 1e3:.1f} ms, os.cpu_count()={os.cpu_count()}",
        "configs0": {"workload": "configs[0]: B=1, T=512, Hq=16, Hkv=8, D=128, fp32, p_hard=0.06, as stated",
                     "ms": tc0 * 1e3, "tflops": f0 / tc0 / 1e12, "flop": f0, "median_of": 10},
        "decode": {"workload": "configs[2] as the reference runs it: one Tq=1 SDPA per sequence (repeat_kv + additive mask), fp32",
                   "sample": f"8 of the 64 sequences (context lengths {lens}): 1/8 of the step's sequences, depth-0 queries only",
                   "ms": td * 1e3, "gbs_of_the_metrics_bytes": dec_bytes / td / 1e9, "median_of": 3},
        "configs3": {"workload": "configs[3] down-scaled: forward + backward (torch autograd) over the dense formulation, fp32",
                     "sample": "one document of 1024 tokens, p_hard=0.10: 1/8 of the tokens, about 1/40 of the step's visible pairs",
                     "ms": t3 * 1e3, "tflops": f3 / t3 / 1e12, "flop": f3, "median_of": 3},
    }


def bench_decode(steps: int, warmup: int):
    """BASELINE configs[2]: one decode step, 64 sequences, context uniform in [1024, 16384], 6 % depth-1 rows."""
    import torch

    from tah_amd import kv_cache
    from tests.cases import build_slabs, make_decode_case

    g = torch.Generator().manual_seed(1236)
    lens = torch.randint(1024, 16385, (64,), generator=g).tolist()
    c = make_decode_case(1236, lens, 0.06)
    # Three copies of the cache, used in turn: a step never reads bytes the two steps before it touched,
    # so nothing is served from what the 256 MB last-level cache kept of an earlier step (2.3 GB per step).
    sets = [build_slabs(c, 16384, 2048, device="cuda") for _ in range(3)]
    s1, s2 = sets[0]
    nseq = len(lens)
    hr = torch.tensor(c["hard_rows"], dtype=torch.int32, device="cuda")
    slot = torch.cat([torch.arange(nseq, dtype=torch.int32, device="cuda"), hr])
    qpos1 = torch.from_numpy(c["q_pos"]).cuda()
    qpos = torch.cat([qpos1, qpos1[hr.long()]])
    qd = torch.tensor([0] * nseq + [1] * len(hr), dtype=torch.int32, device="cuda")
    q = torch.cat([c["q1"].cuda(), c["q2"].cuda()])
    n2 = [int(c["cu_k2"][b + 1] - c["cu_k2"][b]) for b in range(nseq)]
    rows = sum(lens) + sum(lens[b] + n2[b] for b in c["hard_rows"])
    nbytes = rows * 2 * 8 * 128 * 2  # K and V, 8 kv heads, 128 bf16
    run = lambda i: kv_cache.decode(q, slot, qpos, sets[i % 3][0], sets[i % 3][1], scale=c["scale"], q_depth=qd)
    yield  # inputs are resident; everything below runs when main() resumes the leg
    for i in range(warmup):
        run(i)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(steps):
        run(i)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / steps
    gbs = nbytes / (ms * 1e-3) / 1e9
    return {"workload": "configs[2]: decode step, 64 seqs, ctx U[1024,16384], 6% depth-1 rows, Hq=16, Hkv=8, D=128 "
                        "(three copies of the cache read in rotation)",
            "ms_per_step": ms, "visible_rows": rows, "algorithmic_bytes": nbytes, "hbm_gbs": gbs,
            "roofline": {"bound": "hbm", "achieved": gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": gbs / PEAK_HBM_GBS,
                         "traffic": measured_traffic("decode"), "kernels": "duo_decode_split_kernel<2> + duo_decode_merge_kernel"},
            "tokens_per_s": nseq / (ms * 1e-3)}


def launch_order(ops, dev, hq=16, hkv=8):
    """The launch-order table of a packed batch (None for one sequence): per-batch data like the boundary arrays,
    built once outside the timed region -- in the model one table serves all 28 layers, forward and backward."""
    return ops.duo_schedule(dev["cu_q1"], dev["cu_k1"], dev["cu_q2"], dev["cu_k2"], dev["pos_q2"], hq, hkv,
                            dev["q1"].shape[0], dev["k1"].shape[0], dev["k2"].shape[0])


def time_schedule_build(ops, dev, n=20):
    import torch
    launch_order(ops, dev)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(n):
        launch_order(ops, dev)
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / n


def bench_fwd_bwd(name: str, seqlens, p_hard: float, seed: int, steps: int, warmup: int, traffic=None):
    """Training forward+backward of duo-causal attention on one packed varlen batch."""
    import torch

    from tah_amd import ops
    from tests.cases import make_varlen_case, varlen_args
    from tests.gpu_util import to_device

    case = make_varlen_case(seed, seqlens, p_hard, std=0.5)
    dev = to_device(case)
    a = varlen_args(dev)
    g = torch.Generator().manual_seed(seed + 1)
    do1 = torch.randn(dev["q1"].shape, generator=g).to(torch.bfloat16).cuda()
    do2 = torch.randn(dev["q2"].shape, generator=g).to(torch.bfloat16).cuda()
    pairs = visible_pairs(case)
    fwd_flops = 4.0 * 128 * 16 * pairs
    sched = launch_order(ops, dev)
    mk = max(seqlens)  # what a caller knows of the batch: no sequence is longer (sizes the backward's dS workspace)
    ws_bytes = ops.duo_bwd_workspace_bytes(len(seqlens), 16, 8, dev["q1"].shape[0], dev["k1"].shape[0], dev["q2"].shape[0],
                                           dev["k2"].shape[0], mk, mk)

    def bwd(o1, lse1, o2, lse2, schedule, ds_workspace=None):
        return ops.duo_bwd_varlen(dev["q1"], dev["k1"], dev["v1"], o1, lse1, do1, dev["cu_q1"], dev["cu_k1"],
                                  dev["q2"], dev["k2"], dev["v2"], o2, lse2, do2, dev["pos_q2"], dev["pos_k2"],
                                  dev["cu_q2"], dev["cu_k2"], dev["scale"], schedule=schedule, ds_workspace=ds_workspace,
                                  max_seqlen_k1=mk, max_seqlen_k2=mk)

    bwd(*ops.duo_fwd_varlen(*a, schedule=sched), sched)  # (allocates the package's dS workspace outside the timed steps)
    yield  # inputs are resident; everything below runs when main() resumes the leg
    def other_way(schedule, ds_workspace):  # the same step in sequence order (no table) / with the three-kernel backward
        t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for i in range(warmup + steps):
            if i == warmup:
                t0.record()
            bwd(*ops.duo_fwd_varlen(*a, schedule=schedule), schedule, ds_workspace)
        t1.record()
        torch.cuda.synchronize()
        return t0.elapsed_time(t1) / steps
    in_sequence_order = lambda: other_way(None, None)

    if sched is not None:
        in_sequence_order()  # (measured again after the timed steps, so that neither order runs on a colder GPU)

    def step():
        bwd(*ops.duo_fwd_varlen(*a, schedule=sched), sched)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        step()
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / steps
    # the two halves on their own (events on the launch stream around each call)
    o1, lse1, o2, lse2 = ops.duo_fwd_varlen(*a, schedule=sched)
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
    half = {"fwd": 0.0, "bwd": 0.0}
    for _ in range(steps):
        ev[0].record()
        ops.duo_fwd_varlen(*a, schedule=sched)
        ev[1].record()
        bwd(o1, lse1, o2, lse2, sched)
        ev[2].record()
        torch.cuda.synchronize()
        half["fwd"] += ev[0].elapsed_time(ev[1]) / steps
        half["bwd"] += ev[1].elapsed_time(ev[2]) / steps
    tf = 3.5 * fwd_flops / (ms * 1e-3) / 1e12
    ms_three = other_way(sched, False)
    order = None
    if sched is not None:  # what one table costs to build (once per batch)
        order = {"table": "heaviest tile first across documents, built once per batch outside the timed region",
                 "table_build_ms": time_schedule_build(ops, dev), "ms_per_step_in_sequence_order": in_sequence_order()}
    return {"workload": name, "ms_per_step": ms, "launch_order": order, "visible_pairs_per_head": pairs, "flop_per_step": 3.5 * fwd_flops,
            "backward": {"path": "dS exchange: dK/dV kernel writes dS (bf16), dQ = scale * dS K reads it back (5 products per "
                                 "tile pair)", "ds_workspace_bytes": ws_bytes,
                         "ms_per_step_with_three_kernel_backward": ms_three,
                         "three_kernel_backward": "dQ and dK/dV each recompute S and dP (7 products per tile pair), no workspace"},
            "tflops": tf, "roofline": {"bound": "mfma", "achieved": tf, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                                       "frac": tf / PEAK_BF16_TFLOPS, "traffic": traffic,
                                       "kernels": "duo_fwd_kernel + duo_bwd_delta_kernel x2 + duo_bwd_dkdv_kernel (dS export) + "
                                                  "duo_bwd_dq_from_ds_kernel",
                                       "kernel_ms": {"forward (duo_fwd_kernel)": half["fwd"],
                                                     "backward (delta x2, dkdv + dS export, dq from dS)": half["bwd"]},
                                       "frac_forward": fwd_flops / (half["fwd"] * 1e-3) / 1e12 / PEAK_BF16_TFLOPS,
                                       "frac_backward": 2.5 * fwd_flops / (half["bwd"] * 1e-3) / 1e12 / PEAK_BF16_TFLOPS},
            "tokens_per_s": sum(seqlens) / (ms * 1e-3)}


def bench_host_layer_train_step(seqlens, p_hard: float, seed: int, steps: int, warmup: int, layers: int = 4):
    """The path a maintainer of the reference runs in training (tah_model.py:580-623 around HF attention layers): per
    decoder layer and latent iteration `build_attention_mask` (once per iteration) -> `TaHDuoCache.update` ->
    `duo_attention_forward`, both iterations, then `.backward()`, on configs[3]'s documents as a batch of padded rows
    with a valid mask -- against the bare packed-varlen launches (`ops.duo_fwd_varlen` + `ops.duo_bwd_varlen`) of the
    same rows."""
    import types

    import torch

    from tah_amd import ops
    from tah_amd.attention import build_attention_mask, duo_attention_forward
    from tah_amd.cache import TaHDuoCache
    from tah_amd.pack import gather_active
    from tests.cases import make_varlen_case, varlen_args
    from tests.gpu_util import to_device

    B, T, Hq, Hkv, D = len(seqlens), max(seqlens), 16, 8, 128
    g = torch.Generator().manual_seed(seed)
    valid = torch.zeros(B, T, dtype=torch.long)
    for b, n in enumerate(seqlens):
        valid[b, :n] = 1  # right-padded rows
    hard = (torch.rand(B, T, generator=g) < p_hard) & valid.bool()
    W = int(hard.sum(-1).max())  # width of the second iteration's pack: the most hard tokens of a row
    mk = lambda n, h: [(torch.randn(B, n, h, D, generator=g) * 0.5).to(torch.bfloat16).cuda().requires_grad_(True) for _ in range(layers)]
    # the projections of every layer as its q / k / v linears leave them: of all tokens at the first iteration, of the
    # packed hard tokens at the second (the model gathers the hidden states once per iteration, tah_model.py:600-603,
    # and every layer projects the gathered rows)
    q1, k1, v1, q2, k2, v2 = mk(T, Hq), mk(T, Hkv), mk(T, Hkv), mk(W, Hq), mk(W, Hkv), mk(W, Hkv)
    hidden = (torch.randn(B, T, 2048, generator=g) * 0.5).to(torch.bfloat16).cuda().requires_grad_(True)
    valid, hard = valid.cuda(), hard.cuda()
    pos = (torch.cumsum(valid, -1) - 1).clamp(min=0)
    w1 = torch.randn(B, T, Hq, D, generator=g).to(torch.bfloat16).cuda()
    wx = torch.randn(B, T, 2048, generator=g).to(torch.bfloat16).cuda()
    mods = [types.SimpleNamespace(layer_idx=l, num_key_value_groups=Hq // Hkv) for l in range(layers)]
    scale = D ** -0.5
    # the bare launches on the same rows, packed (one call serves both iterations)
    case = make_varlen_case(seed, list(seqlens), p_hard, std=0.5)
    dev = to_device(case)
    a = varlen_args(dev)
    do1 = torch.randn(dev["q1"].shape, generator=g).to(torch.bfloat16).cuda()
    do2 = torch.randn(dev["q2"].shape, generator=g).to(torch.bfloat16).cuda()
    sched = launch_order(ops, dev)
    yield

    def host_step():
        cache = TaHDuoCache()
        m0 = build_attention_mask(pos, valid, cache, 0, dtype=torch.bfloat16)
        cache.current_iter_depth, cache.position_ids_to_cache, cache.valid_mask_to_cache = 0, pos, valid
        outs = []
        for l in range(layers):
            k, v = cache.update(k1[l].transpose(1, 2), v1[l].transpose(1, 2), l)
            outs.append(duo_attention_forward(mods[l], q1[l].transpose(1, 2), k, v, m0, scaling=scale)[0])
        # second iteration: the hard tokens, packed per row (one index for all layers, as the model's loop has it)
        _, pos2, val2, x2 = gather_active(hard, pos, valid, hidden)
        outs.append(x2)
        gq, gk, gv = q2, k2, v2
        m1 = build_attention_mask(pos2, val2, cache, 1, dtype=torch.bfloat16)
        cache.current_iter_depth, cache.position_ids_to_cache, cache.valid_mask_to_cache = 1, pos2, val2
        for l in range(layers):
            k, v = cache.update(gk[l].transpose(1, 2), gv[l].transpose(1, 2), l)
            outs.append(duo_attention_forward(mods[l], gq[l].transpose(1, 2), k, v, m1, scaling=scale)[0])
        # upstream gradients as given (no loss arithmetic); the gathered hidden rows get theirs too (the scatter back)
        torch.autograd.backward(outs, [w1[:, : o.shape[1]] if o.dim() == 4 else wx[:, : o.shape[1]] for o in outs])
        for t in q1 + k1 + v1 + q2 + k2 + v2 + [hidden]:
            t.grad = None

    def bare_step():
        for _ in range(layers):
            o1, lse1, o2, lse2 = ops.duo_fwd_varlen(*a, schedule=sched)
            ops.duo_bwd_varlen(dev["q1"], dev["k1"], dev["v1"], o1, lse1, do1, dev["cu_q1"], dev["cu_k1"],
                               dev["q2"], dev["k2"], dev["v2"], o2, lse2, do2, dev["pos_q2"], dev["pos_k2"],
                               dev["cu_q2"], dev["cu_k2"], dev["scale"], schedule=sched, max_seqlen_k1=T, max_seqlen_k2=T)

    def timed(f):
        for _ in range(max(2, warmup // 2)):
            f()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            f()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / steps

    host_ms, bare_ms = timed(host_step), timed(bare_step)
    return {"workload": f"configs[3] as the host layer sees it: {B} rows padded to {T}, valid lengths {list(seqlens)}, "
                        f"p_hard={p_hard}, {layers} attention layers x 2 latent iterations, forward + backward",
            "path": "build_attention_mask -> TaHDuoCache.update -> duo_attention_forward (both iterations; gather_active of the hidden "
                    "states once for the second) -> backward(); wall clock, includes the packing of valid rows and autograd's own kernels",
            "ms_per_step": host_ms, "ms_per_layer": host_ms / layers,
            "bare_launches_ms_per_step": bare_ms, "bare_launches_ms_per_layer": bare_ms / layers,
            "ratio_to_bare_launches": host_ms / bare_ms, "layers": layers}


def device_clock():
    """Shader clock the device reports right now (rocm-smi), or None where the tool is not there."""
    import subprocess
    try:
        out = subprocess.run(["rocm-smi", "--showclocks"], capture_output=True, text=True, timeout=20).stdout
    except (OSError, subprocess.SubprocessError):
        return None
    for line in out.splitlines():
        if "sclk" in line and "(" in line:
            return line.split("(")[-1].split(")")[0]
    return None


def bench_device_context(steps: int):
    """What the 2.5 PFLOP/s figure means on the device at hand.  The shader clock follows the power the work draws,
    and that depends on the data: the same instruction stream runs faster on zeros than on random values.  This leg
    times (a) the library's own bf16 GEMM (8192^3, torch.matmul: no softmax, no masks, nothing but the matrix pipe
    and its operand traffic) and (b) the duo-causal forward and backward kernels of the headline shape, each on random
    data and on zeros, and reads the clock the device reports while each of them runs."""
    import threading

    import torch

    from tah_amd import ops
    from tests.cases import make_varlen_case, varlen_args
    from tests.gpu_util import to_device

    dev = to_device(make_varlen_case(1238, [8192], 0.06, std=0.5))
    g = torch.Generator().manual_seed(3)
    do1 = torch.randn(dev["q1"].shape, generator=g).to(torch.bfloat16).cuda()
    do2 = torch.randn(dev["q2"].shape, generator=g).to(torch.bfloat16).cuda()
    zero = dict(dev)
    for k in ("q1", "k1", "v1", "q2", "k2", "v2"):
        zero[k] = torch.zeros_like(dev[k])
    n = 8192
    mats = {"random": (torch.randn(n, n, device="cuda").to(torch.bfloat16), torch.randn(n, n, device="cuda").to(torch.bfloat16)),
            "zeros": (torch.zeros(n, n, device="cuda", dtype=torch.bfloat16), torch.zeros(n, n, device="cuda", dtype=torch.bfloat16))}
    yield

    def attention_calls(d, g1, g2):
        a = varlen_args(d)
        o1, lse1, o2, lse2 = ops.duo_fwd_varlen(*a)
        return (lambda: ops.duo_fwd_varlen(*a),
                lambda: ops.duo_bwd_varlen(d["q1"], d["k1"], d["v1"], o1, lse1, g1, d["cu_q1"], d["cu_k1"], d["q2"], d["k2"], d["v2"], o2,
                                           lse2, g2, d["pos_q2"], d["pos_k2"], d["cu_q2"], d["cu_k2"], d["scale"], max_seqlen_k1=8192,
                                           max_seqlen_k2=8192))

    def measure(fn):
        for _ in range(10):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / steps
        seen = []

        def sample():  # four readings, half a second apart (one reading is a snapshot of a clock that moves)
            for _ in range(4):
                seen.append(device_clock())
                time.sleep(0.5)

        th = threading.Thread(target=sample)
        th.start()
        while th.is_alive():  # keep the device at this work while the clock is read
            for _ in range(20):
                fn()
            torch.cuda.synchronize()
        th.join()
        return ms, seen

    out = {"what": "the same kernels on random data and on zeros, with the shader clock the device reports meanwhile; "
                   "2.5 PFLOP/s assumes 2.4 GHz", "library_bf16_gemm_8192": {}, "duo_fwd_seq8192": {}, "duo_bwd_seq8192": {}}
    for name, (a, b) in mats.items():
        ms, clk = measure(lambda: a @ b)
        out["library_bf16_gemm_8192"][name] = {"ms": ms, "tflops": 2.0 * n ** 3 / (ms * 1e-3) / 1e12, "sclk": clk}
    for name, (d, g1, g2) in {"random": (dev, do1, do2), "zeros": (zero, torch.zeros_like(do1), torch.zeros_like(do2))}.items():
        fwd, bwd = attention_calls(d, g1, g2)
        for key, fn in (("duo_fwd_seq8192", fwd), ("duo_bwd_seq8192", bwd)):
            ms, clk = measure(fn)
            out[key][name] = {"ms": ms, "sclk": clk}
    return out


def bench_qk_prep(steps: int, warmup: int):
    """q/k RMSNorm + rotary embedding + KV append for the prefill rows of configs[1] (B=4, T=4096): the
    step before the attention call.  HBM-bound: every q, k, v row is read and written once."""
    import torch

    from tah_amd.kv_cache import KvSlabs, qk_norm_rope
    from tests.qk_prep_cases import make_case, to_torch

    B, T, hq, hkv = 4, 4096, 16, 8
    rows = B * T
    c = make_case(1240, rows, hq, hkv, scale=0.5, max_pos=T)
    t = to_torch(c, "cuda")
    cu = torch.arange(0, rows + 1, T, dtype=torch.int32, device="cuda")
    # every step appends to slabs of its own (67 MB a set), so no step has to reset lengths first; beyond 64
    # steps the sets are used again and their lengths cleared on the way (one extra 4-element fill per 64 steps)
    nsets = min(steps + warmup, 64)
    sets = [KvSlabs(B, T, hkv, with_pos=False, device="cuda") for _ in range(nsets)]

    def step(i):
        slabs = sets[i % nsets]
        if i >= nsets:
            slabs.len.zero_()
        qk_norm_rope(t["q"], t["k"], t["qw"], t["kw"], t["cos"], t["sin"], c["eps"], v=t["v"], cache=slabs, cu_new=cu)

    yield  # inputs are resident; everything below runs when main() resumes the leg
    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(steps):
        step(warmup + i)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / steps
    # the backward of the preparation (training; no append): q, k and the two output gradients read, dq and dk written
    from tah_amd import _lib
    gq, gk = torch.randn_like(t["q"]), torch.randn_like(t["k"])
    bwd = lambda: _lib.lib().qk_prep_bwd(t["q"], t["k"], gq, gk, t["qw"], t["kw"], t["cos"], t["sin"], c["eps"], 4096)
    for _ in range(warmup):
        bwd()
    e0.record()
    for _ in range(steps):
        bwd()
    e1.record()
    torch.cuda.synchronize()
    bwd_ms = e0.elapsed_time(e1) / steps
    bwd_bytes = rows * (3 * (hq + hkv) * 256 + 2 * 256)
    # per token row: q, k, v read and q, K, V written (256 B per head), cos and sin rows read
    nbytes = rows * (2 * (hq + 2 * hkv) * 256 + 2 * 256)
    gbs = nbytes / (ms * 1e-3) / 1e9
    return {"workload": "step before attention for configs[1]: q/k RMSNorm + rotary + KV append, 16384 token rows, "
                        "Hq=16, Hkv=8, D=128 (fresh slabs every step)",
            "ms_per_step": ms, "algorithmic_bytes": nbytes, "hbm_gbs": gbs,
            "roofline": {"bound": "hbm", "achieved": gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": gbs / PEAK_HBM_GBS,
                         "traffic": measured_traffic("qk_prep_prefill"), "kernels": "qk_prep_kernel + kv_append_len_kernel"},
            "backward": {"kernel": "qk_prep_bwd_kernel", "ms_per_step": bwd_ms, "algorithmic_bytes": bwd_bytes,
                         "hbm_gbs": bwd_bytes / (bwd_ms * 1e-3) / 1e9, "frac": bwd_bytes / (bwd_ms * 1e-3) / 1e9 / PEAK_HBM_GBS},
            "tokens_per_s": rows / (ms * 1e-3)}


def bench_topk_mix(steps: int, warmup: int, rows: int = 1024, vocab: int = 151936, hidden: int = 2048, topk: int = 100):
    """Next-iteration input of hard tokens (tah_model.py:57-75): top-100 softmax mix of embedding rows for `rows` rows of
    the full vocabulary, and the top-k logit values alone (the decider's features, iter_decider.py:281) next to
    torch.topk on the same rows.  Per row the kernel reads the logits once and k embedding rows.  Also the learned
    decider's whole decision (iter_decider.py:265-301) for the 32 rows of a generation step, replayed from a graph as the
    engine runs it: its dense layers on tah_linear_rows, and on the library's GEMMs."""
    import torch

    from tah_amd import ops
    from tah_amd.decider import MLPIterDecider

    torch.manual_seed(1241)
    decider = MLPIterDecider(hidden_states_size=hidden).cuda().eval()
    g = torch.Generator().manual_seed(1241)
    logits = [(torch.randn(rows, vocab, generator=g) * 3).to(torch.bfloat16).cuda() for _ in range(2)]  # two sets in rotation
    emb = (torch.randn(vocab, hidden, generator=g) * 0.02).to(torch.bfloat16).cuda()
    out = torch.empty(rows, hidden, dtype=torch.bfloat16, device="cuda")
    feats = torch.randn(32, hidden * len(decider.hidden_states_layer_nums), generator=g).to(torch.bfloat16).cuda()
    yield

    def replayed(f, per_graph=10):
        """ms per call of f from a captured graph of `per_graph` calls."""
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):
            f()
            side.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                for _ in range(per_graph):
                    f()
            graph.replay()
            side.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(side)
            for _ in range(max(1, steps)):
                graph.replay()
            e1.record(side)
            side.synchronize()
        return e0.elapsed_time(e1) / (max(1, steps) * per_graph)

    def timed(f):
        for i in range(warmup):
            f(i)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(steps):
            f(i)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / steps

    mix_ms = timed(lambda i: ops.topk_mix(logits[i % 2], emb, topk, out=out))
    val_ms = timed(lambda i: ops.topk_values(logits[i % 2], topk))
    torch_ms = timed(lambda i: torch.topk(logits[i % 2], topk, dim=-1))
    decide = lambda: decider.decide_selected(logits[0][:32], 1, feats)
    decider_ms = replayed(decide)
    decider.fused_layers = False
    decider_library_ms = replayed(decide)
    nbytes = rows * (vocab * 2 + topk * hidden * 2 + hidden * 2)
    gbs = nbytes / (mix_ms * 1e-3) / 1e9
    return {"workload": f"top-{topk} softmax mix of embedding rows, {rows} rows of {vocab} bf16 logits, hidden {hidden} "
                        "(two sets of logits in rotation)",
            "ms_per_step": mix_ms, "algorithmic_bytes": nbytes, "hbm_gbs": gbs,
            "roofline": {"bound": "hbm", "achieved": gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": gbs / PEAK_HBM_GBS,
                         "traffic": measured_traffic("topk_mix") if (rows, vocab, hidden, topk) == (1024, 151936, 2048, 100) else None,
                         "kernels": "topk_mix_kernel<19>"},
            "topk_values_ms": val_ms, "torch_topk_ms": torch_ms, "rows_per_s": rows / (mix_ms * 1e-3),
            "learned_decider_32_rows": {"ms_per_decision": decider_ms, "ms_per_decision_with_library_gemms": decider_library_ms,
                                        "what": "MLPIterDecider.decide_selected (top-k values, 11 dense layers, threshold), "
                                                f"hidden {hidden}, replayed from a graph"}}


def bench_sample_rows(steps: int, warmup: int, vocab: int = 151936, temperature: float = 0.6, top_p: float = 0.95):
    """The draw of a generation step without a top-k filter (tah/model/utils.py:84-125): one tah_sample_rows launch over the
    32 rows of the end-to-end workload, next to the torch formulation it replaces (softmax, sort over the vocabulary,
    cumulative sum, scatter, renormalisation, draw), and over 1024 rows against the bytes of the logits."""
    import torch

    from tah_amd import ops
    from tah_amd.engine import TaHDecodeEngine

    g = torch.Generator().manual_seed(1242)
    logits = [(torch.randn(1024, vocab, generator=g) * 3).to(torch.bfloat16).cuda() for _ in range(2)]  # two sets in rotation
    u = torch.rand(1024, generator=g).cuda()
    out = torch.zeros(1024, dtype=torch.int64, device="cuda")
    # rows with a language model's range: the bulk of the vocabulary around -2 +- 2.5, twenty tokens 22 to 30 above it
    lm = torch.randn(32, vocab, generator=g) * 2.5 - 2.0
    lm.scatter_add_(1, torch.randint(0, vocab, (32, 20), generator=g), 22.0 + 8.0 * torch.rand(32, 20, generator=g))
    lm = lm.to(torch.bfloat16).cuda()
    yield

    def timed(f, n):
        for i in range(warmup):
            f(i)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(n):
            f(i)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / n

    ms32 = timed(lambda i: ops.sample_rows(logits[i % 2][:32], u[:32], temperature, top_p=top_p, out=out[:32]), steps)
    torch32 = timed(lambda i: TaHDecodeEngine.sample(logits[i % 2][:32].float(), temperature, top_p=top_p), max(3, steps // 4))
    ms32_lm = timed(lambda i: ops.sample_rows(lm, u[:32], temperature, top_p=top_p, out=out[:32]), steps)
    ms1024 = timed(lambda i: ops.sample_rows(logits[i % 2], u, temperature, top_p=top_p, out=out), steps)
    nbytes = 1024 * vocab * 2
    gbs = nbytes / (ms1024 * 1e-3) / 1e9
    return {"workload": f"temperature {temperature} / top_p {top_p} draw without a top-k filter, rows of {vocab} bf16 logits",
            "ms_per_step_32_rows": ms32, "torch_ms_per_step_32_rows": torch32,
            "ms_per_step_32_rows_with_a_language_models_range": ms32_lm,
            "ms_per_step": ms1024, "rows": 1024, "algorithmic_bytes": nbytes, "hbm_gbs": gbs,
            "roofline": {"bound": "hbm", "achieved": gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": gbs / PEAK_HBM_GBS,
                         "traffic": None, "kernels": "sample_rows_kernel<19, false>"},
            "rows_per_s": 1024 / (ms1024 * 1e-3)}


def bench_e2e_decode(new_tokens: int, B: int = 32, prompt_len: int = 512, temperature: float = 0.0, top_p: float = 0.95, top_k: int = 0):
    """BASELINE configs[4]: end-to-end TaH decode, Qwen3-1.7B architecture with random weights, a two-layer MLP
    decider whose threshold is set so that about 6 % of the prompt tokens iterate, batch 32, 512-token prompts.
    One HIP graph replay per generated token (both latent iterations, sampling included)."""
    import torch

    from tah_amd.engine import EngineConfig, TaHDecodeEngine, Weights

    cfg = EngineConfig()
    w = Weights.random_init(cfg, "cuda", seed=1239)
    extra_steps = 40  # replays of the step without its attention kernels, after the timed generation
    eng = TaHDecodeEngine(w, B, prompt_len + new_tokens + 8 + extra_steps, device="cuda")
    g = torch.Generator().manual_seed(1239)
    ids = torch.randint(0, cfg.vocab, (B * prompt_len,), generator=g).cuda()
    cu = torch.arange(0, B * prompt_len + 1, prompt_len, dtype=torch.int32, device="cuda")
    yield  # weights and prompts are resident; everything below runs when main() resumes the leg
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    first, hard = eng.prefill(ids, cu, calibrate=0.06)
    torch.cuda.synchronize()
    prefill_s = time.perf_counter() - t0
    # the generation: greedy, rows at different latent iterations share a batch (one captured tick per replay; a row's
    # token costs it one tick, or two when it is hard), the host looks every 8 ticks whether all rows have their tokens
    draw = dict(temperature=temperature, top_p=top_p, top_k=top_k) if temperature > 0.0 else {}
    eng.capture_ticks(-1, new_tokens, **draw)  # (graph capture is set-up, like the engine's buffers)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    toks = eng.generate(first, new_tokens, use_graph=True, **draw)
    torch.cuda.synchronize()
    gen_s = time.perf_counter() - t0
    ticks = eng.ticks
    n_tokens = int(eng.n_steps)
    assert n_tokens == B * (new_tokens - 1) and int(eng.out_len.min()) == new_tokens
    frac_hard = int(eng.n_hard) / max(n_tokens, 1)
    step_ms = gen_s * 1e3 / ticks
    ctx = float(eng.pos.float().mean())
    # one tick at the final context, with and without the attention launches, all rows busy; and launched from Python
    eng.finished.zero_()
    eng.out_len.zero_()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    n_probe = (extra_steps - 10) // 3

    def ticks_ms(without_attention: bool, graph: bool):
        eng.measure_without_attention = without_attention
        eng._tick_graphs = None
        graphs = eng.capture_ticks(-1, eng.max_len) if graph else None
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        e0.record()
        for i in range(n_probe):
            if graphs is not None:
                graphs[i % 2].replay()
            else:
                eng._tick(i % 2, -1, eng.max_len)
        e1.record()
        host = (time.perf_counter() - t0) / n_probe
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / n_probe, host * 1e3

    with_ms, _ = ticks_ms(False, True)
    # what a replay costs the host when the queue is empty
    enqueue = []
    for i in range(5):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        eng._tick_graphs[i % 2].replay()
        enqueue.append(time.perf_counter() - t0)
    eager_ms, host_eager_ms = ticks_ms(False, False)
    without_ms, _ = ticks_ms(True, True)
    eng.measure_without_attention = False
    eng._tick_graphs = None
    attn_ms = max(with_ms - without_ms, 0.0)
    attn_bytes = cfg.layers * B * ctx * 2 * cfg.hkv * cfg.head_dim * 2
    params = sum(t.numel() for L in w.layers for k, t in L.items() if not k.endswith("_p")) + w.embed.numel() + w.norm.numel()
    return {"workload": "configs[4]: end-to-end TaH decode, Qwen3-1.7B architecture (28 layers, hidden 2048, 16/8 heads, "
                        f"vocab 151936), random weights, B={B}, {prompt_len}-token prompts, {new_tokens} generated tokens, "
                        + (f"sampling at temperature {temperature}, top-p {top_p}, top-k {top_k}" if temperature > 0.0 else "greedy sampling")
                        + ", MLP decider 2048->512->1 thresholded at the 94th percentile of the prompt tokens",
            "tokens_per_s": n_tokens / gen_s, "ms_per_step": step_ms, "steps_timed": ticks,
            "schedule": "every replay is one pass of all rows, each at the latent iteration its own token needs next "
                        "(a hard token costs its row two passes, any other one); the loop that keeps the batch in step "
                        "costs two passes per token",
            "tokens_per_pass": n_tokens / ticks, "passes_per_token_of_the_slowest_row": ticks / (new_tokens - 1),
            "hard_fraction_decode": frac_hard, "hard_fraction_prompt": float(hard.float().mean()),
            "pass_ms_at_final_context": with_ms, "attention_ms_per_pass_at_final_context": attn_ms,
            "attention_share_of_pass_at_final_context": attn_ms / with_ms, "pass_ms_without_attention_kernels": without_ms,
            "attention_kernels": "duo_decode_step_kernel<2> (q/k preparation + append + attention), 28 layers",
            "attention_cache_bytes_per_pass_at_final_context": attn_bytes, "attention_cache_gbs": attn_bytes / (attn_ms * 1e-3) / 1e9,
            "host_enqueue_ms_per_replay": sorted(enqueue)[2] * 1e3, "eager_ms_per_pass": eager_ms, "host_ms_per_pass_eager": host_eager_ms,
            "prefill_s": prefill_s, "weight_bytes": params * 2, "mean_context_at_end": ctx}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--e2e-tokens", type=int, default=1024, help="generated tokens of the end-to-end decode leg")
    ap.add_argument("--e2e-temperature", type=float, default=0.0,
                    help="end-to-end decode leg: sample at this temperature with top-p 0.95 instead of greedy decoding")
    ap.add_argument("--e2e-top-k", type=int, default=0, help="with --e2e-temperature: top-k filter (0: none)")
    ap.add_argument("--spinup", type=int, default=200,
                    help="untimed launches of the headline kernel before its warm-up steps (the GPU's clock needs tens of "
                         "milliseconds of work to leave its idle state)")
    ap.add_argument("--only", choices=["all", "fwd", "decode", "fwd_bwd", "host_layer", "context", "qk_prep", "topk_mix", "sample_rows", "e2e"], default="all",
                    help="profiling aid: run only one leg (the JSON line then lacks the other legs)")
    ap.add_argument("--calib-copy", action="store_true",
                    help="profiling aid: also run one plain 256 MiB device copy (known traffic for counter scaling)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no sharding, no collectives); use --gpus 1", file=sys.stderr)
        return 2

    import torch

    from tah_amd import ops
    from tests.cases import make_varlen_case, varlen_args
    from tests.gpu_util import to_device

    seed, B, T, p = 1235, 4, 4096, 0.06
    case = make_varlen_case(seed, [T] * B, p, std=0.5)
    dev = to_device(case)
    a = varlen_args(dev)
    pairs = visible_pairs(case)
    flops = 4.0 * 128 * 16 * pairs

    if args.calib_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda")
        src.clone()
        torch.cuda.synchronize()
    # Two phases.  First every leg builds its inputs (host-side generation, copies to HBM); then everything runs back
    # to back: the headline, the forward+backward legs, decode, q/k preparation, and the end-to-end decode last.
    # The order matters because the clock does: a freshly started process finds the GPU at idle clocks, and they fall
    # back within milliseconds whenever the GPU waits for the host, so the host work is done beforehand and the
    # headline starts with `spinup` untimed launches (60 ms) on top of its `warmup` steps; and seconds of sustained
    # memory streaming (the end-to-end leg) leave the chip at a lower clock for whatever follows (the same forward
    # launches read 5-10 % slower right after it), so that leg runs last.  `sustained` below is the headline kernel over
    # about half a second of back-to-back launches, for comparison with the 20 timed steps.
    legs = []
    if args.only in ("all", "fwd_bwd"):
        legs.append(("fwd_bwd_seq8192_p06", bench_fwd_bwd(
            "north-star headline: fwd+bwd, one sequence of 8192, p_hard=0.06, Hq=16, Hkv=8, D=128", [8192], 0.06, 1238,
            args.steps, args.warmup, measured_traffic("fwd_bwd_seq8192_p06"))))
        legs.append(("fwd_bwd_4docs_p10", bench_fwd_bwd(
            "configs[3]: fwd+bwd, 8192 packed tokens in 4 documents, p_hard=0.10", [1397, 3210, 2561, 1024], 0.10, 1237,
            args.steps, args.warmup, measured_traffic("fwd_bwd_4docs_p10"))))
    if args.only in ("all", "host_layer"):
        legs.append(("host_layer_train_step", bench_host_layer_train_step([1397, 3210, 2561, 1024], 0.10, 1237,
                                                                          max(3, args.steps // 4), args.warmup)))
    if args.only in ("all", "decode"):
        legs.append(("decode", bench_decode(args.steps, args.warmup)))
    if args.only in ("all", "context"):
        legs.append(("device_context", bench_device_context(args.steps)))
    if args.only in ("all", "qk_prep"):
        legs.append(("qk_prep_prefill", bench_qk_prep(args.steps, args.warmup)))
    if args.only in ("all", "topk_mix"):
        legs.append(("topk_mix", bench_topk_mix(args.steps, args.warmup)))
    if args.only in ("all", "sample_rows"):
        legs.append(("sample_rows", bench_sample_rows(args.steps, args.warmup)))
    if args.only in ("all", "e2e"):
        legs.append(("e2e_decode", bench_e2e_decode(args.e2e_tokens, temperature=args.e2e_temperature, top_k=args.e2e_top_k)))
    for _, leg in legs:
        next(leg)  # runs the leg up to its `yield`: inputs built and resident
    sched = launch_order(ops, dev)
    torch.cuda.synchronize()

    fwd_steps = args.steps if args.only in ("all", "fwd") else 1
    fwd_warmup = args.warmup if args.only in ("all", "fwd") else 1
    spinup = args.spinup if args.only in ("all", "fwd") else 0
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    def in_sequence_order():  # for comparison: the tiles in sequence order (no table)
        for i in range(fwd_warmup + fwd_steps):
            if i == fwd_warmup:
                ev0.record()
            ops.duo_fwd_varlen(*a)
        ev1.record()
        torch.cuda.synchronize()
        return ev0.elapsed_time(ev1) / fwd_steps

    for _ in range(spinup):
        ops.duo_fwd_varlen(*a, schedule=sched)
    in_sequence_order()  # (measured again after the timed steps, so that neither order runs on a colder GPU)
    for _ in range(fwd_warmup):
        ops.duo_fwd_varlen(*a, schedule=sched)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ev0.record()
    for _ in range(fwd_steps):
        ops.duo_fwd_varlen(*a, schedule=sched)
    ev1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_wall = wall * 1e3 / fwd_steps           # the K timed steps between two synchronisations: `ms_per_step` and `value`
    ms = ev0.elapsed_time(ev1) / fwd_steps    # the same launches by HIP events on their stream: the roofline's kernel time
    tflops = flops / (ms * 1e-3) / 1e12
    value = flops / (ms_wall * 1e-3) / 1e12
    ms_sequence_order = in_sequence_order()
    sustained = None
    if args.only in ("all", "fwd"):
        n_sus = 1500
        ev0.record()
        for _ in range(n_sus):
            ops.duo_fwd_varlen(*a, schedule=sched)
        ev1.record()
        torch.cuda.synchronize()
        ms_sus = ev0.elapsed_time(ev1) / n_sus
        sustained = {"launches": n_sus, "ms_per_step": ms_sus, "tflops": flops / (ms_sus * 1e-3) / 1e12}
    table_build_ms = time_schedule_build(ops, dev) if args.only in ("all", "fwd") else None
    extra = {}
    for name, leg in legs:
        try:
            next(leg)
            raise RuntimeError(f"leg {name} yielded twice")
        except StopIteration as done:
            extra[name] = done.value

    out = {
        "metric": "duo-causal attn TFLOP/s (% bf16 MFMA peak) prefill; decode HBM GB/s",
        "value": value, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_wall, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "timing": {"value_and_ms_per_step": "wall clock of the timed steps between two device synchronisations",
                   "roofline": "HIP events on the launch stream around the same steps (kernel_ms)",
                   "untimed_launches_before_the_timed_steps": spinup + 2 * fwd_warmup + fwd_steps,
                   "of_which": {"spinup": spinup, "warmup": fwd_warmup, "same_kernel_in_sequence_order": fwd_warmup + fwd_steps}},
        "config": {"workload": "configs[1]: duo-causal prefill forward, B=4, T=4096, Hq=16, Hkv=8, D=128, p_hard=0.06",
                   "visible_pairs_per_head": pairs, "flop_per_step": flops, "tokens_per_s": B * T / (ms_wall * 1e-3),
                   "launch_order": {"table": "heaviest tile first across the 4 sequences (tah_duo_schedule_build), built once "
                                             "per batch outside the timed region: one table serves all 28 layers",
                                    "table_build_ms": table_build_ms, "ms_per_step_in_sequence_order": ms_sequence_order},
                   "spinup_launches": spinup, "sustained": sustained},
        "roofline": {"bound": "mfma", "achieved": tflops, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": tflops / PEAK_BF16_TFLOPS, "traffic": measured_traffic("prefill_fwd"), "kernel": "duo_fwd_kernel<2, false, 4>",
                     "kernel_ms": ms},
    }
    out["extra"] = extra
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(seed, T, p)
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
