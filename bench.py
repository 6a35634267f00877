#!/usr/bin/env python3
"""Benchmark of the packed decode-attention hot path on one MI355X.

A "step" is one decode step of the attention hot path over every layer of the workload:
the fused flash-decoding kernel reads the whole packed cache (all layers, all KV heads) once
for one query per layer and writes out [L*H_q,128] + lse.  Inputs are synthetic, seeded, and
resident in HBM before the timed region.  Default workload: configuration 1 (Llama-3.1-8B
shapes, 32 layers, 32k context, per-head Dirichlet bit allocation).

Prints ONE JSON line: the headline on configuration 1 with
`roofline` and `cpu_baseline`, and beside it compact figures of the other configurations
(`configs`), the one-layer-per-call form (`sequential`), the reference-layout entry points
(`padded`), the prefill packer (`pack`, `select`) and the whole-model decode loops (`decode_loop`).
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

HBM_PEAK_GBPS = 8000.0
# HBM bytes per launch of the fused kernel by workload configuration, from two rocprofv3 --pmc runs
# of `python3 bench.py --config N --fused-only` (FETCH_SIZE x 2.000 and WRITE_SIZE x 1.000, the
# factors a plain copy kernel of known size gives in the same runs).  A constant read off the named
# profile summary, not something a run of this script observes: it goes stale when the layout
# changes, which is why the JSON names its source.
MEASURED_TRAFFIC = {
    1: (1122714583, "profiles/decode_fused_kernel_c1_llama31_8b_32k.txt"),
    2: (2856765295, "profiles/decode_fused_kernel_c2_mistral_7b_128k.txt"),
    3: (11114367255, "profiles/decode_fused_kernel_c3_qwen25_72b_128k.txt"),
}
PACK_SAMPLE_LAYERS = 8                      # layers of one sequence packed back to back for the pack throughput


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--config", type=int, default=1, help="workload configuration 0..4 (default 1)")
    ap.add_argument("--layers", type=int, default=None, help="override the layer count (debug)")
    ap.add_argument("--context", type=int, default=None, help="override the context length (debug)")
    ap.add_argument("--batch", type=int, default=None, help="override the batch (config 4)")
    ap.add_argument("--work-kib", type=int, default=None,
                    help="streamed KiB per work item, one workgroup each (default: balanced resident groups)")
    ap.add_argument("--groups-per-cu", type=int, default=1, help="workgroups per compute unit")
    ap.add_argument("--no-graph", action="store_true", help="do not time the graph-replayed step")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-dense", action="store_true")
    ap.add_argument("--no-check", action="store_true")
    ap.add_argument("--no-configs", action="store_true", help="skip the compact figures of the other configurations")
    ap.add_argument("--configs", type=str, default="0,2,3,4", help="configurations of the compact block")
    ap.add_argument("--fused-only", action="store_true",
                    help="only build the workload and run the fused step (for profiling): prints a short JSON")
    ap.add_argument("--sequential-only", action="store_true",
                    help="only the one-layer-per-call leg (for profiling): prints its JSON and exits")
    ap.add_argument("--padded-only", action="store_true",
                    help="only the reference-layout entry points on one layer (for profiling): prints its JSON")
    ap.add_argument("--pack-only", action="store_true",
                    help="only the prefill pack of one sequence of the workload (for profiling): prints its JSON")
    ap.add_argument("--knapsack-only", action="store_true",
                    help="only the V knapsack of the selection over 1, 8 and all layers' score rows per launch "
                         "(for profiling): prints its JSON")
    ap.add_argument("--no-decode-loop", action="store_true",
                    help="skip the whole-model greedy decode loop (random-weight Llama-3.1-8B-shaped model)")
    return ap.parse_args()


def time_region(fn, steps, torch):
    """HIP-event time of `steps` back-to-back calls on the current stream (ms per call)."""
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(steps):
        fn()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / steps


def graph_of(fn, torch):
    """`fn` (which neither allocates nor synchronizes once warm) captured on a side stream; returns
    (graph, stream).  Time `graph.replay` inside `with torch.cuda.stream(stream)`."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()                                  # workspaces of this stream exist before capture
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            fn()
        for _ in range(3):
            graph.replay()
        torch.cuda.synchronize()
    return graph, side


# ---------------------------------------------------------------------------------------------
# workload construction and the fused step
# ---------------------------------------------------------------------------------------------
def build_workload(cfg, dev, torch, on_first=None, pack_sample=None):
    """Pack every (sequence, layer) of `cfg` with the HIP packer.  Returns the list of
    (packed layer, new_v_only, q).  `on_first(K, V, q, vb, kb)` sees the fp16 inputs of layer 0 of
    sequence 0; `pack_sample` (a list) receives (K, V, vb, kb) of the first layers of sequence 0."""
    from rdkv_amd import packing, synth
    groups = []
    for seq in range(cfg.batch):
        for layer in range(cfg.layers):
            vb, kb, oc = synth.layer_allocation(cfg, layer, seq)
            K, V, q = synth.layer_data(cfg, layer, dev, seq, outliers=oc)
            pl, nvo = packing.pack_layer_per_head(K, V, vb, kb, cfg.G)
            groups.append((pl, nvo, q))
            if seq == 0 and layer == 0 and on_first is not None:
                on_first(K, V, q, vb, kb)
            if pack_sample is not None and seq == 0 and layer < PACK_SAMPLE_LAYERS and cfg.layers > 1:
                pack_sample.append((K, V, vb, kb))
            del K, V
    return groups


def fused_step_times(cache, qs, out, lse, steps, warmup, torch, graph=True, rounds=5):
    """The timed regions of the fused step, `rounds` times in alternation so that clock and
    temperature drift reach all of them alike, the median of each kind reported:
      (a) `steps` steps through ``decode_attn_fused`` (streaming launch + merge launch, eagerly
          issued), bracketed by events and synchronization: ms per step, the headline;
      (b) the same steps issued as the library's two calls with a HIP event on the same stream
          before and after every streaming launch: the mean in-step interval is the duration of the
          streaming kernel inside a step (it cannot exceed the step of its own region; the events
          themselves cost that region ~3 %, which is why (a) is the headline);
      (c) `steps` launches of the streaming kernel alone, back to back.
    Beside them the step replayed from a HIP graph.  Returns (step, ms_step, ms_kernel, extras)."""
    import numpy as np
    from rdkv_amd import _lib, stream_cache
    lib = _lib.load()
    dev = qs.device

    def step():
        stream_cache.decode_attn_fused(cache, qs, out, lse)

    # untimed: the W warm-up steps, then keep stepping for ~0.3 s so that the device clocks have
    # ramped before the timed region (a 0.3 ms step is far shorter than the governor's window)
    for _ in range(max(warmup, 1)):
        step()
    torch.cuda.synchronize()
    t_ramp = time.time()
    while time.time() - t_ramp < 0.3:
        for _ in range(20):
            step()
        torch.cuda.synchronize()
    ws = _lib.workspace(dev, lib.rdkv_decode_fused_workspace_bytes(cache.n_work, cache.G))
    stream = _lib.stream_of(dev)
    q_dt = _lib.DTYPE_CODE[qs.dtype]

    def partials_only():
        _lib.check(lib.rdkv_decode_fused_partials(
            None, cache.units.data_ptr(), cache.n_units, cache.work.data_ptr(), cache.n_work,
            _lib.ptr(cache.groups), cache.n_groups, cache.row_dwords_arg, qs.data_ptr(), q_dt, qs.stride(0),
            cache.G, None, None, 0, ws.data_ptr(), ws.numel(), stream))

    def merge_only():
        _lib.check(lib.rdkv_decode_fused_merge(cache.units.data_ptr(), cache.n_units, cache.n_work, cache.G,
                                               out.data_ptr(), out.stride(0), lse.data_ptr(), ws.data_ptr(),
                                               ws.numel(), stream))

    before = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    after = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)

    def evented_region():
        torch.cuda.synchronize()
        start.record()
        for i in range(steps):
            before[i].record()
            partials_only()
            after[i].record()
            merge_only()
        end.record()
        torch.cuda.synchronize()
        return start.elapsed_time(end) / steps, sum(a.elapsed_time(b) for a, b in zip(before, after)) / steps

    plain, ev_step, ev_kernel, alone = [], [], [], []
    for _ in range(rounds):
        plain.append(time_region(step, steps, torch))
        es, ek = evented_region()
        ev_step.append(es)
        ev_kernel.append(ek)
        alone.append(time_region(partials_only, steps, torch))
    med = lambda v: float(np.median(v))
    extras = {"timing_rounds": rounds, "ms_per_step_regions": plain,
              "ms_per_step_with_inner_events": med(ev_step), "ms_per_launch_kernel_alone": med(alone),
              "ms_per_step_graph_replay": None}
    if graph:
        g, side = graph_of(step, torch)
        with torch.cuda.stream(side):
            extras["ms_per_step_graph_replay"] = time_region(g.replay, steps, torch)
        torch.cuda.current_stream().wait_stream(side)
        # the same step eight times per graph: what a replay costs beyond its kernels is paid once per
        # replay, not once per launch, so it shrinks with the number of steps a graph holds
        per_graph = 8

        def eight_steps():
            for _ in range(per_graph):
                step()
        g8, side = graph_of(eight_steps, torch)
        with torch.cuda.stream(side):
            extras["ms_per_step_graph_replay_8_steps_per_graph"] = (
                time_region(g8.replay, max(steps // per_graph, 3), torch) / per_graph)
        torch.cuda.current_stream().wait_stream(side)
    return step, med(plain), med(ev_kernel), extras


def oracle_layer(pl, nvo, torch):
    """The packed layer as the NumPy oracle's dataclass over the same bytes."""
    import dataclasses
    from oracle import rdkv_oracle as O
    kw = {}
    for f in dataclasses.fields(O.PackedKVLayer):
        v = getattr(pl, f.name)
        kw[f.name] = v.detach().cpu().numpy() if torch.is_tensor(v) else v
    return O.PackedKVLayer(**kw), (nvo.cpu().numpy() if nvo is not None else None)


def check_layer0(first_pl, first_nvo, q0, got, torch):
    """Layer 0 of what was timed against the CPU oracle (tolerance of the parity tests)."""
    import numpy as np
    from oracle import rdkv_oracle as O
    ora, ora_nvo = oracle_layer(first_pl, first_nvo, torch)
    exp_out, _, _ = O.decode_attn_ref(q0, ora, ora_nvo)
    err = float(np.abs(got - exp_out).max())
    return {"layer0_max_abs_err": err, "layer0_ref_max_abs": float(np.abs(exp_out).max()),
            "within_tolerance": bool(err <= 2e-3 and err <= 1e-2 * np.abs(exp_out).max())}


def compact_config(index, args, torch, dev):
    """One configuration measured the same way as the headline, in short: build, eager step,
    streaming kernel alone, layer-0 check.  Configuration 4 also packs one whole sequence (all
    its layers) from resident fp16 K/V: its second metric."""
    import numpy as np
    from rdkv_amd import packing, stream_cache, synth
    cfg = synth.CONFIGS[index]
    t0 = time.time()
    sample = [] if index == 4 else None
    groups = build_workload(cfg, dev, torch)
    qs = torch.cat([g[2] for g in groups]).contiguous()
    cache = stream_cache.build_stream_cache([(g[0], g[1]) for g in groups], cfg.G)
    first_pl, first_nvo = groups[0][0], groups[0][1]
    del groups
    torch.cuda.empty_cache()
    torch.cuda.synchronize()
    build_s = time.time() - t0
    out = torch.empty(cache.rows, 128, dtype=torch.float32, device=dev)
    lse = torch.empty(cache.rows, dtype=torch.float32, device=dev)
    steps = max(5, min(args.steps, int(2000 / max(cache.algorithmic_bytes / 6e9, 0.01))))   # ~2 s at most
    _, ms_eager, ms_kernel, _ = fused_step_times(cache, qs, out, lse, steps, args.warmup, torch, graph=False, rounds=3)
    algo = cache.algorithmic_bytes
    n_groups = cfg.batch * cfg.layers
    res = {"workload": cfg.name, "layers": cfg.layers, "batch": cfg.batch, "context": cfg.context, "G": cfg.G,
           "steps": steps, "ms_per_step": ms_eager, "ms_per_launch_fused_kernel": ms_kernel,
           "algorithmic_bytes_per_step": algo, "GBps": algo / (ms_eager * 1e-3) / 1e9,
           "frac_step": algo / (ms_eager * 1e-3) / 1e9 / HBM_PEAK_GBPS,
           "frac_kernel": algo / (ms_kernel * 1e-3) / 1e9 / HBM_PEAK_GBPS,
           "us_per_sequence_layer": ms_eager * 1e3 / n_groups, "work_items": cache.n_work,
           "kernel_variant_max_row_dwords": cache.max_row_dwords,
           "kernel_variant_row_shape": [cache.row_shape >> 16, (cache.row_shape >> 8) & 255, cache.row_shape & 255]
           if cache.row_shape else None,
           "compression_ratio": synth.dense_fp16_bytes(cfg) * n_groups / algo, "build_seconds": build_s}
    if not args.no_check:
        res["check"] = check_layer0(first_pl, first_nvo, qs[:cfg.H_q].cpu().numpy(), out[:cfg.H_q].cpu().numpy(), torch)
    del cache, out, lse, qs, first_pl, first_nvo
    torch.cuda.empty_cache()
    if index == 4:
        res["pack_one_sequence"] = pack_sequence_section(cfg, torch, dev)
    if index in (2, 3):
        # the long-context configurations through the reference-layout entry points as well
        pad = padded_section(cfg, torch, dev, layers=2, steps=10)
        res["padded_us_per_layer"] = {k: v["us_per_layer"] for k, v in pad.items() if isinstance(v, dict)}
    return res


# ---------------------------------------------------------------------------------------------
# the prefill packer
# ---------------------------------------------------------------------------------------------
def pack_sequence_section(cfg, torch, dev, seq=0):
    """One sequence's full prefill cache (every layer of sequence `seq`) packed from resident fp16
    K and V: wall time of `packing.pack_layers_per_head`, as GB/s of the fp16 input read once."""
    import numpy as np
    from rdkv_amd import packing, synth
    Ks, Vs, vbs, kbs = [], [], [], []
    for layer in range(cfg.layers):
        vb, kb, oc = synth.layer_allocation(cfg, layer, seq)
        K, V, _ = synth.layer_data(cfg, layer, dev, seq, outliers=oc)
        Ks.append(K), Vs.append(V), vbs.append(vb), kbs.append(kb)
    vb_all, kb_all = torch.stack(vbs).to(dev), torch.stack(kbs).to(dev)
    times = []
    for _ in range(4):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        packing.pack_layers_per_head(Ks, Vs, vb_all, kb_all, cfg.G)
        torch.cuda.synchronize()
        times.append((time.perf_counter() - t0) * 1e3)
    in_bytes = sum(2 * k.numel() * k.element_size() for k in Ks)
    ms = float(np.median(times[1:]))
    # the same layers straight into the streaming format (rdkv_pack_layer_stream), eight layers per call
    from rdkv_amd import stream_cache
    vbs_dev, kbs_dev = [v.to(dev) for v in vbs], [k.to(dev) for k in kbs]
    times = []
    for _ in range(4):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for first in range(0, cfg.layers, 8):
            c = stream_cache.build_stream_cache_from_kv(
                [(Ks[l], Vs[l], vbs_dev[l], kbs_dev[l]) for l in range(first, min(first + 8, cfg.layers))], cfg.G)
            del c
        torch.cuda.synchronize()
        times.append((time.perf_counter() - t0) * 1e3)
    ms_stream = float(np.median(times[1:]))
    return {"layers": cfg.layers, "tokens": int(Ks[0].shape[2]), "fp16_input_bytes": in_bytes, "pack_ms": ms,
            "pack_ms_per_layer": ms / cfg.layers, "pack_GBps_of_fp16_input": in_bytes / (ms * 1e-3) / 1e9,
            "pack_to_stream_ms_per_layer": ms_stream / cfg.layers,
            "pack_to_stream_GBps_of_fp16_input": in_bytes / (ms_stream * 1e-3) / 1e9,
            "note": "packing.pack_layers_per_head over all layers of one sequence, and "
                    "stream_cache.build_stream_cache_from_kv over the same layers eight at a time; wall time, "
                    "median of 3 after 1 warm-up"}


def pack_layer_sections(cfg, K, V, vb, kb, args, torch, dev):
    """Layer 0: wall time of the whole-layer packer and of the re-layout, and of the prefill
    selection feeding the packer (pooling, per-head V knapsack, per-head K allocation, pack)."""
    import numpy as np
    from rdkv_amd import knapsack_solver, obkv_fast, packing, stream_cache
    # the allocations are inputs like K and V: resident on the device before the timed region (a
    # prefill hands them over from the selection kernels; as host tensors their upload alone is 0.1 ms)
    vb, kb = vb.to(dev), kb.to(dev)
    pack_ms, relayout_ms = [], []
    for _ in range(6):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        pl_t, nvo_t = packing.pack_layer_per_head(K, V, vb, kb, cfg.G)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        stream_cache.build_stream_cache([(pl_t, nvo_t)], cfg.G)
        torch.cuda.synchronize()
        pack_ms.append((t1 - t0) * 1e3)
        relayout_ms.append((time.perf_counter() - t1) * 1e3)
    del pl_t, nvo_t
    # the same call repeated on its own (K and V still in the memory-side cache from the call before,
    # no re-layout in between)
    again = []
    for _ in range(6):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        pl_t = packing.pack_layer_per_head(K, V, vb, kb, cfg.G)
        torch.cuda.synchronize()
        again.append((time.perf_counter() - t0) * 1e3)
    del pl_t
    in_bytes = 2 * K.numel() * K.element_size()
    pack_info = {"fp16_input_bytes_per_layer": in_bytes,
                 "pack_ms_per_layer": float(np.median(pack_ms[1:])),
                 "pack_GBps_of_fp16_input": in_bytes / (float(np.median(pack_ms[1:])) * 1e-3) / 1e9,
                 "pack_ms_per_layer_repeated": float(np.median(again[1:])),
                 "relayout_ms_per_layer": float(np.median(relayout_ms[1:])),
                 "note": "wall time of packing.pack_layer_per_head (+ stream_cache.build_stream_cache) "
                         "on layer 0 (fp16 K, V and the bit allocations resident on the device), median of 5 "
                         "after 1 warm-up, each pack following a re-layout; pack_ms_per_layer_repeated: the pack "
                         "call alone, repeated; K is read twice (min/max pass, then emit)"}
    # seeded log-normal scores; the budget is a quarter of the context, half of it for K
    gsel = torch.Generator().manual_seed(4242)
    H_kv, T_ctx = int(K.shape[1]), int(K.shape[2])
    tok_scores = torch.exp(torch.randn(H_kv, T_ctx, generator=gsel) * 1.5 + 2.0).to(dev)
    ch_scores = torch.exp(torch.randn(H_kv, 128, generator=gsel)).to(dev)
    sel_kw = dict(gqa_factor=cfg.G, token_budget=max(T_ctx // 4, 1), k_budget_ratio=0.5, obs_window=32,
                  pool_kernel_size=7, pool_padding="reflect", pool_type="avg", v_bit_options=None,
                  k_bit_options=torch.tensor([0.0, 2.0, 4.0, 8.0]),
                  eps_V=knapsack_solver.DEFAULT_EPSILON_V, eps_K=knapsack_solver.DEFAULT_EPSILON_K)
    sel_ms, stages = [], {}
    for _ in range(6):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        obkv_fast._perhead_select_and_pack_joint(K, V, tok_scores, ch_scores, **sel_kw)
        torch.cuda.synchronize()
        sel_ms.append((time.perf_counter() - t0) * 1e3)
    obkv_fast._perhead_select_and_pack_joint(K, V, tok_scores, ch_scores, timing=stages, **sel_kw)
    select_info = {"select_and_pack_ms_per_layer": float(np.median(sel_ms[1:])),
                   "stages_ms": {k: round(v, 4) for k, v in stages.items()},
                   "rows": H_kv, "tokens_per_row": T_ctx,
                   "note": "wall time of obkv_fast._perhead_select_and_pack_joint on layer 0 (median of "
                           "5 after 1 warm-up); stages from one extra call that synchronizes after "
                           "each stage (quantization_ms = the whole-layer packer)"}
    if not args.no_cpu_baseline:
        from oracle import select_oracle
        t0 = time.perf_counter()
        select_oracle.select_joint(
            tok_scores.cpu().numpy(), ch_scores.cpu().numpy(), head_dim=128,
            token_budget=sel_kw["token_budget"], k_budget_ratio=0.5, pool_kernel_size=7,
            pool_padding="reflect", k_bit_options=(0, 2, 4, 8))
        select_info["cpu_oracle_allocation_ms"] = (time.perf_counter() - t0) * 1e3
        select_info["gpu_allocation_ms"] = float(sum(v for k, v in stages.items()
                                                     if k in ("pooling_ms", "v_allocation_ms", "k_allocation_ms")))
    return pack_info, select_info


def pack_sample_section(pack_sample, pack_info, cfg, torch, dev, select_info=None):
    """The first layers of a sequence packed back to back (one planning launch and one host read
    for all of them, the host side of a layer overlapping the kernels of the one before)."""
    import numpy as np
    from rdkv_amd import packing
    vb_all = torch.stack([p[2] for p in pack_sample]).to(dev)
    kb_all = torch.stack([p[3] for p in pack_sample]).to(dev)
    times = []
    for _ in range(4):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        packing.pack_layers_per_head([p[0] for p in pack_sample], [p[1] for p in pack_sample], vb_all, kb_all, cfg.G)
        torch.cuda.synchronize()
        times.append((time.perf_counter() - t0) * 1e3)
    sample_bytes = sum(2 * p[0].numel() * p[0].element_size() for p in pack_sample)
    pack_info["pack_layers_sample"] = len(pack_sample)
    pack_info["pack_ms_per_layer_batched"] = float(np.median(times[1:])) / len(pack_sample)
    pack_info["pack_GBps_of_fp16_input_batched"] = sample_bytes / (float(np.median(times[1:])) * 1e-3) / 1e9
    # the streaming re-layout of the same layers in one call (one unit table, one partition)
    from rdkv_amd import stream_cache
    packed = packing.pack_layers_per_head([p[0] for p in pack_sample], [p[1] for p in pack_sample], vb_all, kb_all, cfg.G)
    times = []
    for _ in range(4):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        stream_cache.build_stream_cache(packed, cfg.G)
        torch.cuda.synchronize()
        times.append((time.perf_counter() - t0) * 1e3)
    pack_info["relayout_ms_per_layer_batched"] = float(np.median(times[1:])) / len(pack_sample)
    del packed
    # the same layers from fp16 K / V straight into the streaming format (rdkv_pack_layer_stream):
    # quantization and layout in one pass, the cache ready for the fused kernel
    entries = [(p[0], p[1], p[2].to(dev), p[3].to(dev)) for p in pack_sample]
    times = []
    for _ in range(6):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        c = stream_cache.build_stream_cache_from_kv(entries, cfg.G)
        torch.cuda.synchronize()
        times.append((time.perf_counter() - t0) * 1e3)
        del c
    pack_info["pack_to_stream_ms_per_layer_batched"] = float(np.median(times[1:])) / len(pack_sample)
    pack_info["pack_to_stream_GBps_of_fp16_input_batched"] = \
        sample_bytes / (float(np.median(times[1:])) * 1e-3) / 1e9
    pack_info["pack_then_relayout_ms_per_layer_batched"] = \
        pack_info["pack_ms_per_layer_batched"] + pack_info["relayout_ms_per_layer_batched"]
    pack_info["note_pack_to_stream"] = (
        "pack_to_stream_*: stream_cache.build_stream_cache_from_kv over the sample layers (fp16 K / V and bit "
        "allocations -> streaming cache, wall time incl. the work partition and table uploads, median of 5 after 1 "
        "warm-up); pack_then_relayout_*: the two-step path it replaces (pack_layers_per_head, then build_stream_cache)")
    if select_info is not None:
        # selection + packing of the same layers in one call: the knapsack launches see
        # layers x heads rows at once instead of one layer's heads
        from rdkv_amd import knapsack_solver, obkv_fast
        gsel = torch.Generator().manual_seed(4243)
        Ks, Vs = [p[0] for p in pack_sample], [p[1] for p in pack_sample]
        H_kv, T_ctx = int(Ks[0].shape[1]), int(Ks[0].shape[2])
        tok = [torch.exp(torch.randn(H_kv, T_ctx, generator=gsel) * 1.5 + 2.0).to(dev) for _ in Ks]
        chn = [torch.exp(torch.randn(H_kv, 128, generator=gsel)).to(dev) for _ in Ks]
        sel_kw = dict(gqa_factor=cfg.G, token_budget=max(T_ctx // 4, 1), k_budget_ratio=0.5, obs_window=32,
                      pool_kernel_size=7, pool_padding="reflect", pool_type="avg", v_bit_options=None,
                      k_bit_options=torch.tensor([0.0, 2.0, 4.0, 8.0]),
                      eps_V=knapsack_solver.DEFAULT_EPSILON_V, eps_K=knapsack_solver.DEFAULT_EPSILON_K)
        times = []
        for _ in range(4):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            obkv_fast._perhead_select_and_pack_layers(Ks, Vs, tok, chn, **sel_kw)
            torch.cuda.synchronize()
            times.append((time.perf_counter() - t0) * 1e3)
        select_info["select_and_pack_layers_sample"] = len(pack_sample)
        select_info["select_and_pack_ms_per_layer_batched"] = float(np.median(times[1:])) / len(pack_sample)


# ---------------------------------------------------------------------------------------------
# one layer per call, and the reference-layout entry points
# ---------------------------------------------------------------------------------------------
def knapsack_rows_section(cfg, torch, dev, steps=20):
    """The V allocation of the prefill-time selection (knapsack_solver.knapsack_allocate: one workgroup per
    score row) with the rows of 1, 8 and all layers of the workload in one launch pair: a single layer's
    H_kv rows leave most compute units idle, the rows of a prompt's layers together fill them."""
    from rdkv_amd import knapsack_solver as ks
    g = torch.Generator(device="cpu").manual_seed(4242)
    T, H = cfg.context, cfg.H_kv
    budget = 4.0                                            # bits per element: a quarter of fp16
    out = {"workload": cfg.name, "tokens_per_row": T, "rows_per_layer": H,
           "budget_bits_per_element": budget, "launches": []}
    for layers in (1, 8, cfg.layers):
        rows = layers * H
        scores = torch.exp(torch.randn(rows, T, generator=g) * 1.5 + 2.0).to(dev)
        bud = torch.full((rows,), budget, device=dev)

        def call():
            ks.knapsack_allocate(scores, bud, ks.DEFAULT_EPSILON_V, group_rows=H, with_counts=True)
        for _ in range(3):
            call()
        ms = time_region(call, steps, torch)
        out["launches"].append({"layers": layers, "rows": rows, "us_per_call": ms * 1e3,
                                "us_per_layer": ms * 1e3 / layers})
        del scores
    return out


def sequential_section(cfg, torch, dev, layers=8, replays=50):
    """One layer per call, the form a sequential model loop issues: `layers` single-layer streaming
    caches (distinct buffers, 280 MB together: more than the last-level cache), their fused calls
    recorded one after the other into one HIP graph, the graph replayed back to back - as two
    launches per call and as one (the merge inside the streaming launch).  Beside it the same number
    of bytes per launch read by a plain streaming kernel, the floor of any single launch of this size."""
    import numpy as np
    from rdkv_amd import _lib, packing, stream_cache, synth
    lib = _lib.load()
    caches, qs, outs = [], [], []
    for layer in range(layers):
        vb, kb, oc = synth.layer_allocation(cfg, layer)
        K, V, q = synth.layer_data(cfg, layer, dev, outliers=oc)
        pl, nvo = packing.pack_layer_per_head(K, V, vb, kb, cfg.G)
        del K, V
        c = stream_cache.build_stream_cache([(pl, nvo)], cfg.G)
        caches.append(c)
        qs.append(q)
        outs.append((torch.empty(c.rows, 128, device=dev), torch.empty(c.rows, device=dev)))
    res = {"layers_rotated": layers, "context": cfg.context}
    algo = float(np.mean([c.algorithmic_bytes for c in caches]))
    for name, one in (("two_launches", False), ("one_launch", True)):
        def all_layers():
            for c, q, (o, l) in zip(caches, qs, outs):
                stream_cache.decode_attn_fused(c, q, o, l, one_launch=one)
        g, side = graph_of(all_layers, torch)
        with torch.cuda.stream(side):
            us_graph = time_region(g.replay, replays, torch) / layers * 1e3
            us_eager = time_region(all_layers, replays, torch) / layers * 1e3
        torch.cuda.current_stream().wait_stream(side)
        res[name] = {"us_per_layer_graph_replay": us_graph, "us_per_layer_eager": us_eager,
                     "GBps_graph_replay": algo / us_graph / 1e3,
                     "frac_hbm_peak_graph_replay": algo / us_graph / 1e3 / HBM_PEAK_GBPS}
    default_one = caches[0].n_work <= stream_cache.ONE_LAUNCH_MAX_WORK
    res["default_form"] = "one_launch" if default_one else "two_launches"
    res["us_per_layer_sequential"] = res[res["default_form"]]["us_per_layer_graph_replay"]
    res["frac_hbm_peak"] = res[res["default_form"]]["frac_hbm_peak_graph_replay"]
    # a plain read of the same number of bytes per launch, rotated over as many distinct buffers
    nbytes = int(np.mean([c.stream_bytes for c in caches])) // 4096 * 4096
    bufs = [torch.empty(nbytes, dtype=torch.uint8, device=dev).random_(0, 255) for _ in range(layers)]
    sink = torch.zeros(1024, dtype=torch.uint8, device=dev)

    def plain_reads():
        st = _lib.stream_of(dev)
        for b in bufs:
            _lib.check(lib.rdkv_probe_read_stream(b.data_ptr(), nbytes, 16 * 1024, sink.data_ptr(), st))
    g, side = graph_of(plain_reads, torch)
    with torch.cuda.stream(side):
        us_read = time_region(g.replay, replays, torch) / layers * 1e3
    torch.cuda.current_stream().wait_stream(side)
    res.update({"algorithmic_bytes_per_layer": algo, "streamed_bytes_per_layer": nbytes,
                "plain_read_us_per_launch": us_read, "plain_read_GBps": nbytes / us_read / 1e3,
                "workgroups_per_layer": caches[0].n_groups or caches[0].n_work,
                "work_items_per_layer": caches[0].n_work,
                "note": "one layer per call, calls of distinct layers back to back in one replayed HIP graph; "
                        "plain_read = a streaming read kernel over the same number of bytes per launch"})
    return res


def padded_section(cfg, torch, dev, steps=50, layers=4):
    """The three reference entry points on the reference layout (k_mixed_qk_dot_into, the masked
    softmax, v_dequant_weighted_sum_dispatch_into), each timed alone over `layers` distinct layers of
    the workload in rotation, against its algorithmic bytes (per-head counts, no padding)."""
    import numpy as np
    from rdkv_amd import _lib, packing, stream_cache, synth
    from rdkv_amd.fast_decode import _pre_squeeze_packed
    from rdkv_amd.k_kernel import k_mixed_qk_dot_into
    from rdkv_amd.v_kernel import v_dequant_weighted_sum_dispatch_into
    lib = _lib.load()
    items = []
    k_bytes = v_bytes = s_bytes = 0
    for layer in range(layers):
        vb, kb, oc = synth.layer_allocation(cfg, layer)
        K, V, q = synth.layer_data(cfg, layer, dev, outliers=oc)
        pl, nvo = packing.pack_layer_per_head(K, V, vb, kb, cfg.G)
        del K, V
        sp = _pre_squeeze_packed((pl,))[0]
        T_v = int(sp.T_eff)
        T_old = int(sp.T_eff_k) if sp.T_eff_k > 0 else T_v
        # a scores buffer with 256-byte aligned rows, as a decode loop keeps it (the reference slices
        # one buffer of its longest bucket, fast_decode.py:1397-1403)
        scores = torch.empty(cfg.H_q, -(-T_old // 64) * 64, dtype=torch.float32, device=dev)[:, :T_old]
        out = torch.empty(cfg.H_q, 128, dtype=torch.float32, device=dev)
        items.append((q.float(), sp, nvo[0].contiguous() if nvo is not None else None, T_v, T_old, scores, out))
        tok, ch = stream_cache._layer_counts(pl, cfg.H_kv)
        for (n2, n4, n8, n16), (c2, c4, c8) in zip(tok, ch):
            kept = n2 + n4 + n8 + n16
            k_bytes += kept * (-(-c2 // 4) + -(-c4 // 2) + c8) + 4 * (c2 + c4 + c8) + cfg.G * kept * 4
            v_bytes += 32 * n2 + 64 * n4 + 128 * n8 + 4 * (n2 + n4 + n8) + 256 * n16 + cfg.G * kept * 4
            s_bytes += cfg.G * kept * 4 * 2 + kept * 4
        k_bytes += cfg.H_q * 128 * 4
        v_bytes += cfg.H_q * 128 * 4
    k_bytes, v_bytes, s_bytes = k_bytes / layers, v_bytes / layers, s_bytes / layers

    def run_k():
        for q32, sp, _, _, T_old, scores, _ in items:
            k_mixed_qk_dot_into(q32, sp, T_old, scores)

    def run_softmax():
        st = _lib.stream_of(dev)
        ws = _lib.workspace(dev, lib.rdkv_softmax_rows_workspace_bytes(cfg.H_q))
        for _, sp, _, _, T_old, scores, _ in items:
            mask = sp.softmax_mask
            _lib.check(lib.rdkv_softmax_rows_ws(
                scores.data_ptr(), scores.stride(0), _lib.ptr(mask), mask.stride(0) if mask is not None else 0,
                T_old, None, 0, 0, scores.data_ptr(), scores.stride(0), None, 0, cfg.H_q, ws.data_ptr(), ws.numel(), st))

    def run_v():
        for _, sp, v16, T_v, _, scores, out in items:
            v_dequant_weighted_sum_dispatch_into(scores, sp, out, V16=v16, n_v16_per_head=sp.n_v16_per_head, max_T_v=T_v)

    res = {"layers_rotated": layers, "context": cfg.context}
    for name, fn, nbytes in (("k_mixed_qk_dot_into", run_k, k_bytes), ("softmax_rows", run_softmax, s_bytes),
                             ("v_dequant_weighted_sum_dispatch_into", run_v, v_bytes)):
        fn()
        us = time_region(fn, steps, torch) / layers * 1e3
        res[name] = {"us_per_layer": us, "algorithmic_bytes_per_layer": nbytes, "GBps": nbytes / us / 1e3,
                     "frac_hbm_peak": nbytes / us / 1e3 / HBM_PEAK_GBPS}
    res["us_per_layer_total"] = sum(res[k]["us_per_layer"] for k in
                                    ("k_mixed_qk_dot_into", "softmax_rows", "v_dequant_weighted_sum_dispatch_into"))
    res["note"] = ("the reference's K / softmax / V call sequence on PackedKVLayer tensors, eager launches; bytes: "
                   "codes + scale/zp + query + fp32 scores written (K), fp32 weights read + codes + scale/zp + "
                   "fp16 zone B + out (V), scores read and written + mask (softmax)")
    return res


# ---------------------------------------------------------------------------------------------
# whole-model decode loops (beside the headline, never as it)
# ---------------------------------------------------------------------------------------------
def decode_loop_section(cfg, torch, dev, tokens=48):
    """ms per generated token of ``fast_decode.greedy_decode_fast`` on a random-weight model of the
    Llama-3.1-8B shape (32 layers, hidden 4096, 32 / 8 heads) over a packed cache of the
    workload's shape: the whole-model figure the reference quotes for its loop (its only
    published latency, triton_v_kernel.py:53-54).  Reported beside the headline, never as it."""
    from transformers import LlamaConfig, LlamaForCausalLM
    from rdkv_amd import fast_decode, packing, synth
    L = 32
    mcfg = LlamaConfig(hidden_size=4096, intermediate_size=14336, num_hidden_layers=L, num_attention_heads=cfg.H_q,
                       num_key_value_heads=cfg.H_kv, head_dim=cfg.D, vocab_size=128256,
                       max_position_embeddings=262144, rms_norm_eps=1e-5, rope_theta=500000.0,
                       tie_word_embeddings=False)
    torch.manual_seed(0)
    with torch.device(dev):
        model = LlamaForCausalLM(mcfg).half().eval()
    sc = synth.scaled(cfg, layers=L)
    layers, v16 = [], []
    for i in range(L):
        vb, kb, oc = synth.layer_allocation(sc, i)
        K, V, _ = synth.layer_data(sc, i, dev, outliers=oc)
        pl, nvo = packing.pack_layer_per_head(K, V, vb, kb, sc.G)
        layers.append(pl)
        v16.append(nvo)
        del K, V
    cache = packing.TriZoneCache(tuple(layers), v16, [None] * L, [None] * L, sc.context)
    first = torch.randn(mcfg.vocab_size, device=dev)
    res = {"model": "Llama-3.1-8B shape, random fp16 weights", "context": sc.context, "tokens": tokens}
    for name, graph in (("eager", False), ("graph", True)):
        best = None
        for _ in range(2):          # the first run builds the streaming caches and warms the libraries
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            ids = fast_decode.greedy_decode_fast(model, cache, first, tokens, [], dev, sc.context,
                                                 use_cuda_graph=graph)
            torch.cuda.synchronize()
            dt = (time.perf_counter() - t0) / max(len(ids), 1) * 1e3
            best = dt if best is None else min(best, dt)
        res[f"ms_per_token_{name}"] = best
    # the blockwise variant: the generated tokens are re-compressed in blocks of 128 (budget 16)
    import contextlib
    import io
    from rdkv_amd import blockwise_decode as bw, knapsack_solver as ks
    conf = bw.BlockwiseRDKVConfig(
        block_size=128, block_budget_tokens=16, k_budget_ratio=0.5, obs_window=32, pool_kernel_size=5,
        pool_padding="reflect", v_bit_options=torch.tensor([0., 2, 4, 8, 16]),
        k_bit_options=torch.tensor([0., 2, 4, 8]), epsilon_v=ks.DEFAULT_EPSILON_V, epsilon_k=ks.DEFAULT_EPSILON_K)
    n_bw = 272
    for name, graph in (("blockwise", False), ("blockwise_graph", True)):
        for _ in range(2):
            with contextlib.redirect_stdout(io.StringIO()):       # the loop logs one event line per block
                ids, report = bw.greedy_decode_blockwise(
                    model=model, dual_cache=cache, next_token_logits=first, max_new_tokens=n_bw, eos_token_ids=[],
                    primary_device=dev, decode_position_start=sc.context, config=conf, use_cuda_graph=graph)
        ts = report["per_token_timestamps_ms"]
        steps = sorted(b - a for a, b in zip(ts, ts[1:]))
        res[name] = {"tokens": len(ids), "block_size": 128, "block_budget_tokens": 16,
                     "ms_per_token_avg": report["avg_tpot_ms"], "ms_per_token_median": steps[len(steps) // 2],
                     "ms_slowest_step": steps[-1], "compressed_blocks": report["num_compressed_decode_blocks"],
                     "final_flush_ms": report["final_flush_time_ms"]}
    return res


# ---------------------------------------------------------------------------------------------
# CPU baseline
# ---------------------------------------------------------------------------------------------
def cpu_baseline_section(ora, ora_nvo, q0, H_q, torch):
    """The reference's dequantize-then-attend path on layer 0 of the workload, on the box's host
    cores, in two restatements: ``torch_port`` (oracle/torch_port.py: the same op sequence on torch
    CPU tensors, the library the reference computes in; one call on one thread, and one call on all
    of this process's cores through the library's own thread pool) and ``numpy_port`` (the NumPy
    oracle: one call pinned to one core, and one call per core at a time as concurrent threads).
    2 warm-ups + 3 repeats, median (the protocol of run_latency.py:107-108).  The top-level value
    is the torch port on one core."""
    import numpy as np
    from concurrent.futures import ThreadPoolExecutor
    from threadpoolctl import threadpool_limits
    from oracle import rdkv_oracle as O
    from oracle import torch_port as TP
    layer_bytes = O.algorithmic_bytes(ora, H_q)
    cpus = sorted(os.sched_getaffinity(0))
    env_threads = os.environ.get("OMP_NUM_THREADS")
    n_all = min(len(cpus), int(env_threads)) if env_threads and env_threads.isdigit() else len(cpus)

    def timed(fn, warm=2, reps=3):
        for _ in range(warm):
            fn()
        ts = []
        for _ in range(reps):
            t0 = time.perf_counter()
            fn()
            ts.append(time.perf_counter() - t0)
        return float(np.median(ts))

    def one_numpy():
        return O.decode_attn_ref(q0, ora, ora_nvo)

    tl = TP.TorchLayer(ora, ora_nvo)
    q_t = torch.from_numpy(q0)

    def one_torch():
        return TP.decode_attn(q_t, tl)

    torch_threads_before = torch.get_num_threads()
    try:
        with threadpool_limits(limits=1):
            torch.set_num_threads(1)
            os.sched_setaffinity(0, {cpus[0]})
            try:
                t1_np = timed(one_numpy)
                t1_t = timed(one_torch)
            finally:
                os.sched_setaffinity(0, set(cpus))
            # NumPy on all cores: n_all oracle calls in flight, each on a thread of its own, library
            # pools still 1 per call (NumPy's elementwise loops are single-threaded)
            with ThreadPoolExecutor(max_workers=n_all) as ex:
                def wave():
                    list(ex.map(lambda _: one_numpy(), range(n_all)))
                t_all_np = timed(wave, warm=1, reps=3)
        # torch on all cores: ONE call, the library's intra-op pool at n_all threads
        torch.set_num_threads(n_all)
        t_all_t = timed(one_torch)
        torch_threads_all = torch.get_num_threads()
    finally:
        torch.set_num_threads(torch_threads_before)
    print(f"bench.py: cpu baseline threads: 1-core legs 1 thread on cpu {cpus[0]}; NumPy all-cores leg {n_all} "
          f"concurrent calls; torch all-cores leg one call, torch.get_num_threads()={torch_threads_all}",
          file=sys.stderr)

    def leg(seconds, cores, calls=1):
        return {"value": calls * layer_bytes / seconds / 1e9, "unit": "GB/s", "cores": cores,
                "ms_per_layer": seconds * 1e3 / calls}

    protocol = "2 warm-ups + 3 repeats, median"
    torch_leg = dict(leg(t1_t, 1), kind="port", library=f"torch {torch.__version__} CPU",
                     sample=f"oracle/torch_port.decode_attn on layer 0 of the workload ({layer_bytes} algorithmic "
                            f"bytes), {protocol}; torch.set_num_threads(1), calling thread pinned to one CPU",
                     all_cores=dict(leg(t_all_t, n_all), sample=f"one call, torch.set_num_threads({n_all}), {protocol}"))
    numpy_leg = dict(leg(t1_np, 1), kind="port", library=f"numpy {np.__version__}",
                     sample=f"oracle/rdkv_oracle.decode_attn_ref on the same layer, {protocol}; calling thread pinned "
                            f"to one CPU, library thread pools limited to 1",
                     all_cores=dict(leg(t_all_np, n_all, calls=n_all),
                                    sample=f"{n_all} concurrent calls (one thread each), 1 warm-up + 3 repeats, median"))
    return dict(torch_leg, torch_port=torch_leg, numpy_port=numpy_leg, host_cpus=os.cpu_count(),
                cpus_of_this_process=len(cpus), torch_num_threads=torch.get_num_threads())


def main():
    args = parse()
    default_workload = (args.layers is None and args.context is None and args.batch is None
                        and args.work_kib is None and args.groups_per_cu == 1)
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU only (the hot path shards by KV head / sequence "
              "without any exchange; no multi-GPU figure is produced). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    import numpy as np
    import torch

    from rdkv_amd import _lib, stream_cache, synth

    if not _lib.available():
        import __graft_entry__
        __graft_entry__.build()
    assert torch.cuda.is_available(), "bench.py needs a HIP device"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    lib = _lib.load()

    cfg = synth.CONFIGS[args.config]
    cfg = synth.scaled(cfg, context=args.context, layers=args.layers, batch=args.batch)
    if args.sequential_only:
        print(json.dumps(sequential_section(cfg, torch, dev, replays=args.steps)))
        return
    if args.padded_only:
        print(json.dumps(padded_section(cfg, torch, dev, steps=args.steps)))
        return
    if args.pack_only:
        print(json.dumps(pack_sequence_section(cfg, torch, dev)))
        return
    if args.knapsack_only:
        print(json.dumps(knapsack_rows_section(cfg, torch, dev, steps=args.steps)))
        return
    t_build = time.time()
    first = {}
    pack_sample = []

    def on_first(K, V, q, vb, kb):
        if not args.fused_only:
            first["pack"], first["select"] = pack_layer_sections(cfg, K, V, vb, kb, args, torch, dev)

    groups = build_workload(cfg, dev, torch, on_first=on_first, pack_sample=None if args.fused_only else pack_sample)
    pack_info, select_info = first.get("pack"), first.get("select")
    if len(pack_sample) > 1:
        pack_sample_section(pack_sample, pack_info, cfg, torch, dev, select_info)
    pack_sample.clear()
    qs = torch.cat([g[2] for g in groups]).contiguous()
    cache = stream_cache.build_stream_cache([(g[0], g[1]) for g in groups], cfg.G,
                                            work_bytes=args.work_kib * 1024 if args.work_kib else None,
                                            groups_per_cu=args.groups_per_cu)
    first_pl, first_nvo = groups[0][0], groups[0][1]
    del groups
    torch.cuda.empty_cache()
    torch.cuda.synchronize()
    t_build = time.time() - t_build
    n_groups = cfg.batch * cfg.layers

    out = torch.empty(cache.rows, 128, dtype=torch.float32, device=dev)
    lse = torch.empty(cache.rows, dtype=torch.float32, device=dev)
    step, ms_step_eager, ms_kernel, step_extras = fused_step_times(
        cache, qs, out, lse, args.steps, args.warmup, torch, graph=not args.no_graph)
    # the headline is the eagerly issued step (two launches per step), the mode every run reports;
    # the graph-replayed step stands beside it
    ms_step = ms_step_eager
    ms_step_graph = step_extras["ms_per_step_graph_replay"]
    algo = cache.algorithmic_bytes
    if args.fused_only:
        # one plain copy of known size in the same process: the launch against which a profiler run
        # of this command scales its traffic counters
        probe = torch.empty(2, 1 << 30, dtype=torch.uint8, device=dev)
        _lib.check(lib.rdkv_probe_copy(probe[0].data_ptr(), probe[1].data_ptr(), 1 << 30, _lib.stream_of(dev)))
        torch.cuda.synchronize()
        print(json.dumps({"workload": cfg.name, "ms_per_step_eager": ms_step_eager, "ms_per_launch_fused_kernel": ms_kernel,
                          "algorithmic_bytes_per_step": algo, "streamed_bytes_per_step": cache.stream_bytes,
                          "frac_kernel": algo / (ms_kernel * 1e-3) / 1e9 / HBM_PEAK_GBPS}))
        return
    stream = _lib.stream_of(dev)

    # plain copy kernel of known size (1 GiB in, 1 GiB out): reference launch for scaling the
    # hardware traffic counters of a profiler run of this same command
    probe_bytes = 1 << 30
    probe_src = torch.empty(probe_bytes, dtype=torch.uint8, device=dev).random_(0, 255)
    probe_dst = torch.empty_like(probe_src)
    _lib.check(lib.rdkv_probe_copy(probe_src.data_ptr(), probe_dst.data_ptr(), probe_bytes, stream))
    ms_copy = time_region(lambda: _lib.check(lib.rdkv_probe_copy(
        probe_src.data_ptr(), probe_dst.data_ptr(), probe_bytes, stream)), 5, torch)
    sink = torch.zeros(1024, dtype=torch.uint8, device=dev)
    ms_read_plain = time_region(lambda: _lib.check(lib.rdkv_probe_read(
        probe_src.data_ptr(), probe_bytes, 256 * 1024, sink.data_ptr(), stream)), 5, torch)
    ms_read_stream = time_region(lambda: _lib.check(lib.rdkv_probe_read_stream(
        probe_src.data_ptr(), probe_bytes, 256 * 1024, sink.data_ptr(), stream)), 5, torch)
    ms_read = min(ms_read_plain, ms_read_stream)

    # The same step with the cache hierarchy flushed before every step (a 1 GiB sweep of
    # unrelated memory): back-to-back steps re-read the same packed cache, and part of it
    # can be served from the 256 MB last-level cache; in a full decode loop the weights
    # stream through between the attention layers.
    cold = []
    for _ in range(10):
        _lib.check(lib.rdkv_probe_read(probe_src.data_ptr(), probe_bytes, 256 * 1024, sink.data_ptr(), stream))
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        step()
        e1.record()
        torch.cuda.synchronize()
        cold.append(e0.elapsed_time(e1))
    ms_step_cold = float(np.median(cold))
    del probe_src, probe_dst

    # ---- equivalent dense fp16 cache of the full context -----------------------------------
    # (a) lower bound for ANY dense kernel: its bytes at this device's measured read ceiling;
    # (b) torch's fused SDPA on real dense fp16 tensors of the same shape, all layers distinct.
    dense_bytes = synth.dense_fp16_bytes(cfg) * n_groups
    read_ceiling = probe_bytes / (ms_read * 1e-3)
    dense = {"bytes_per_step": dense_bytes, "ideal_ms_at_read_ceiling": dense_bytes / read_ceiling * 1e3,
             "sdpa_ms": None}
    if not args.no_dense and cfg.batch == 1 and dense_bytes < 64e9:
        try:
            import torch.nn.functional as F
            T = cfg.context
            K_all = torch.randn(cfg.layers, 1, cfg.H_kv, T, cfg.D, device=dev, dtype=torch.float16)
            V_all = torch.randn(cfg.layers, 1, cfg.H_kv, T, cfg.D, device=dev, dtype=torch.float16)
            Kd, Vd = list(K_all), list(V_all)
            qd = qs.view(cfg.layers, 1, cfg.H_q, 1, cfg.D)

            def dense_step():
                for i in range(cfg.layers):
                    F.scaled_dot_product_attention(qd[i], Kd[i], Vd[i], enable_gqa=True)

            dense_step()
            dense["sdpa_ms"] = time_region(dense_step, max(3, args.steps // 5), torch)
            # the same dense cache through this library's own dense fp16 flash-decoding kernel (two
            # launches per layer): a dense kernel that does run near the read ceiling
            if cfg.G in (4, 8):
                chunks = 32
                ws_d = torch.empty(lib.rdkv_probe_dense_decode_workspace_bytes(cfg.H_q, chunks), dtype=torch.uint8,
                                   device=dev)
                out_d = torch.empty(cfg.layers, cfg.H_q, cfg.D, dtype=torch.float32, device=dev)
                q16 = qs.half().view(cfg.layers, cfg.H_q, cfg.D)

                def dense_hip_step():
                    for i in range(cfg.layers):
                        _lib.check(lib.rdkv_probe_dense_decode(
                            q16[i].data_ptr(), Kd[i].data_ptr(), Vd[i].data_ptr(), T, cfg.H_kv, cfg.G, chunks,
                            out_d[i].data_ptr(), ws_d.data_ptr(), ws_d.numel(), stream))

                dense_hip_step()
                dense["dense_hip_kernel_ms"] = time_region(dense_hip_step, max(3, args.steps // 5), torch)
                dense["dense_hip_kernel_GBps"] = dense_bytes / (dense["dense_hip_kernel_ms"] * 1e-3) / 1e9
                # ... and with all layers in one launch (+ one merge), the form the packed step is timed in
                heads_all = cfg.layers * cfg.H_kv
                chunks_all = max(1, min(32, 2048 // heads_all))
                ws_all = torch.empty(lib.rdkv_probe_dense_decode_workspace_bytes(heads_all * cfg.G, chunks_all),
                                     dtype=torch.uint8, device=dev)

                def dense_hip_one_launch():
                    _lib.check(lib.rdkv_probe_dense_decode(
                        q16.data_ptr(), K_all.data_ptr(), V_all.data_ptr(), T, heads_all, cfg.G, chunks_all,
                        out_d.data_ptr(), ws_all.data_ptr(), ws_all.numel(), stream))

                out_layers = out_d.clone()
                dense_hip_one_launch()
                torch.cuda.synchronize()
                dense["dense_hip_one_launch_max_abs_diff_vs_per_layer"] = float((out_d - out_layers).abs().max())
                dense["dense_hip_kernel_one_launch_ms"] = time_region(dense_hip_one_launch, max(3, args.steps // 5), torch)
                dense["dense_hip_kernel_one_launch_GBps"] = dense_bytes / (dense["dense_hip_kernel_one_launch_ms"] * 1e-3) / 1e9
                del ws_all
            del Kd, Vd, K_all, V_all
        except Exception as e:  # the comparison is informative; never fail the benchmark on it
            dense["sdpa_error"] = repr(e)[:200]

    gbps = algo / (ms_step * 1e-3) / 1e9
    kernel_gbps = algo / (ms_kernel * 1e-3) / 1e9

    # ---- correctness of what was timed (layer 0 against the CPU oracle), CPU baseline -----
    check = None
    cpu_base = None
    if not args.no_check:
        check = check_layer0(first_pl, first_nvo, qs[:cfg.H_q].cpu().numpy(), out[:cfg.H_q].cpu().numpy(), torch)
    if not args.no_cpu_baseline:
        ora, ora_nvo = oracle_layer(first_pl, first_nvo, torch)
        cpu_base = cpu_baseline_section(ora, ora_nvo, qs[:cfg.H_q].cpu().numpy(), cfg.H_q, torch)
        del ora, ora_nvo

    main_run = default_workload and args.config == 1
    sequential = padded = None
    stream_bytes, n_work, n_wg = cache.stream_bytes, cache.n_work, cache.n_groups or cache.n_work
    if main_run:
        del cache, step
        torch.cuda.empty_cache()
        sequential = sequential_section(cfg, torch, dev, replays=args.steps)
        padded = padded_section(cfg, torch, dev, steps=args.steps)
        torch.cuda.empty_cache()
    configs = None
    if main_run and not args.no_configs:
        configs = {}
        for idx in (int(x) for x in args.configs.split(",") if x.strip()):
            try:
                configs[f"C{idx}"] = compact_config(idx, args, torch, dev)
            except Exception as e:  # the block is informative; a configuration that fails says so
                configs[f"C{idx}"] = {"error": repr(e)[:300]}
            torch.cuda.empty_cache()
    loop_info = None
    if main_run and not args.no_decode_loop:
        try:
            loop_info = decode_loop_section(cfg, torch, dev)
        except Exception as e:  # informative section; never fail the benchmark on it
            loop_info = {"error": repr(e)[:300]}

    traffic = MEASURED_TRAFFIC.get(args.config) if default_workload else None
    result = {
        "metric": "packed decode-attn achieved HBM GB/s (algorithmic bytes / step time)",
        "value": gbps, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u8/fp16 codes, fp32 accumulate", "data": "synthetic",
        "timing_mode": f"eager launches (streaming launch + merge launch per step); median of "
                       f"{step_extras['timing_rounds']} regions of `steps` steps each, alternating with the regions "
                       f"roofline.ms_per_launch comes from (the same steps with a HIP event before and after every "
                       f"streaming launch: mean in-step interval)",
        "ms_per_step_eager": ms_step_eager, "ms_per_step_graph_replay": ms_step_graph,
        "ms_per_step_graph_replay_8_steps_per_graph": step_extras.get("ms_per_step_graph_replay_8_steps_per_graph"),
        "ms_per_step_regions": step_extras["ms_per_step_regions"],
        "us_per_step_per_layer": ms_step * 1e3 / n_groups,
        "us_per_layer_sequential": sequential["us_per_layer_sequential"] if sequential else None,
        "pct_hbm_peak": 100.0 * gbps / HBM_PEAK_GBPS,
        "config": {"workload": cfg.name, "config_index": cfg.index, "layers": cfg.layers, "batch": cfg.batch,
                   "H_q": cfg.H_q, "H_kv": cfg.H_kv, "head_dim": cfg.D, "context": cfg.context,
                   "token_budget_metadata": cfg.token_budget,
                   "launch": "one fused launch + one merge launch per step over all layers",
                   "class_fractions_apply_to": "context tokens",
                   "algorithmic_bytes_per_step": algo, "algorithmic_bytes_per_layer": algo / n_groups,
                   "streamed_bytes_per_step": stream_bytes, "work_items": n_work, "workgroups": n_wg,
                   "dense_fp16_bytes_per_layer": synth.dense_fp16_bytes(cfg),
                   "compression_ratio": synth.dense_fp16_bytes(cfg) * n_groups / algo,
                   "build_seconds": t_build},
        "roofline": {"bound": "hbm", "achieved": kernel_gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": kernel_gbps / HBM_PEAK_GBPS,
                     "traffic": traffic[0] if traffic else None,
                     "traffic_source": (f"{traffic[1]}, a constant from that profiler run (not observed by this run)"
                                        if traffic else None),
                     "kernel": "decode_fused_kernel", "ms_per_launch": ms_kernel,
                     "ms_per_step_of_the_regions_with_inner_events": step_extras["ms_per_step_with_inner_events"],
                     "ms_per_launch_kernel_alone": step_extras["ms_per_launch_kernel_alone"],
                     "algorithmic_bytes_per_launch": algo, "streamed_bytes_per_launch": stream_bytes,
                     "ms_per_step_flushed_caches": ms_step_cold,
                     "step_GBps_flushed_caches": algo / (ms_step_cold * 1e-3) / 1e9,
                     "device_read_ceiling_GBps": probe_bytes / (ms_read * 1e-3) / 1e9,
                     "device_read_GBps_plain_loads": probe_bytes / (ms_read_plain * 1e-3) / 1e9,
                     "device_read_GBps_streaming_hint": probe_bytes / (ms_read_stream * 1e-3) / 1e9,
                     "device_copy_GBps_read_plus_write": 2 * probe_bytes / (ms_copy * 1e-3) / 1e9},
        "cpu_baseline": cpu_base,
        "dense_fp16": dict(dense, compression_ratio=dense_bytes / algo,
                           required_speedup=0.7 * dense_bytes / algo,
                           speedup_vs_ideal_dense=dense["ideal_ms_at_read_ceiling"] / ms_step,
                           speedup_vs_sdpa=(dense["sdpa_ms"] / ms_step) if dense.get("sdpa_ms") else None,
                           speedup_vs_dense_hip_kernel=(dense["dense_hip_kernel_ms"] / ms_step)
                           if dense.get("dense_hip_kernel_ms") else None,
                           speedup_vs_dense_hip_kernel_one_launch=(dense["dense_hip_kernel_one_launch_ms"] / ms_step)
                           if dense.get("dense_hip_kernel_one_launch_ms") else None),
        "sequential": sequential,
        "padded": padded,
        "configs": configs,
        "pack": pack_info,
        "select": select_info,
        "decode_loop": loop_info,
        "check": check,
    }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
