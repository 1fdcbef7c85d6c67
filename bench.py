#!/usr/bin/env python3
"""Benchmark of the GraphSAGE sampling hot path on one MI355X.

One "step" = one super-batch through the whole pipeline: for every fanout in
[15, 10, 5]: fused column slice + uniform sampling without replacement, then
per-batch unique (first-occurrence order) + relabel; the unique frontier of a
layer is the seed set of the next.  Inputs (CSC graph, seeds) are resident in
HBM before the timed region starts.

Prints ONE JSON line.  `value` is sampled edges per second over the timed
steps; `roofline` describes the kernel with the largest share of GPU time
(durations from HIP events recorded by the library on the launch stream while
the same steps run once more); `cpu_baseline` is the CPU oracle timed on a
bounded sample of the same workload on this machine's host cores.
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

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published peak

WORKLOADS = {
    # name: (nodes, edges, generator, batches, batch size, fanouts)
    "c2": dict(nodes=2_450_000, edges=124_000_000, gen="chung_lu", batches=64,
               batch_size=1024, fanouts=[15, 10, 5],
               desc="GraphSAGE 3-layer uniform [15,10,5], 64 batches x 1024 seeds per "
                    "launch, Chung-Lu power-law (exp 2.1) 2.45M nodes / 124M edges, CSC int64"),
    "c1": dict(nodes=100_000, edges=2_000_000, gen="rmat", batches=1,
               batch_size=1024, fanouts=[25, 10],
               desc="GraphSAGE 2-layer uniform [25,10], 1024 seeds, R-MAT 100K nodes / 2M edges"),
    "c3": dict(kind="ladies", nodes=233_000, edges=115_000_000, gen="chung_lu", seeds=512,
               fanouts=[512, 512],
               desc="LADIES 2 layers, 512 seeds, K=512 per layer, Chung-Lu power-law 233K nodes / "
                    "115M edges, fp32 edge weights U(0,1], through Matrix / gs.jit.compile"),
    "ops": dict(kind="ops", nodes=2_450_000, edges=124_000_000, gen="chung_lu", batches=64,
                batch_size=1024, fanouts=[15, 10, 5],
                desc="every operator of the path on its own: C2's graph, the frontiers and edge "
                     "lists of one GraphSAGE step as inputs, LogNormal weights"),
    "c4": dict(kind="node2vec", nodes=2_450_000, edges=124_000_000, gen="chung_lu",
               walks=1_000_000, length=80, p=2.0, q=0.5,
               desc="node2vec, 1M walks x 80 steps, p=2.0 q=0.5, C2's graph with sorted columns"),
    "c5s": dict(nodes=2_450_000, edges=124_000_000, gen="chung_lu", batches=64,
                batch_size=1024, fanouts=[15, 10, 5], weighted=True,
                desc="weighted GraphSAGE [15,10,5] (fp32 edge weights LogNormal(0,1), persistent CDF), 64 batches x "
                     "1024 seeds, on c2's graph: a 1/13-scale stand-in for the 1.6B-edge weighted "
                     "configuration"),
    "c5": dict(nodes=111_000_000, edges=1_600_000_000, gen="chung_lu", batches=128,
               batch_size=1024, fanouts=[15, 10, 5], weighted=True,
               desc="large-graph weighted GraphSAGE [15,10,5] (fp32 edge weights LogNormal(0,1), "
                    "persistent CDF), 128 batches x 1024 seeds, Chung-Lu power-law (exp 2.1) "
                    "111M nodes / 1.6B edges, CSC int64, all resident in HBM"),
    "gather": dict(kind="gather", nodes=2_450_000, edges=124_000_000, gen="chung_lu", batches=64,
                   batch_size=1024, fanouts=[15, 10, 5], feat=128,
                   desc="feature fetch for the input nodes of one c2 step: fp32 features "
                        "[2.45M, 128] gathered by the layer-3 frontier of 64 mini-batches"),
    "linerate": dict(kind="linerate", nodes=2_450_000, edges=124_000_000, gen="chung_lu",
                     batches=64, batch_size=1024, fanouts=[15, 10, 5],
                     desc="yardsticks on this GPU: streaming copy, scattered 128-byte lines "
                          "(one per lane), and the layer-3 launch of c2's uniform sampler with "
                          "parts switched off"),
    "tiny": dict(nodes=50_000, edges=1_000_000, gen="chung_lu", batches=8,
                 batch_size=256, fanouts=[15, 10, 5],
                 desc="1/50-scale twin of c2 (smoke runs)"),
}


def graphsage_step(be, indptr, indices, seeds, ptr, fanouts, seed, call_base, probs=None,
                   cdf=None, by_pointer=False):
    """The pipeline, written once for both back ends (`be` is gsampler_amd.capi
    on torch CUDA tensors or oracle.binding on numpy arrays).  With `probs`
    (fp32 per edge) neighbours are drawn by weight instead of uniformly, through
    the matrix's persistent CDF when `cdf` is given.  `by_pointer`: the relabel
    pass takes the column of an edge from the sampled matrix's column pointer; the
    sampler, told where the batches of its columns begin, writes every column's
    place inside its batch, which is the column's label while the seeds of a batch
    are distinct, so that the relabel pass only rewrites batches where they are not
    (same outputs).
    Returns per-layer (S, E, U) and the last layer's outputs."""
    sizes, last = [], None
    for layer, fanout in enumerate(fanouts):
        how = dict(col_batch_ptr=ptr) if by_pointer else {}
        if probs is None:
            sub_indptr, coo_col, rows, sel = be.sample_uniform(
                indptr, indices, seeds, fanout, False, 0, seed, call_base + layer, **how)
        else:
            sub_indptr, coo_col, rows, sel = be.sample_weighted(
                indptr, indices, probs, seeds, fanout, False, seed, call_base + layer,
                cdf=cdf, **how)
        # (a plain index_select on the device: advanced indexing costs the host three
        # times as long per call, and the first two layers are bound by the host)
        edge_ptr = sub_indptr.index_select(0, ptr) if hasattr(sub_indptr, "index_select") \
            else sub_indptr[ptr]
        if by_pointer:
            uniq, uniq_ptr, out_row, out_col = be.unique_relabel(
                seeds, rows, ptr, edge_ptr, col_indptr=sub_indptr, out_col=coo_col)
        else:
            uniq, uniq_ptr, out_row, out_col = be.unique_relabel(
                seeds, rows, ptr, edge_ptr, coo_col)
        sizes.append((int(seeds.shape[0]), int(rows.shape[0]), int(uniq.shape[0])))
        last = (uniq, uniq_ptr, out_row, out_col, sel)
        seeds, ptr = uniq, uniq_ptr
    return sizes, last


CALIBRATION_BYTES = 256 << 20


def kernel_bytes(name, sizes):
    """Algorithmic bytes moved by all launches of `name` in one step: the
    compulsory reads and writes of the kernel's interface (hash-table, scratch
    and re-read traffic excluded)."""
    total = 0
    for S, E, U in sizes:
        N = S + E
        total += {
            # the fill pass's interface: span and sub_indptr of every column, gather, and
            # row id, edge position and column of every edge (the column is stored as the
            # column's place inside its batch, which the relabel pass then leaves alone)
            "sample_uniform": 16 * S + 32 * E,
            "sample_weighted_cdf": 16 * S + 32 * E,  # the same interface as the uniform sampler
            "col_count": 40 * S,                 # seeds, indptr pair in; counts and spans out
            "unique_scatter": 16 * N,            # keys in, packed entries out
            "unique_dedup": 12 * N,              # packed entries in, first positions out
            "unique_flag": 4 * N + N // 4,       # first positions in, rank words out
            "unique_fill": N // 4 + 16 * U,      # rank words + first keys in, frontier out
            "unique_relabel": 12 * E,            # first position in, row label out
            # frontier and labels from one launch: the two lines above together
            "unique_fill_relabel": N // 4 + 16 * U + 12 * E,
        }.get(name, 0)
    return total


def batch_graphsage_sampler(A, seeds, seeds_ptr, fanouts):
    """The super-batched sampler of the reference's examples/graphsage/graphsage_e2e.py."""
    ret = []
    for k in fanouts:
        subA = A[:, seeds::seeds_ptr]
        sampleA = subA.individual_sampling(k, None, False)
        seeds, seeds_ptr = sampleA.all_nodes()
        ret.append(sampleA.to_dgl_block())
    return ret


def batch_weighted_graphsage_sampler(A, seeds, seeds_ptr, fanouts):
    ret = []
    for k in fanouts:
        subA = A[:, seeds::seeds_ptr]
        sampleA = subA.individual_sampling(k, subA.edata["w"], False)
        seeds, seeds_ptr = sampleA.all_nodes()
        ret.append(sampleA.to_dgl_block())
    return ret


def api_step_factory(indptr, indices, seeds, ptr, fanouts, probs):
    """step(i) -> (sizes, None) through BatchMatrix, gs.jit.compile and libgs.so."""
    import gsampler_amd as gs
    m = gs.Matrix()
    m.load_graph("CSC", [indptr, indices])
    func = batch_graphsage_sampler
    if probs is not None:
        m.edata["w"] = probs
        func = batch_weighted_graphsage_sampler
    bm = gs.BatchMatrix()
    bm.load_from_matrix(m, False)
    compiled = gs.jit.compile(func=func, args=(bm, seeds, ptr, fanouts), try_compact=False,
                              format_select=False)

    def step(i):
        layers = compiled(bm, seeds, ptr, fanouts)
        # every layer is a BlockList: its blocks are views of the layer's arrays
        sizes = []
        for blocks in layers:
            src, dst, edges = blocks.totals()
            sizes.append((dst, edges, src))
        return sizes, layers
    return step


def _kernel_table(capi, bytes_of):
    """Per-kernel totals of the library's event timers -> sorted list of dicts."""
    kernels = []
    for name, (calls, ms) in capi.profile_totals().items():
        nbytes = bytes_of(name)
        kernels.append(dict(kernel=name, launches=calls, avg_ms=round(ms / max(calls, 1), 4),
                            total_ms=round(ms, 4), algorithmic_bytes=nbytes,
                            gbs=round(nbytes / (ms * 1e-3) / 1e9, 1) if ms > 0 else 0.0))
    kernels.sort(key=lambda k: -k["total_ms"])
    return kernels


def _roofline(dom):
    return dict(bound="hbm", kernel=dom["kernel"], achieved=dom["gbs"], peak=HBM_PEAK_GBS,
                unit="GB/s", frac=round(dom["gbs"] / HBM_PEAK_GBS, 4), traffic=None,
                avg_launch_ms=dom["avg_ms"], launches=dom["launches"])


def run_node2vec(args, wl, capi, dev):
    """Second-order walks over C2's graph.  A step = one launch of all walks."""
    import torch
    from gsampler_amd.utils import chung_lu_csc
    t0 = time.time()
    indptr, indices = chung_lu_csc(wl["nodes"], wl["edges"], seed=1, device=dev)
    indices = capi.segment_sort(indptr, indices, wl["nodes"])   # node2vec needs sorted columns
    g = torch.Generator(device=dev)
    g.manual_seed(3)
    seeds = torch.randint(0, wl["nodes"], (wl["walks"],), generator=g, device=dev)
    torch.cuda.synchronize()
    t_build = time.time() - t0
    L = wl["length"]

    def step(i):
        return capi.node2vec(indptr, indices, seeds, L, wl["p"], wl["q"], args.seed, i)

    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        trace = step(args.warmup + i)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    hops = int((trace[1:] >= 0).sum().item())             # hops taken in the last step
    capi.profile_reset()
    capi.profile_enable(True)
    for i in range(args.steps):
        step(args.warmup + i)
    torch.cuda.synchronize()
    # per hop: indptr pair 16 B + one candidate row id 8 B + trace write 8 B (retries of the
    # rejection loop and the connectivity searches come on top and are not counted)
    kernels = _kernel_table(capi, lambda name: 32 * hops * args.steps if name == "node2vec" else 0)
    capi.profile_enable(False)
    cpu = None
    if args.cpu_seconds > 0:
        from oracle import binding as orc
        h_indptr, h_indices = indptr.cpu().numpy(), indices.cpu().numpy()
        n = 20_000
        h_seeds = seeds[:n].cpu().numpy()
        orc.node2vec(h_indptr, h_indices, h_seeds[:1000], L, wl["p"], wl["q"], args.seed, 0)
        t_cpu, h_cpu, runs = 0.0, 0, 0
        while t_cpu < args.cpu_seconds and runs < 1000:
            t = time.perf_counter()
            tr = orc.node2vec(h_indptr, h_indices, h_seeds, L, wl["p"], wl["q"], args.seed, runs)
            t_cpu += time.perf_counter() - t
            h_cpu += int((tr[1:] >= 0).sum())
            runs += 1
        cpu = dict(value=round(h_cpu / t_cpu, 1), unit="hops/s", cores=orc.num_threads(),
                   kind="port", sample=f"{runs} runs of the first {n} walks ({L} steps each) in "
                                       f"{t_cpu:.1f} s, OpenMP oracle", host_cpus=os.cpu_count())
    value = hops * args.steps / elapsed
    return {
        "metric": "walk_hops_per_sec", "value": round(value, 1), "unit": "hops/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(elapsed / args.steps * 1e3, 3), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "int64", "data": "synthetic",
        "config": {"workload": f"{args.workload}: {wl['desc']}", "walks": wl["walks"],
                   "walk_length": L, "p": wl["p"], "q": wl["q"], "hops_per_step": hops},
        "roofline": _roofline(kernels[0]), "cpu_baseline": cpu,
        "gpu_over_cpu": round(value / cpu["value"], 1) if cpu else None,
        "kernels": kernels, "graph_build_s": round(t_build, 1),
    }


def run_gather(args, wl, capi, dev):
    """The fetch that follows sampling in a training loop: features[input_nodes]
    for the frontier of the last layer of one c2 step.  A step = one gather."""
    import numpy as np
    import torch
    from gsampler_amd.utils import batched_seeds, chung_lu_csc
    t0 = time.time()
    indptr, indices = chung_lu_csc(wl["nodes"], wl["edges"], seed=1, device=dev)
    seeds, ptr = batched_seeds(wl["nodes"], wl["batches"], wl["batch_size"], seed=2, device=dev)
    _, last = graphsage_step(capi, indptr, indices, seeds, ptr, wl["fanouts"], args.seed, 0)
    ids = last[0].clone()
    del indptr, indices, last
    F = wl["feat"]
    g = torch.Generator(device=dev)
    g.manual_seed(11)
    table = torch.rand((wl["nodes"], F), generator=g, device=dev)
    torch.cuda.synchronize()
    t_build = time.time() - t0
    n = ids.numel()
    step_bytes = 8 * n + 2 * n * F * 4       # ids + every row read once and written once

    for _ in range(args.warmup):
        capi.gather_rows(table, ids)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        out = capi.gather_rows(table, ids)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    check = bool(torch.equal(out[::997], table[ids[::997]]))
    del out
    capi.profile_reset()
    capi.profile_enable(True)
    for _ in range(args.steps):
        capi.gather_rows(table, ids)
    torch.cuda.synchronize()
    kernels = _kernel_table(capi, lambda name: step_bytes * args.steps if name == "gather_rows" else 0)
    capi.profile_enable(False)
    # torch's own indexing on the same inputs, for scale
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        ref = table[ids]
    torch.cuda.synchronize()
    torch_ms = (time.perf_counter() - t0) / args.steps * 1e3
    del ref
    cpu = None
    if args.cpu_seconds > 0:
        from oracle import binding as orc
        m = min(n, 2_000_000)
        h_table, h_ids = table.cpu().numpy(), ids[:m].cpu().numpy()
        orc.gather_rows(h_table, h_ids[:1000])
        t_cpu, rows, runs = 0.0, 0, 0
        while t_cpu < args.cpu_seconds and runs < 1000:
            t = time.perf_counter()
            orc.gather_rows(h_table, h_ids)
            t_cpu += time.perf_counter() - t
            rows += m
            runs += 1
        cpu = dict(value=round(rows / t_cpu, 1), unit="rows/s", cores=orc.num_threads(),
                   kind="port", sample=f"{runs} gathers of the first {m} ids in {t_cpu:.1f} s, "
                                       f"OpenMP oracle", host_cpus=os.cpu_count())
    value = n * args.steps / elapsed
    return {
        "metric": "gathered_rows_per_sec", "value": round(value, 1), "unit": "rows/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(elapsed / args.steps * 1e3, 3), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"{args.workload}: {wl['desc']}", "rows_per_step": n,
                   "row_bytes": F * 4, "spot_check_against_torch_indexing": check,
                   "torch_indexing_ms": round(torch_ms, 3)},
        "roofline": _roofline(kernels[0]), "cpu_baseline": cpu,
        "gpu_over_cpu": round(value / cpu["value"], 1) if cpu else None,
        "kernels": kernels, "graph_build_s": round(t_build, 1),
    }


def _event_ms(fn, repeats):
    """Average milliseconds of fn() over `repeats` calls, by events on the current stream."""
    import torch
    fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(repeats):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / repeats


def run_linerate(args, wl, capi, dev):
    """What this GPU delivers to the two access patterns the path consists of, measured with
    the library's own kernels, and the sampler's largest launch of a c2 step taken apart.
      stream copy:  1 GiB read + 1 GiB written, 16 bytes per lane;
      line gather:  2^26 lanes each read 4 bytes of a 128-byte line of their own, chosen by a
                    hash, in a 4 GiB table (sixteen times the last-level cache) and in a 64 MiB
                    table (inside it); the same number of lines in address order for scale;
      sampler:      the layer-3 launch (3.5 M columns, fan-out 5, int32 row ids) as shipped and
                    with parts switched off (gs_probe_sample_uniform)."""
    import torch
    from gsampler_amd.utils import batched_seeds, chung_lu_csc
    reps = max(3, min(args.steps, 20))
    gib = 1 << 30
    src = torch.empty(gib // 8, dtype=torch.int64, device=dev).random_()
    dst = torch.empty_like(src)
    copy_ms = _event_ms(lambda: capi.probe_stream_copy(src, dst), reps)
    assert torch.equal(src[::4097], dst[::4097])
    del src, dst
    # 4 GiB of lines for 2^26 picks: a line is asked for twice on average, a long way apart
    table_bytes = 4 * gib
    src = torch.empty(table_bytes // 8, dtype=torch.int64, device=dev).random_()
    picks = 1 << 26
    out = torch.empty(picks // 4 + 1, dtype=torch.int32, device=dev)
    salt = [0]

    def gather(table, ordered):
        salt[0] += 1
        capi.probe_line_gather(table, picks, salt[0], ordered, out)

    big_ms = _event_ms(lambda: gather(src, False), reps)
    ordered_ms = _event_ms(lambda: gather(src, True), reps)
    small = src[: (64 << 20) // 8]
    small_ms = _event_ms(lambda: gather(small, False), reps)
    del small
    lines_per_s = picks / (big_ms * 1e-3)
    yard = {
        "stream_copy_gbs": round(2 * gib / (copy_ms * 1e-3) / 1e9, 1),
        "stream_copy_frac_of_hbm_peak": round(2 * gib / (copy_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
        "scattered_lines_per_s": round(lines_per_s, 1),
        "scattered_lines_gbs_at_128B": round(lines_per_s * 128 / 1e9, 1),
        "scattered_lines_frac_of_hbm_peak": round(lines_per_s * 128 / 1e9 / HBM_PEAK_GBS, 4),
        "lines_in_address_order_per_s": round(picks / (ordered_ms * 1e-3), 1),
        "scattered_lines_in_a_64MiB_table_per_s": round(picks / (small_ms * 1e-3), 1),
        "picks": picks, "table_bytes": table_bytes,
    }
    del src, out
    # ---- the sampler's layer-3 launch of a c2 step
    indptr, indices = chung_lu_csc(wl["nodes"], wl["edges"], seed=1, device=dev)
    seeds, ptr = batched_seeds(wl["nodes"], wl["batches"], wl["batch_size"], seed=2, device=dev)
    idx32 = indices.to(torch.int32)
    f, fp = seeds, ptr
    for layer, k in enumerate(wl["fanouts"][:-1]):
        s_ = capi.sample_uniform(indptr, idx32, f, k, False, 0, args.seed, layer, with_coo=False)
        r_ = capi.unique_relabel(f, s_[2], fp, s_[0][fp], col_indptr=s_[0])
        f, fp = r_[0], r_[1]
    K = wl["fanouts"][-1]
    S = int(f.numel())
    col_span = torch.empty(S, dtype=torch.int64, device=dev)
    sub_indptr = capi.col_count(indptr, f, K, False, col_span=col_span)
    E = int(sub_indptr[-1].item())
    bound = S * K
    outs = (torch.empty(bound, dtype=torch.int64, device=dev),
            torch.empty(bound, dtype=torch.int64, device=dev),
            torch.empty(bound, dtype=torch.int64, device=dev))
    avg_deg = int(indices.numel() // wl["nodes"])
    variants = [
        ("as shipped: column spans from the count pass; row id, edge position and column of "
         "every edge stored (the benched path also looks up the batch of the column)", 0, True),
        ("column pointer looked up again instead (no spans)", -1, True),
        ("row id and edge position stored", 0, False),
        ("a multiplicative hash in place of Philox", 1, False),
        ("no exchange among a column's lanes", 2, False),
        ("column pointer not read (every column %d long)" % avg_deg, 4, False),
        ("row ids not read, two stores", 8, False),
        ("row ids not read, one store", 24, False),
        ("row ids read, one store", 16, False),
        ("row ids read, nothing stored", 32, False),
        ("row ids not read, nothing stored", 40, False),
    ]
    table = []
    for name, variant, with_col in variants:
        o = (outs[0] if with_col else None, outs[1], outs[2])
        spans = col_span if variant >= 0 else None
        ms = _event_ms(lambda: capi.probe_sample_uniform(indptr, idx32, f, K, max(variant, 0),
                                                         sub_indptr, o, probe_degree=avg_deg,
                                                         seed=args.seed, call_id=2,
                                                         col_span=spans), reps)
        table.append({"variant": name, "bits": max(variant, 0), "spans": spans is not None,
                      "us": round(ms * 1e3, 1)})
    benched = table[0]["us"] * 1e-6
    # Lines the launch visits: the distinct lines of int32 row ids under its picks, counted
    # from the picks themselves (without spans also one line of the column pointer per column,
    # two when the pair straddles a line: column_pointer_lines); the 8-byte span, offset and
    # output streams come on top as bytes.
    capi.probe_sample_uniform(indptr, idx32, f, K, 0, sub_indptr, (outs[0], outs[1], outs[2]),
                              seed=args.seed, call_id=2, col_span=col_span)
    col, sel = outs[0][:E], outs[2][:E]
    row_lines = int(torch.unique(col * (1 << 32) + sel // 32).numel())
    ptr_lines = S + int(((f % 16) == 15).sum().item())
    lines = row_lines
    stream_bytes = 16 * S + 24 * E   # spans and offsets in; row id, edge position, column out
    floor_us = lines / lines_per_s * 1e6 + stream_bytes / (2 * gib / (copy_ms * 1e-3)) * 1e6
    sampler = {
        "columns": S, "picks": E, "fanout": K, "variants": table,
        "moved_bytes": 16 * S + 32 * E,
        "moved_gbs": round((16 * S + 32 * E) / benched / 1e9, 1),
        "frac_of_hbm_peak_by_bytes_moved": round((16 * S + 32 * E) / benched / 1e9 / HBM_PEAK_GBS, 4),
        "lines_visited": lines, "row_id_lines": row_lines,
        "column_pointer_lines_without_spans": ptr_lines,
        "streamed_bytes": stream_bytes,
        "time_of_those_lines_and_streams_at_the_measured_rates_us": round(floor_us, 1),
        "frac_of_measured_rates": round(floor_us * 1e-6 / benched, 4),
    }
    return {
        "metric": "scattered_128B_lines_per_sec", "value": round(lines_per_s, 1), "unit": "lines/s",
        "n_gpus": 1, "steps": reps, "warmup": 1, "ms_per_step": round(big_ms, 3),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "u32",
        "data": "synthetic", "config": {"workload": f"{args.workload}: {wl['desc']}"},
        "roofline": dict(bound="hbm", kernel="probe_line_gather",
                         achieved=yard["scattered_lines_gbs_at_128B"], peak=HBM_PEAK_GBS,
                         unit="GB/s", frac=yard["scattered_lines_frac_of_hbm_peak"], traffic=None,
                         avg_launch_ms=round(big_ms, 4), launches=reps),
        "cpu_baseline": None, "yardsticks": yard, "sampler_layer3": sampler,
    }


def ladies_sampler(A, seeds, fanouts):
    """The layer-wise sampler of the reference's examples/ladies/ladies.py:7-21."""
    ret = []
    for K in fanouts:
        subA = A[:, seeds]
        subA.edata["p"] = subA.edata["w"] ** 2
        prob = subA.sum("p", axis=1)
        sampleA, select_index = subA.collective_sampling(K, prob, False)
        sampleA = sampleA.div("w", prob[select_index], axis=1)
        out = sampleA.sum("w", axis=0)
        sampleA = sampleA.div("w", out, axis=0)
        seeds = sampleA.all_nodes()
        ret.append(sampleA.to_dgl_block(prefetch_edata={"w"}))
    return seeds, ret


def ladies_layer_sizes(A, seeds, fanouts):
    """(columns sliced, edges of the column slice, edges kept by the row slice) per layer of
    one eager run of ladies_sampler: what the byte counts of a step are taken from."""
    sizes = []
    for K in fanouts:
        subA = A[:, seeds]
        subA.edata["p"] = subA.edata["w"] ** 2
        prob = subA.sum("p", axis=1)
        sampleA, _ = subA.collective_sampling(K, prob, False)
        sizes.append((int(seeds.numel()), int(subA.num_edges()), int(sampleA.num_edges())))
        seeds = sampleA.all_nodes()
    return sizes


def ladies_kernel_bytes(name, sizes, num_rows):
    """Algorithmic bytes of all launches of `name` in one LADIES step (interface reads
    and writes; tables, scratch and re-reads excluded)."""
    total = 0
    for S, nnz, kept in sizes:
        total += {
            "col_slice_fill": 24 * S + 32 * nnz,          # seeds, indptr pair, row id in; 3 outputs
            "gather_rows": 16 * nnz + 16 * kept,          # edge data of both slices: index + value in, value out
            "member_flag": 8 * nnz,                       # row id of every edge
            "member_fill": 4 * kept + 24 * kept,          # staged ids in; row, column, position out
            "rowsum_hist": 8 * nnz, "rowsum_scatter": 12 * nnz + 8 * nnz,
            "rowsum_accumulate": 8 * nnz + 4 * num_rows,
            "spmm_coo_sum": 12 * nnz + 4 * num_rows,
            "spmm_csc_sum": 4 * kept + 4 * S,
            "sddmm": 2 * 20 * kept,                       # two quotients: value, id and operand in, value out
            "first_position": 8 * kept,
        }.get(name, 0)
    return total


def ladies_step_oracle(orc, indptr, indices, w, seeds, fanouts, num_rows, call_base):
    """The same two LADIES layers on the CPU: the oracle's operators chained by hand
    (column slice, e^2 row sums, weighted collective pick, row slice, the two
    normalisations, relabel).  Returns the number of block edges."""
    import numpy as np
    edges = 0
    for layer, K in enumerate(fanouts):
        sub_indptr, coo_col, rows, sel = orc.col_slice(indptr, indices, seeds)
        w_sub = w[sel]
        prob = orc.e_square_sum(("coo", rows, coo_col), w_sub, 2, num_rows)
        selected, _ = orc.list_sample_weighted(prob, K, call_id=call_base + layer)
        out_indptr, major, minor, select = orc.minor_slice(rows, selected, indptr=sub_indptr)
        w2 = orc.sddmm(("csc", out_indptr, minor), "div", w_sub[select], prob[selected], 1, 0)
        col_sum = orc.spmm(("csc", out_indptr, minor), "copy_rhs", "sum", None, w2, 0,
                           seeds.size)
        w3 = orc.sddmm(("csc", out_indptr, minor), "div", w2, col_sum, 1, 2)
        uniq, _, _, _ = orc.unique_relabel(seeds, selected[minor], edge_col=major)
        edges += int(minor.size)
        seeds = uniq
        del w3
    return edges


def run_ops(args, wl, capi, dev):
    """Every operator of the path timed on its own.  Device time = the sum of
    the operator's kernels by the library's event timers (a count pass and a
    fill pass belong to one operator); bytes = the operator's compulsory
    reads and writes.  Inputs: C2's graph and what one GraphSAGE step makes of
    it (layer-2 frontier: ~0.6 M columns; layer-3 frontier: ~3.5 M columns and
    17 M sampled edges)."""
    import torch
    from gsampler_amd.utils import batched_seeds, chung_lu_csc
    t0 = time.time()
    indptr, indices = chung_lu_csc(wl["nodes"], wl["edges"], seed=1, device=dev)
    N, nnz = wl["nodes"], int(indices.numel())
    seeds, ptr = batched_seeds(N, wl["batches"], wl["batch_size"], seed=2, device=dev)
    g = torch.Generator(device=dev)
    g.manual_seed(5)
    probs = torch.randn(nnz, generator=g, device=dev).exp_().float()
    cdf = capi.weight_cdf(indptr, probs, indices, N)
    # frontiers of a step
    s1 = capi.sample_uniform(indptr, indices, seeds, 15, False, 0, args.seed, 0)
    r1 = capi.unique_relabel(seeds, s1[2], ptr, s1[0][ptr], s1[1])
    s2 = capi.sample_uniform(indptr, indices, r1[0], 10, False, 0, args.seed, 1)
    r2 = capi.unique_relabel(r1[0], s2[2], r1[1], s2[0][r1[1]], s2[1])
    f2, f3, f3_ptr = r1[0][:131072].contiguous(), r2[0], r2[1]   # f2: the first two mini-batches' worth
    s3 = capi.sample_uniform(indptr, indices, f3, 5, False, 0, args.seed, 2)
    e3_ptr = s3[0][f3_ptr]
    S2, S3, E3 = int(f2.numel()), int(f3.numel()), int(s3[2].numel())
    torch.cuda.synchronize()
    t_build = time.time() - t0
    rows = []

    def measure(name, ref, fn, nbytes, note):
        out = fn()                       # warm-up; the result sizes the byte count if needed
        if callable(nbytes):
            nbytes = nbytes(out)
        del out
        torch.cuda.synchronize()
        capi.profile_reset()
        capi.profile_enable(True)
        t = time.perf_counter()
        for _ in range(args.steps):
            fn()
        torch.cuda.synchronize()
        wall = (time.perf_counter() - t) / args.steps * 1e3
        capi.profile_enable(False)
        dev_ms = sum(ms for _, ms in capi.profile_totals().values()) / args.steps
        gbs = nbytes / (dev_ms * 1e-3) / 1e9 if dev_ms > 0 else 0.0
        rows.append(dict(operator=name, reference=ref, device_ms=round(dev_ms, 4),
                         wall_ms=round(wall, 4), algorithmic_mb=round(nbytes / 1e6, 1),
                         gbs=round(gbs, 1), frac_of_hbm_peak=round(gbs / HBM_PEAK_GBS, 4),
                         input=note))

    # column slice of the layer-2 frontier
    measure("column slice", "OnIndptrSlicingCUDA", lambda: capi.col_slice(indptr, indices, f2),
            lambda o: 24 * S2 + 32 * int(o[2].numel()), f"{S2} columns")
    sl = capi.col_slice(indptr, indices, f2)
    sl_nnz = int(sl[2].numel())
    # row slice of that slice by 512 picked rows per ... here: 65 536 picked ids
    picked = torch.randperm(N, generator=g, device=dev)[:65536]
    measure("row slice", "OnIndicesSlicingCUDA", lambda: capi.minor_slice(sl[2], picked, indptr=sl[0]),
            lambda o: 8 * 65536 + 8 * sl_nnz + 32 * int(o[2].numel()),
            f"{sl_nnz} edges against 65536 picked rows")
    e_w = probs[sl[3]]
    coo_view = ("coo", sl[2], sl[1])
    csc_view = ("csc", sl[0], sl[2])
    measure("e^2 row sums (edge list)", "ESquareSumCOO",
            lambda: capi.e_square_sum(coo_view, e_w, 2, N), 12 * sl_nnz + 4 * N, f"{sl_nnz} edges onto {N} rows")
    measure("column sums (compressed)", "SpMMCSC",
            lambda: capi.spmm(csc_view, "copy_rhs", "sum", None, e_w, 0, S2), 4 * sl_nnz + 12 * S2,
            f"{sl_nnz} edges onto {S2} columns")
    col_sum = capi.spmm(csc_view, "copy_rhs", "sum", None, e_w, 0, S2)
    measure("edge / column value (edge list)", "SDDMMCOO",
            lambda: capi.sddmm(coo_view, "div", e_w, col_sum, 1, 2),
            24 * sl_nnz, f"{sl_nnz} edges")
    measure("edge / column value (compressed)", "SDDMMCSC",
            lambda: capi.sddmm(csc_view, "div", e_w, col_sum, 1, 2), 16 * sl_nnz + 16 * S2,
            f"{sl_nnz} edges")
    measure("edges' columns from offsets", "CSC2COOCUDA", lambda: capi.csc2coo(sl[0], sl_nnz),
            8 * S2 + 8 * sl_nnz, f"{sl_nnz} edges")
    del sl, e_w, col_sum, coo_view, csc_view
    # samplers on the layer-3 frontier
    idx32 = indices.to(torch.int32)      # the copy a loaded matrix keeps for this sampler
    measure("uniform slice + sample, K=5", "FusedCSCColSlicingSamplingCUDA",
            lambda: capi.sample_uniform(indptr, idx32, f3, 5, False, 0, args.seed, 2),
            32 * S3 + 32 * E3, f"{S3} columns")
    measure("weighted slice + sample, K=5 (CDF)", "CSCColSamplingProbsCUDA",
            lambda: capi.sample_weighted(indptr, indices, probs, f3, 5, False, args.seed, 2, cdf=cdf),
            32 * S3 + 32 * E3, f"{S3} columns")
    measure("unique + relabel, 64 batches", "BatchCOORelabelCUDA",
            lambda: capi.unique_relabel(f3, s3[2], f3_ptr, e3_ptr, s3[1]),
            lambda o: 8 * S3 + 24 * E3 + 8 * int(o[0].numel()), f"{S3} + {E3} keys")
    node_w = torch.rand(N, generator=g, device=dev)
    measure("collective pick of 512", "ListSamplingProbsCUDA",
            lambda: capi.list_sample_weighted(node_w, 512, False, None, args.seed, 3), 4 * N + 8 * 512,
            f"{N} weights")
    walkers = torch.randint(0, N, (1_000_000,), generator=g, device=dev)
    measure("random walk, 80 steps", "FusedRandomWalkCUDA",
            lambda: capi.random_walk(indptr, indices, walkers, 80, args.seed, 4),
            lambda o: 32 * int((o[1:] >= 0).sum()), "1 M walks")
    measure("per-column sort", "SortIndicesCUDA", lambda: capi.segment_sort(indptr, indices, N), 16 * nnz,
            f"{nnz} edges in {N} columns")
    coo_col = capi.csc2coo(indptr, nnz)
    measure("edge list -> compressed", "COO2CSCCUDA", lambda: capi.coo_to_csc(indices, coo_col, N),
            8 * nnz * 2 + 8 * nnz * 2 + 8 * N, f"{nnz} edges")
    measure("weight CDF build", "(none)", lambda: capi.weight_cdf(indptr, probs, indices, N),
            12 * nnz + 8 * nnz, f"{nnz} edges")
    rows.sort(key=lambda r: -r["device_ms"])
    dom = rows[0]
    return {
        "metric": "operators_measured", "value": len(rows), "unit": "operators", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(sum(r["device_ms"] for r in rows), 3), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "int64", "data": "synthetic",
        "config": {"workload": f"{args.workload}: {wl['desc']}"},
        "roofline": dict(bound="hbm", kernel=dom["operator"], achieved=dom["gbs"],
                         peak=HBM_PEAK_GBS, unit="GB/s", frac=dom["frac_of_hbm_peak"],
                         traffic=None, avg_launch_ms=dom["device_ms"], launches=args.steps),
        "cpu_baseline": None, "operators": rows, "graph_build_s": round(t_build, 1),
    }


def run_ladies(args, wl, capi, dev):
    """LADIES through the Python Matrix API and the torch custom class (the
    whole drop-in stack), compiled with gs.jit.compile.  A step = one 2-layer sample."""
    import torch
    import gsampler_amd as gs
    from gsampler_amd.utils import chung_lu_csc
    t0 = time.time()
    indptr, indices = chung_lu_csc(wl["nodes"], wl["edges"], seed=1, device=dev)
    g = torch.Generator(device=dev)
    g.manual_seed(4)
    w = 1.0 - torch.rand(indices.numel(), generator=g, device=dev, dtype=torch.float32)
    A = gs.Matrix()
    A.load_graph("CSC", [indptr, indices])
    A.edata["w"] = w
    seeds = torch.randperm(wl["nodes"], generator=g, device=dev)[:wl["seeds"]]
    fanouts = wl["fanouts"]
    compiled = gs.jit.compile(ladies_sampler, (A, seeds, fanouts))
    torch.cuda.synchronize()
    t_build = time.time() - t0

    def step():
        _, blocks = compiled(A, seeds, fanouts)
        return blocks

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    edges = 0
    for _ in range(args.steps):
        blocks = step()
        edges += sum(int(b.num_edges()) for b in blocks)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    capi.profile_reset()
    capi.profile_enable(True)
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    totals_seen = capi.profile_totals()
    capi.profile_enable(False)
    layer_sizes = ladies_layer_sizes(A, seeds, fanouts)
    kernels = []
    for name, (calls, ms) in totals_seen.items():
        nbytes = ladies_kernel_bytes(name, layer_sizes, A.num_rows()) * args.steps
        kernels.append(dict(kernel=name, launches=calls, avg_ms=round(ms / max(calls, 1), 4),
                            total_ms=round(ms, 4), algorithmic_bytes=nbytes,
                            gbs=round(nbytes / (ms * 1e-3) / 1e9, 1) if ms > 0 else 0.0))
    kernels.sort(key=lambda k: -k["total_ms"])
    sliced = [int(b.num_edges()) for b in blocks]
    cpu = None
    if args.cpu_seconds > 0:
        from oracle import binding as orc
        h = [t.cpu().numpy() for t in (indptr, indices, w, seeds)]
        ladies_step_oracle(orc, *h, fanouts, A.num_rows(), 0)          # warm-up
        t_cpu, e_cpu, runs = 0.0, 0, 0
        while t_cpu < args.cpu_seconds and runs < 1000:
            t = time.perf_counter()
            e_cpu += ladies_step_oracle(orc, *h, fanouts, A.num_rows(), 2 * (runs + 1))
            t_cpu += time.perf_counter() - t
            runs += 1
        cpu = dict(value=round(e_cpu / t_cpu, 1), unit="edges/s", cores=orc.num_threads(),
                   kind="port", sample=f"{runs} two-layer samples on the same graph and seeds in "
                                       f"{t_cpu:.1f} s, OpenMP oracle operators chained by hand",
                   host_cpus=os.cpu_count())
    value = edges / elapsed
    return {
        "metric": "sampled_edges_per_sec", "value": round(value, 1), "unit": "edges/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(elapsed / args.steps * 1e3, 3), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"{args.workload}: {wl['desc']}", "fanouts": fanouts,
                   "seeds": wl["seeds"], "block_edges_last_step": sliced,
                   "layer_sizes_cols_sliced_kept": layer_sizes},
        "roofline": _roofline(kernels[0]), "cpu_baseline": cpu,
        "gpu_over_cpu": round(value / cpu["value"], 1) if cpu else None,
        "kernels": kernels, "graph_build_s": round(t_build, 1),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c2", choices=sorted(WORKLOADS))
    ap.add_argument("--cpu-seconds", type=float, default=15.0,
                    help="target CPU time of the oracle baseline (0 = skip)")
    ap.add_argument("--seed", type=int, default=7777)
    ap.add_argument("--no-api", action="store_true",
                    help="skip the second timing of the same workload through the Python API")
    ap.add_argument("--path", default="abi", choices=["abi", "api"],
                    help="abi: the C ABI through ctypes (default); api: the same GraphSAGE "
                         "workload through BatchMatrix + gs.jit.compile and the torch "
                         "custom class, per-batch blocks included")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build drives exactly one GPU (the super-batch is the unit "
                 "that would be dealt out across GPUs); run with --gpus 1")

    import numpy as np
    import torch
    from gsampler_amd import capi
    from gsampler_amd.utils import batched_seeds, chung_lu_csc, rmat_csc

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    capi.lib()  # fail loudly when the kernel library is missing
    dev = torch.device("cuda:0")
    wl = WORKLOADS[args.workload]
    if wl.get("kind") == "node2vec":
        return print(json.dumps(run_node2vec(args, wl, capi, dev)))
    if wl.get("kind") == "gather":
        return print(json.dumps(run_gather(args, wl, capi, dev)))
    if wl.get("kind") == "ladies":
        return print(json.dumps(run_ladies(args, wl, capi, dev)))
    if wl.get("kind") == "ops":
        return print(json.dumps(run_ops(args, wl, capi, dev)))
    if wl.get("kind") == "linerate":
        return print(json.dumps(run_linerate(args, wl, capi, dev)))

    t0 = time.time()
    gen = chung_lu_csc if wl["gen"] == "chung_lu" else rmat_csc
    indptr, indices = gen(wl["nodes"], wl["edges"], seed=1, device=dev)
    seeds, ptr = batched_seeds(wl["nodes"], wl["batches"], wl["batch_size"], seed=2, device=dev)
    torch.cuda.synchronize()
    t_build = time.time() - t0
    fanouts = wl["fanouts"]
    probs = cdf = None
    t_cdf = 0.0
    if wl.get("weighted"):
        g = torch.Generator(device=dev)
        g.manual_seed(5)
        probs = torch.randn(indices.numel(), generator=g, device=dev).exp_().float()
        torch.cuda.synchronize()
        t0 = time.time()
        cdf = capi.weight_cdf(indptr, probs, indices, wl["nodes"])   # once per (graph, weights)
        torch.cuda.synchronize()
        t_cdf = time.time() - t0

    # One plain streaming kernel of known size (reads 256 MiB, writes 256 MiB):
    # the yardstick that hardware traffic counters of a profiled run are scaled by.
    yard = torch.zeros(CALIBRATION_BYTES // 8, dtype=torch.int64, device=dev)
    yard = torch.bitwise_xor(yard, 1)
    del yard

    # the int32 copy of the row ids that a loaded matrix keeps for the uniform sampler
    # (the operator class makes the same copy on its first sampling call)
    pick_ids = indices
    if probs is None and wl["nodes"] < 2 ** 31 and indices.numel() >= 1 << 20:
        pick_ids = indices.to(torch.int32)

    def step(i):
        return graphsage_step(capi, indptr, pick_ids, seeds, ptr, fanouts, args.seed,
                              i * len(fanouts), probs, cdf, by_pointer=True)

    if args.path == "api":
        step = api_step_factory(indptr, indices, seeds, ptr, fanouts, probs)

    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    edges = 0
    sizes = None
    for i in range(args.steps):
        sizes, _ = step(args.warmup + i)
        edges += sum(E for _, E, _ in sizes)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3
    edges_per_s = edges / elapsed
    batches_per_s = wl["batches"] * args.steps / elapsed

    # ---- per-kernel durations: same steps again with the library's event timers on
    capi.profile_reset()
    capi.profile_enable(True)
    prof_sizes = []
    for i in range(args.steps):
        s, _ = step(args.warmup + i)
        prof_sizes.append(s)
    torch.cuda.synchronize()
    totals = capi.profile_totals()
    capi.profile_enable(False)
    kernels = []
    for name, (calls, ms) in totals.items():
        nbytes = sum(kernel_bytes(name, s) for s in prof_sizes)
        kernels.append(dict(kernel=name, launches=calls, avg_ms=ms / max(calls, 1),
                            total_ms=ms, algorithmic_bytes=nbytes,
                            gbs=(nbytes / (ms * 1e-3) / 1e9) if ms > 0 else 0.0))
    kernels.sort(key=lambda k: -k["total_ms"])
    dom = kernels[0]
    # Bytes that the L2s exchanged with the memory fabric per launch (rocprofv3 FETCH_SIZE +
    # WRITE_SIZE; reads served by the Infinity Cache are included, the counters cannot tell
    # them from HBM accesses).  Not measured in this run: transcribed from the committed
    # counter summary of this same command, which names the commit it was taken at.
    traffic, traffic_source = None, None
    tname = f"graphsage_{args.workload}_hbm_traffic.txt"
    tpath = os.path.join(ROOT, "profiles", tname)
    if os.path.exists(tpath):
        commit = None
        for line in open(tpath):
            f = line.split()
            if line.startswith("# commit:") and len(f) >= 3:
                commit = f[2]
            if len(f) == 5 and f[0] == dom["kernel"]:
                traffic = int(f[4])
        traffic_source = {"file": f"profiles/{tname}", "commit": commit,
                          "kind": "transcribed, not measured in this run"}
    roofline = dict(bound="hbm", kernel=dom["kernel"], achieved=round(dom["gbs"], 1),
                    peak=HBM_PEAK_GBS, unit="GB/s", frac=round(dom["gbs"] / HBM_PEAK_GBS, 4),
                    traffic=traffic, avg_launch_ms=round(dom["avg_ms"], 4),
                    launches=dom["launches"])
    if dom["kernel"] in ("sample_uniform", "sample_weighted_cdf"):
        roofline["bytes"] = ("16S + 32E per launch: the fill pass's interface (column spans from "
                             "the count pass, which reads the seeds and the indptr pairs: 40S)")
    if sum(S + E for S, E, _ in sizes) < (1 << 20):
        # a step this small is a chain of launches, not of bytes: say how many
        roofline["launches_per_step"] = round(
            sum(k["launches"] for k in kernels) / max(args.steps, 1), 1)
        roofline["device_ms_per_step"] = round(
            sum(k["total_ms"] for k in kernels) / max(args.steps, 1), 4)
        roofline["note"] = ("launch-bound step: the dominant kernel's bytes say nothing here; "
                            "launches_per_step and device_ms_per_step do")
    if traffic and dom["avg_ms"] > 0:
        roofline["traffic_source"] = traffic_source
        # the same bytes over this run's launch duration: the rate at the L2-fabric
        # boundary, not an HBM rate
        roofline["fabric_traffic_gbs"] = round(traffic / (dom["avg_ms"] * 1e-3) / 1e9, 1)
    pipeline_bytes = sum(40 * S + 56 * E + 8 * U for S, E, U in sizes)

    # ---- the same workload through the drop-in stack: BatchMatrix + gs.jit.compile +
    # the torch operator class (libgs.so), every layer handed out as per-batch blocks
    api = None
    if args.path == "abi" and not args.no_api:
        api_step = api_step_factory(indptr, indices, seeds, ptr, fanouts, probs)
        for i in range(args.warmup):
            api_step(i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        api_edges = 0
        for i in range(args.steps):
            api_sizes, _ = api_step(args.warmup + i)
            api_edges += sum(E for _, E, _ in api_sizes)
        torch.cuda.synchronize()
        api_elapsed = time.perf_counter() - t0
        # ... and with a Block object made for every mini-batch of every layer
        t0 = time.perf_counter()
        made = 0
        for i in range(args.steps):
            _, layers = api_step(args.warmup + i)
            made += sum(len(blocks.materialize()) for blocks in layers)
        torch.cuda.synchronize()
        api_made = time.perf_counter() - t0
        api = dict(ms_per_step=round(api_elapsed / args.steps * 1e3, 3),
                   value=round(api_edges / api_elapsed, 1),
                   ms_per_step_blocks_materialised=round(api_made / args.steps * 1e3, 3),
                   blocks_per_step=made // max(args.steps, 1),
                   layer_sizes_match=bool(api_sizes == sizes))

    # ---- CPU baseline: the oracle on the first few batches of the same super-batch
    cpu = None
    if args.cpu_seconds > 0:
        from oracle import binding as orc
        h_indptr, h_indices = indptr.cpu().numpy(), indices.cpu().numpy()
        h_seeds, h_ptr = seeds.cpu().numpy(), ptr.cpu().numpy()
        h_probs = probs.cpu().numpy() if probs is not None else None
        h_cdf = cdf.cpu().numpy() if cdf is not None else None

        def cpu_run(call_base):
            t = time.perf_counter()
            sz, _ = graphsage_step(orc, h_indptr, h_indices, h_seeds, h_ptr, fanouts,
                                   args.seed, call_base, h_probs, h_cdf)
            return time.perf_counter() - t, sum(E for _, E, _ in sz)

        cpu_run(0)  # warm-up (page in the graph, spin up the thread pool)
        t_cpu, e_cpu, n_cpu = 0.0, 0, 0
        while t_cpu < args.cpu_seconds and n_cpu < 1000:
            t, e = cpu_run((n_cpu + 1) * len(fanouts))
            t_cpu, e_cpu, n_cpu = t_cpu + t, e_cpu + e, n_cpu + 1
        cpu = dict(value=round(e_cpu / t_cpu, 1), unit="edges/s", cores=orc.num_threads(),
                   kind="port",
                   sample=f"{n_cpu} full super-batches ({wl['batches']} batches each, same "
                          f"graph and seeds, a new sampler call id each) in {t_cpu:.1f} s, "
                          f"OpenMP oracle after one warm-up pass",
                   host_cpus=os.cpu_count())

    out = {
        "metric": "sampled_edges_per_sec", "value": round(edges_per_s, 1), "unit": "edges/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 3), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "int64", "data": "synthetic",
        "config": {"workload": f"{args.workload}: {wl['desc']}", "path": args.path,
                   "fanouts": fanouts, "batches_per_launch": wl["batches"],
                   "seeds_per_batch": wl["batch_size"], "sampler_seed": args.seed,
                   "layer_sizes_S_E_U": sizes},
        "batches_per_sec": round(batches_per_s, 1),
        "pipeline_algorithmic_gbs": round(pipeline_bytes / (ms_per_step * 1e-3) / 1e9, 1),
        "pipeline_frac_of_hbm_peak": round(pipeline_bytes / (ms_per_step * 1e-3) / 1e9
                                           / HBM_PEAK_GBS, 4),
        "roofline": roofline,
        "cpu_baseline": cpu,
        "gpu_over_cpu": round(edges_per_s / cpu["value"], 1) if cpu else None,
        "api_ms_per_step": api["ms_per_step"] if api else None,
        "api_value": api["value"] if api else None,
        "api": api,
        "kernels": [{k: (round(v, 4) if isinstance(v, float) else v) for k, v in kk.items()}
                    for kk in kernels],
        "graph_build_s": round(t_build, 1),
    }
    if cdf is not None:
        out["weight_cdf_build_ms"] = round(t_cdf * 1e3, 2)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
