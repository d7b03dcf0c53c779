#!/usr/bin/env python3
"""Benchmark of the fused per-rank sparse step on one MI355X.

One "step" = score -> exact top-k (lowest-index ties) -> index pack (int32 idx
+ bf16 values) -> residual update -> residual-aware AdamW over the
Llama-3.2-1B-shaped gradient set (1,235,814,400 elements, 146 tensors, bf16
Student-t(3) gradients, fp32 p/m/v/residual) with every input resident in HBM.

The headline is the drop-in layout (resid / p / m / v as the caller's four
flat tensors, as the reference's buffers are) with the Adam-normalised score
(`update`) at 1 %, through the single-sweep step (every array read once;
--two-sweep headlines the step that reads the score inputs twice; its figures
ride along as `two_sweep` either way).

Output: the LAST stdout line is one compact JSON object (a few KB): the
headline, `roofline` of the dominant kernel (timed live with HIP events on its
launch stream), `step_roofline` (the whole step against the bytes it has to
move), `two_sweep`, `packed_layout`, one-line summaries of the Qwen3-0.6B
per-bucket row (`cfg2`) and the 1e9-element stress row (`cfg5`), `replay` and
`cpu_baseline`.  Everything longer -- per-leg tables, the optional full sweep
(--sweep: step variants x scores x ratios x layouts), per-kernel replay
figures, the replay stress draw -- goes to a side file (--detail, default
gpurun_out/bench_detail.json), never to the last line.  Every field called
`frac` is a fraction of the 8 TB/s HBM peak of bytes the measured code has to
move, so none can exceed 1.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12          # MI355X HBM3E, B/s
ALG_BYTES_FINAL = 34.0     # final sweep: read g,r,p,m,v (18) + write r,p,m,v (16)
PROF_FINAL, PROF_SWEEP, PROF_PASS3, PROF_PASS1 = 0, 1, 2, 3     # include/sga_hip_bench.h
# score axis of the replay configuration: |g| (residual-blind, a build-side score with no reference
# counterpart), |g + r| (the registry's abs_g on the accumulated buffer) and the Adam-normalised
# `update`
REPLAY_SCORES = ("abs_g_blind", "abs_g", "update")


def sweep_bytes_per_elem(score, g_bytes=2.0):
    """Algorithmic bytes per element of the select's one data sweep: it reads
    the gradient and the residual, and for the Adam-normalised scores p, m, v
    as well."""
    return g_bytes + 4.0 + (12.0 if score in ("update", "coi") else 0.0)


def step_bytes_per_elem(score, g_bytes=2.0):
    """Whole step: the select sweep + the final sweep (reads g, r, p, m, v,
    writes r, p, m, v)."""
    return sweep_bytes_per_elem(score, g_bytes) + g_bytes + 32.0


def prof_read(L, tag):
    tot, cnt = ctypes.c_double(0), ctypes.c_int(0)
    L.bench_call("sga_prof_read", tag, ctypes.byref(tot), ctypes.byref(cnt))
    return tot.value, cnt.value


def prof_enable(L, on):
    L.bench_call("sga_prof_enable", int(on))


def student_t_dev(n, seed, dev, scale=1e-3, nu=3, chunk=1 << 26):
    import torch
    out = torch.empty(n, dtype=torch.bfloat16, device=dev)
    gen = torch.Generator(device=dev).manual_seed(seed)
    for a in range(0, n, chunk):
        b = min(n, a + chunk)
        z = torch.randn(b - a, generator=gen, device=dev)
        chi = torch.zeros(b - a, device=dev)
        for _ in range(nu):
            chi += torch.randn(b - a, generator=gen, device=dev).pow_(2)
        out[a:b] = (z / torch.sqrt(chi / nu) * scale).to(torch.bfloat16)
    return out


def cpu_baseline(sample_n, steps, ratio, score="abs_g"):
    """Oracle (torch CPU restatement of the reference's pure-torch path) on the
    first ``sample_n`` elements of the same tensor list."""
    import torch
    from oracle import fused_step as OF
    from sga_amd.shapes import llama32_1b, segments_for
    from tests.util import student_t
    shapes, acc = [], 0
    for name, n in llama32_1b()[1:]:          # layer tensors, skipping the embedding
        if acc + n > sample_n:
            break
        shapes.append((name, n))
        acc += n
    segs, n = segments_for(shapes)
    gen = torch.Generator().manual_seed(0)
    p = torch.randn(n, generator=gen) * 0.02
    m, v, r = torch.zeros(n), torch.zeros(n), torch.zeros(n)
    grads = [student_t(n, 100 + s).to(torch.bfloat16) for s in range(steps)]
    OF.fused_sparse_step(grads[0], r, p, m, v, segs, 1, ratio_percent=ratio, score=score,
                         values_dtype=torch.bfloat16)             # warm-up step
    t0 = time.perf_counter()
    for s in range(steps):
        OF.fused_sparse_step(grads[s], r, p, m, v, segs, s + 2, ratio_percent=ratio, score=score,
                             values_dtype=torch.bfloat16)
    dt = time.perf_counter() - t0
    return {"value": n * steps / dt, "unit": "elem/s", "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": f"{len(shapes)} layer tensors of the Llama-3.2-1B list "
                      f"({n} elements), score {score}, {steps} steps at {ratio}% after 1 warm-up step, "
                      f"{dt:.1f} s; host cpu_count={os.cpu_count()}"}


REPLAY_AXES = [(sc, r, t) for sc in REPLAY_SCORES for r in (0.1, 1.0, 10.0) for t in (1, 4, 16)]
# A second, fixed draw that leans on the expensive arms: five Adam-normalised configs (`update`,
# `coi`) at cycle lengths 4 and 16 -- re-selections that read w, m, v and evaluate the exact
# score chain -- and none at T = 1.
REPLAY_STRESS_DRAW = [("update", 1.0, 4), ("update", 0.1, 16), ("coi", 1.0, 4), ("update", 10.0, 4),
                      ("abs_g", 1.0, 4), ("abs_g_blind", 1.0, 16), ("abs_g", 10.0, 16),
                      ("coi", 0.1, 16)]


def replay_draw(G=8, seed=4):
    import random
    return random.Random(seed).sample(REPLAY_AXES, G)


def replay_bytes(n, W, picks):
    """Algorithmic bytes of one window for a list of (score, ratio, T) configs
    (bf16 g read once per pass for the whole group)."""
    alg_p1 = alg_p3 = alg_sw = 0.0
    n_resel = 0
    for s in range(W):
        alg_p1 += 2.0 * n                                    # g in pass 1
        alg_p3 += 2.0 * n                                    # g in pass 3
        for score, _ratio, T in picks:
            bnd = s % T == 0
            rz = s == 0 or (s - 1) % T == 0                  # res is all zeros: no traffic for it
            alg_p1 += ((0.0 if rz else 4.0) if bnd else 0.125) * n  # pass 1: res | sel (1 bit)
            # pass 3: m, v, w read+write; res read unless zero, written unless it stays zero
            alg_p3 += (24.0 + (0.0 if rz else 4.0) + (0.0 if (bnd and rz) else 4.0)
                       + (0.0 if bnd else 0.125)) * n
            if bnd and s > 0 and s + 1 < W:
                if score == "abs_g_blind":
                    per = 2.0                                # the gradient alone
                else:
                    per = (6.0 if score == "abs_g" else 18.0) - (4.0 if rz else 0.0)
                alg_sw += (per + 0.125) * n                  # one score sweep + the new mask bits
                n_resel += 1
    return alg_p1, alg_p3, alg_sw, n_resel


def replay_bench(draws=None, W=32):
    """Fused offline replay on the Qwen3-0.6B shapes: a window of W recorded
    bf16 gradient steps resident in HBM, G = 8 configs from score {|g|, |g+r|,
    update} x ratio {0.1, 1, 10} % x cycle length {1, 4, 16}; per-config fp32
    w/m/v/residual + mask bit planes.  ``draws``: list of (name, picks); the
    window and the branch state are built once and every draw replays it."""
    import torch
    from sga_amd import _lib as L
    from sga_amd.replay import select_topk_flat
    from sga_amd.replay_group import Config, ReplayGroup
    from sga_amd.shapes import qwen3_06b, segments_for
    dev = torch.device("cuda:0")
    if draws is None:
        draws = [("seed 4", replay_draw())]
    segs, n = segments_for(qwen3_06b())
    entries = [{"a": s["start"], "n": s["n"], "b1": s["b1"], "b2": s["b2"], "eps": s["eps"],
                "wd": s["wd"]} for s in segs]
    gen = torch.Generator(device=dev).manual_seed(1)
    w0 = torch.randn(n, generator=gen, device=dev) * 0.02
    m0 = torch.randn(n, generator=gen, device=dev) * 1e-4
    v0 = torch.rand(n, generator=gen, device=dev) * 1e-8
    # slowly drifting per-tensor scale: one scale vector per step applied on the fly
    window = [student_t_dev(n, 500 + s, dev, scale=1e-3 * (1.0 + 0.02 * s)) for s in range(W)]
    base = window[0].float().abs()
    meta = {"clip_grad": 1.0, "grad_norm": float("nan"), "lr": 1e-4}
    out = []
    for name, picks in draws:
        cfgs = [Config(*p) for p in picks]
        G = len(cfgs)
        # branch selection on |g0| (cheap stand-in for the front block)
        sel0 = [select_topk_flat(base, max(1, int(round(c.ratio / 100.0 * n))))[0] for c in cfgs]
        grp = ReplayGroup(entries, w0, m0, v0, sel0, cfgs, t0=100, window=W)
        del sel0
        torch.cuda.synchronize()
        prof_enable(L, 1)
        t0 = time.perf_counter()
        for s in range(W):
            grp.step(window[s], meta)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        p3_ms, p3_n = prof_read(L, PROF_PASS3)
        p1_ms, p1_n = prof_read(L, PROF_PASS1)
        sw_ms, sw_n = prof_read(L, PROF_SWEEP)
        prof_enable(L, 0)
        del grp
        torch.cuda.empty_cache()
        alg_p1, alg_p3, alg_sw, n_resel = replay_bytes(n, W, picks)
        alg = alg_p1 + alg_p3 + alg_sw
        kernels = {}
        for kname, ms, cnt, b in (("k_replay_pass3", p3_ms, p3_n, alg_p3),
                                  ("k_replay_pass1 (launches of one step)", p1_ms, p1_n, alg_p1),
                                  ("k_bracket_sweep<SrcReplay>", sw_ms, sw_n, alg_sw)):
            if cnt:
                kernels[kname] = {"launches": cnt, "total_ms": ms, "avg_ms": ms / cnt,
                                  "alg_bytes": b,
                                  "frac": b / (ms * 1e-3) / HBM_PEAK if ms > 0 else None}
        timed = p3_ms + p1_ms + sw_ms
        out.append({
            "draw": name, "metric": "replay config-steps/s", "value": G * W / dt,
            "unit": "config-steps/s", "ms_per_window": dt * 1e3, "G": G, "W": W, "n": n,
            "reselects": n_resel, "configs": [list(p) for p in picks],
            "alg_bytes": alg, "achieved_GBps": alg / dt / 1e9, "frac": alg / dt / HBM_PEAK,
            "roofline": {"bound": "hbm", "kernel": "k_replay_pass3",
                         "achieved": alg_p3 / (p3_ms * 1e-3) / 1e9 if p3_ms > 0 else None,
                         "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                         "frac": alg_p3 / (p3_ms * 1e-3) / HBM_PEAK if p3_ms > 0 else None,
                         "avg_ms": p3_ms / max(p3_n, 1), "traffic": None},
            "kernels": kernels,
            "other_kernels_and_gaps_ms": dt * 1e3 - timed,
            "workload": "Qwen3-0.6B shapes (596,049,920 elems, 310 tensors), bf16 Student-t(3) "
                        "window, per-config fp32 w/m/v/res + mask bit planes resident, clip 1.0"})
    return out


def replay_cpu_baseline(G=8, W=8, seed=4, frac=24):
    """The oracle's group loop (the reference's eager torch chain) on a 1/frac
    prefix of the Qwen3-0.6B tensor list, same config draw as replay_bench, W
    steps; the rate is scaled linearly to the full shard."""
    import random
    import torch
    from oracle import replay as OR
    from oracle import select as SEL
    from sga_amd.shapes import qwen3_06b, segments_for
    from tests.util import student_t
    full_n = sum(n for _, n in qwen3_06b())
    shapes, acc = [], 0
    for name, n in qwen3_06b()[1:]:               # layer tensors, skipping the embedding
        if acc + n > full_n // frac:
            break
        shapes.append((name, n))
        acc += n
    segs, n = segments_for(shapes)
    entries = [{"a": s["start"], "n": s["n"], "b1": s["b1"], "b2": s["b2"], "eps": s["eps"],
                "wd": s["wd"]} for s in segs]
    cfgs = [OR.Config(*p) for p in replay_draw(G, seed)]
    gen = torch.Generator().manual_seed(1)
    w0 = torch.randn(n, generator=gen) * 0.02
    m0 = torch.randn(n, generator=gen) * 1e-4
    v0 = torch.rand(n, generator=gen) * 1e-8
    window = [(student_t(n, 500 + s) * (1.0 + 0.02 * s)).to(torch.bfloat16) for s in range(W)]
    base = window[0].float().abs()
    sel0 = [SEL.select_topk_flat(base, SEL.replay_k(n, c.ratio))[0] for c in cfgs]
    metas = [{"clip_grad": 1.0, "grad_norm": float("nan"), "lr": 1e-4}] * W
    t0 = time.perf_counter()
    OR.group_replay(entries, w0, m0, v0, sel0, cfgs, window, metas, 100)
    dt = time.perf_counter() - t0
    return {"value": G * W / dt * n / full_n, "unit": "config-steps/s", "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": f"{len(shapes)} layer tensors of the Qwen3-0.6B list ({n} elements = 1/"
                      f"{full_n / n:.1f} of the shard), G={G}, W={W}, {dt:.1f} s; rate scaled "
                      f"linearly to the full shard; host cpu_count={os.cpu_count()}"}


def primitives_bench(n=1 << 28, ratio=1.0):
    """The drop-in primitives on their own (one flat fp32 bucket of n elements,
    k = ratio %): algorithmic bytes over wall time per call."""
    import torch
    from sga_amd import kernels as K
    from sga_amd import replay_kernels as RK
    from sga_amd.adamw import (adamw_grad_correct, adamw_grad_correct_compact, build_dir_table)
    from sga_amd.replay import select_topk_flat
    from sga_amd.selection import select_masks_histogram
    from sga_amd.support import IndexPool, compact_mask_u8
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev).manual_seed(0)
    g = torch.randn(n, generator=gen, device=dev) * 1e-3
    p = torch.randn(n, generator=gen, device=dev) * 0.02
    m = torch.randn(n, generator=gen, device=dev) * 1e-4
    v = torch.rand(n, generator=gen, device=dev) * 1e-8
    k = max(1, int(round(n * ratio / 100.0)))
    score = g.abs()
    mask_b, _ = select_topk_flat(score, k)
    mask = mask_b.view(torch.uint8)
    pool = IndexPool()
    idx = compact_mask_u8(mask, pool).clone()
    values = torch.empty(k, device=dev)
    total = torch.zeros(1, device=dev)
    table = build_dir_table(idx, n)
    out = torch.empty(n, device=dev)
    rows = []

    def timed(name, alg_bytes, fn, reps=5):
        fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) / reps * 1e3
        rows.append({"op": name, "ms": ms, "alg_GB": alg_bytes / 1e9,
                     "GBps": alg_bytes / ms / 1e6, "frac": alg_bytes / ms / 1e6 / 8000.0})

    timed("select_topk_flat (exact, lowest-index ties, mask out)", n * 5.0,
          lambda: select_topk_flat(score, k, check=False))
    timed("select_masks_histogram exact (ties all)", n * 5.0,
          lambda: select_masks_histogram([g], k, mode="exact"))
    timed("select_masks_histogram balanced", n * (4.0 / 8 + 5.0),
          lambda: select_masks_histogram([g], k, mode="balanced"))
    timed("compact_mask_u8", n * 2.0 + k * 4.0, lambda: compact_mask_u8(mask, pool))
    timed("pack_selected (fp32 values)", k * (4 + 32 + 32 + 4.0),
          lambda: K.pack_selected(g, idx, values, 1.0))
    timed("scatter_selected", k * (4 + 4 + 32.0), lambda: K.scatter_selected(g, idx, values))
    timed("compact_norm_sq_contribution", k * 4.0,
          lambda: K.compact_norm_sq_contribution(values, total))
    timed("masked_norm_sq_contribution", n * 5.0,
          lambda: K.masked_norm_sq_contribution(g, mask, total))
    timed("adamw_grad_correct sparse (mask, clear)", n * 33.0,
          lambda: adamw_grad_correct(p, g, m, v, 1e-4, 0.9, 0.95, 1e-8, 0.1, 3, mask=mask,
                                     coeff=0.5, clear=True))
    timed("adamw_grad_correct full (emit update)", n * 32.0,
          lambda: adamw_grad_correct(p, g, m, v, 1e-4, 0.9, 0.95, 1e-8, 0.1, 3,
                                     emit_score="update"))
    timed("adamw_grad_correct_compact (dir table)", n * 24.0 + k * 8.0,
          lambda: adamw_grad_correct_compact(p, g, m, v, idx, values, 0, 1e-4, 0.9, 0.95, 1e-8,
                                             0.1, 3, coeff=0.5, dir_table=table))
    timed("formula('update') score", n * 20.0,
          lambda: RK.formula("update")(p, m, v, g, 0.9, 0.95, 1e-8, 0.1, 0.271, 0.143))   # w, m, v, g
    timed("opt_step_inplace (replay commit)", n * 28.0,
          lambda: RK.opt_step_inplace(g, m, v, p, None, 1e-4, 0.1, 0.9, 0.95, 0.271, 0.143, 1e-8))
    from sga_amd.clip import scale_masked_
    from sga_amd.selection import threshold_masks
    tau = float(score.float().kthvalue(n - k + 1).values) if n <= (1 << 24) else 2.58e-3
    timed("threshold_masks (|g| >= tau, mask + count)", n * 5.0, lambda: threshold_masks([g], tau))
    timed("scale_masked_ (clip scale under a mask)", n * 1.0 + k * 64.0,
          lambda: scale_masked_(g, mask, 1.0))
    timed("scale_masked_ (whole tensor)", n * 8.0, lambda: scale_masked_(g, None, 1.0))
    timed("gt_eq_counts (two masks + counts)", n * 6.0, lambda: RK.gt_eq_counts(score, tau))
    timed("hist_top16 (incl. 256 KiB histogram to host)", n * 4.0, lambda: RK.hist_top16(score))
    return {"n": n, "k": k, "rows": rows,
            "note": "pack/scatter bytes count a 32-byte sector per random 4-byte access"}


def trace_io_bench(W=4, tmp=None):
    """Recorded-trace leg: writes a W-step bf16 trace of the Qwen3-0.6B shapes in
    the reference writer's layout under a temp dir, then streams it back through
    the pread reader (page cache warm) -- once on its own and once feeding the
    dense reference pass -- to measure the PCIe-inclusive rates."""
    import shutil
    import tempfile
    import torch
    from sga_amd import trace_io as T
    from sga_amd.replay_dense import DenseReplay
    from sga_amd.shapes import qwen3_06b
    dev = torch.device("cuda:0")
    shapes = qwen3_06b()
    d = tempfile.mkdtemp(prefix="sga_trace_", dir=tmp)
    try:
        cat = {name: {"shape": [n], "dtype": "torch.float32"} for name, n in shapes}
        meta = {"step": 100, "phase": "shadow", "lr": [1e-4], "grad_norm": float("nan"),
                "clip_grad": 0.0, "weight_decay": 0.1, "adam_beta1": 0.9, "adam_beta2": 0.95,
                "adam_eps": 1e-8}
        T.write_catalog(d, cat, meta, "bf16")
        gen = torch.Generator().manual_seed(0)
        zeros = {name: torch.zeros(n) for name, n in shapes}
        w = {name: torch.randn(n, generator=gen) * 0.02 for name, n in shapes}
        T.write_state(d, 100, meta, w, zeros, zeros)
        del zeros
        for s in range(W):
            T.write_grad(d, 100 + s, dict(meta, step=100 + s),
                         {name: (torch.randn(n, generator=gen) * 1e-3) for name, n in shapes},
                         torch.bfloat16)
        catalog, names, _o, N, s_files, g_files = T.discover_trace(d)
        sp = T.ShardParams(names, catalog, meta, 0, N)
        steps = T.window_steps_for(g_files, 100, W)
        cache = {}
        for _gs, _m, g in T.WindowReader(g_files, steps, sp, dev, index_cache=cache):
            pass                                           # warm: page cache, index, buffers
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _gs, _m, g in T.WindowReader(g_files, steps, sp, dev, index_cache=cache):
            pass
        torch.cuda.synchronize()
        dt_read = time.perf_counter() - t0
        w0, m0, v0, _ = T.load_branch_state(s_files[100], sp, dev)
        dense = DenseReplay(sp.entries, w0, m0, v0, 100)
        t0 = time.perf_counter()
        for gs, gm, g in T.WindowReader(g_files, steps, sp, dev, index_cache=cache):
            dense.step(gs, g, gm)
        torch.cuda.synchronize()
        dt_dense = time.perf_counter() - t0
        t0 = time.perf_counter()
        for _ in range(W):                                 # same step, gradient resident
            dense.step(gs, g, gm)
        torch.cuda.synchronize()
        dt_res = time.perf_counter() - t0
        return {"workload": f"Qwen3-0.6B shapes, {W} recorded bf16 steps ({N} elems each), "
                            "files in the page cache",
                "reader_GBps": W * N * 2 / dt_read / 1e9, "reader_ms_per_step": dt_read / W * 1e3,
                "dense_pass_ms_per_step": dt_dense / W * 1e3,
                "dense_pass_elem_per_s": W * N / dt_dense,
                "dense_step_resident_ms": dt_res / W * 1e3}
    finally:
        shutil.rmtree(d, ignore_errors=True)


def qwen_mask_layout_row(steps=5, warmup=2):
    """Qwen3-0.6B-shaped set, bf16 Gaussian grads with per-tensor std
    log-uniform in [1e-5, 1e-2], per-bucket exact top-k at 1 % (the embedding,
    then seven buckets of four layers), mask backend layout: the step's outputs
    are the uint8 mask and the ordered payload (what `torch_pipelined_mask`
    hands to the all-reduce), fp32 values."""
    import torch
    from sga_amd.fused_step import FusedSparseStep, fused_step_multi, k_for
    from sga_amd.shapes import qwen3_06b, segments_for
    dev = torch.device("cuda:0")
    segs, n = segments_for(qwen3_06b())
    gen = torch.Generator(device=dev).manual_seed(5)
    cpu_gen = torch.Generator().manual_seed(5)
    grads = []
    for rep in range(2):
        g = torch.empty(n, dtype=torch.bfloat16, device=dev)
        for s in segs:
            std = 10 ** (-5 + 3 * float(torch.rand(1, generator=cpu_gen)))
            g[s["start"]:s["start"] + s["n"]] = (
                torch.randn(s["n"], generator=gen, device=dev) * std).to(torch.bfloat16)
        grads.append(g)
    cuts = [0, segs[1]["start"]] + [segs[1 + 11 * j]["start"] for j in range(4, 28, 4)] + [n]
    p = torch.randn(n, generator=gen, device=dev) * 0.02
    m, v, r = (torch.zeros(n, device=dev) for _ in range(3))
    buckets = []
    for lo, hi in zip(cuts[:-1], cuts[1:]):
        bsegs = [dict(s, start=s["start"] - lo) for s in segs if lo <= s["start"] < hi]
        k = k_for(hi - lo, 1.0)
        buckets.append((lo, hi, k, FusedSparseStep(hi - lo, bsegs, dev, values_dtype=torch.float32,
                                                   max_k=k, want_mask=True)))

    # The eight buckets go out as ONE call: the short dependent kernels around a select run once
    # for all of them (the kernels take the bucket from the grid's second dimension), only the
    # sweeps are launched per bucket.
    steppers = [b[3] for b in buckets]
    ks = [b[2] for b in buckets]
    views = [[t[lo:hi] for lo, hi, _k, _fs in buckets] for t in (r, p, m, v)]

    def one(t):
        g = grads[t % 2]
        fused_step_multi(steppers, [g[lo:hi] for lo, hi, _k, _fs in buckets], *views, t + 1, ks=ks)

    torch.cuda.synchronize()
    for t in range(warmup):
        one(t)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for t in range(warmup, warmup + steps):
        one(t)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    for lo, hi, k, fs in buckets:
        res = fs.read_result()
        assert res.status == 0 and res.n_selected == k, vars(res)
    ktot = sum(b[2] for b in buckets)
    alg = n * (step_bytes_per_elem("abs_g") + 1.0) + ktot * 8.0       # + u8 mask, idx + fp32 payload
    return {"workload": "Qwen3-0.6B-shaped set (596,049,920 elems, 310 tensors), bf16 Gaussian grads "
                        "with per-tensor std log-uniform in [1e-5, 1e-2], per-bucket exact top-k 1 % "
                        f"over {len(buckets)} buckets, score abs_g, mask layout (u8 mask + ordered "
                        "fp32 payload), four flat state tensors, all buckets in one "
                        "sga_fused_sparse_step_multi call",
            "n": n, "buckets": len(buckets), "k_total": ktot,
            "ms_per_step": dt * 1e3,
            "elem_per_s": n / dt, "alg_bytes_per_step": alg,
            "step_frac": alg / dt / HBM_PEAK}


def stress_row(steps=3):
    """One contiguous 1.0e9-element fp32 gradient buffer, heavy-tailed with
    5 % duplicated magnitudes: the exact global top-k alone at 0.01 % and 1 %
    (mask out), then the fused residual-aware AdamW step at 1 % (fp32 grads,
    index pack int32 + fp32)."""
    import torch
    from sga_amd.fused_step import FusedSparseStep, k_for
    from sga_amd.replay import select_topk_flat
    dev = torch.device("cuda:0")
    n = 1_000_000_000
    g = student_t_dev(n, 7, dev).float()
    gen = torch.Generator(device=dev).manual_seed(1)
    dup = torch.randint(0, n, (n // 20,), generator=gen, device=dev)
    g[dup] = g[dup.roll(1)]
    del dup
    score = g.abs()
    sel = {}
    for ratio in (0.01, 1.0):
        k = k_for(n, ratio)
        select_topk_flat(score, k, check=False)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            mask, th = select_topk_flat(score, k, check=False)
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / steps
        assert int(mask.sum()) == k
        sel[str(ratio)] = {"k": k, "ms": dt * 1e3, "elem_per_s": n / dt,
                           "frac": n * (4.0 + 1.0) / dt / HBM_PEAK}
        del mask
    del score
    segs = [dict(start=0, n=n, lr=1e-4, b1=0.9, b2=0.95, eps=1e-8, wd=0.1)]
    p = torch.randn(n, generator=gen, device=dev) * 0.02
    m, v, r = (torch.zeros(n, device=dev) for _ in range(3))
    k = k_for(n, 1.0)
    fs = FusedSparseStep(n, segs, dev, values_dtype=torch.float32, max_k=k)
    fs.step(g, r, p, m, v, 1, k=k)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for t in range(steps):
        fs.step(g, r, p, m, v, t + 2, k=k)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    res = fs.read_result()
    assert res.status == 0 and res.n_selected == k, vars(res)
    alg = n * step_bytes_per_elem("abs_g", 4.0) + k * 8.0
    return {"workload": "one contiguous 1.0e9-element fp32 buffer, Student-t(3) with 5 % duplicated "
                        "magnitudes; select_topk_flat alone (mask out; bytes = 4 read "
                        "+ 1 mask) and the fused step at 1 % (fp32 grads, idx int32 + fp32 values)",
            "n": n, "select_only": sel,
            "fused_step": {"k": k, "ms_per_step": dt * 1e3, "elem_per_s": n / dt,
                           "alg_bytes_per_step": alg, "step_frac": alg / dt / HBM_PEAK,
                           "path": res.path}}


def load_traffic(layout, score, ratio, single):
    """HBM bytes per launch of the final sweep from the committed counter
    profile -- only when that profile was taken on this very configuration."""
    tpath = os.path.join(ROOT, "profiles", "fused_final_llama1b_traffic.json")
    try:
        entries = json.load(open(tpath))
    except Exception:
        return None, None
    if isinstance(entries, dict):
        entries = [entries]
    for e in entries:
        c = e.get("config", {})
        if (c.get("layout"), c.get("score"), c.get("ratio_percent"),
                bool(c.get("single_sweep", False))) == (layout, score, ratio, bool(single)):
            return e.get("hbm_bytes_per_launch"), "profiles/fused_final_llama1b_traffic.json"
    return None, None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--ratio", type=float, default=1.0)
    ap.add_argument("--score", default="update",
                    help="headline score: update (the Adam-normalised score of the benchmark "
                         "configuration) or abs_g (|g + residual|)")
    ap.add_argument("--layout", choices=("separate", "packed"), default="separate",
                    help="headline state layout: separate = the drop-in entry point on four flat "
                         "tensors; packed = the library-owned 64 KiB records")
    ap.add_argument("--two-sweep", dest="single_sweep", action="store_false",
                    help="headline the two-sweep step (select sweep + final sweep: the score "
                         "inputs are read twice) instead of the single-sweep step")
    ap.add_argument("--in-place", action="store_true",
                    help="headline the IN-PLACE single-sweep step (a missed bracket ends in status 3 "
                         "with the state overwritten) instead of the out-of-place one on ping-pong "
                         "state, which redoes a missed bracket on the device")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--cpu-sample", type=int, default=1 << 28)
    ap.add_argument("--calib", action="store_true",
                    help="also launch one plain copy of 2^30 fp32 (k_calib_copy) and the math-free "
                         "stream stand-in so counter runs can be scaled against known traffic")
    ap.add_argument("--no-replay", action="store_true", help="skip the fused replay leg")
    ap.add_argument("--sweep", action="store_true",
                    help="also time the whole sweep {two-sweep, single-sweep} x {update, abs_g} x "
                         "{0.1, 1, 10 %} x {separate, packed} (24 legs; written to the detail file)")
    ap.add_argument("--headline-only", action="store_true",
                    help="time the headline configuration alone: no other step variant, no other "
                         "layout, no stream-mix copy (what the profiles are taken on)")
    ap.add_argument("--no-rows", action="store_true",
                    help="skip the Qwen3-0.6B mask-layout row and the 1e9 stress row")
    ap.add_argument("--detail", default=os.path.join(ROOT, "gpurun_out", "bench_detail.json"),
                    help="side file for everything longer than the compact last line "
                         "('' = do not write one)")
    ap.add_argument("--trace-io", action="store_true",
                    help="run just the recorded-trace leg (writes a temporary trace, streams it "
                         "back through the pread reader and the dense pass) and print its JSON")
    ap.add_argument("--primitives", action="store_true",
                    help="time the drop-in primitives on their own and print their JSON")
    ap.add_argument("--only-rows", action="store_true",
                    help="run just the Qwen3-0.6B mask-layout row and the 1e9 stress row (for "
                         "profiling) and print their JSON")
    ap.add_argument("--only-replay", action="store_true",
                    help="run just the fused replay leg (for profiling) and print its JSON")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs one data-parallel rank's share on ONE GPU; "
              "there are no collectives, so --gpus must be 1", file=sys.stderr)
        sys.exit(2)

    import torch
    from sga_amd import _lib as L
    L.load_bench()          # timing observer + calibration kernels: before libsga_hip.so binds
    from sga_amd.fused_step import FusedSparseStep, PackedState, k_for
    from sga_amd.shapes import llama32_1b, segments_for

    L.load()
    if args.only_rows:
        torch.cuda.set_device(0)
        print(json.dumps({"qwen06b_mask_layout": qwen_mask_layout_row(),
                          "stress_1e9": stress_row()}))
        return
    if args.only_replay:
        torch.cuda.set_device(0)
        print(json.dumps(replay_bench()[0]))
        return
    if args.trace_io:
        torch.cuda.set_device(0)
        print(json.dumps(trace_io_bench()))
        return
    if args.primitives:
        torch.cuda.set_device(0)
        print(json.dumps(primitives_bench()))
        return
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    segs, n = segments_for(llama32_1b())
    gen = torch.Generator(device=dev).manual_seed(0)
    p = torch.randn(n, generator=gen, device=dev) * 0.02
    m = torch.zeros(n, device=dev)
    v = torch.zeros(n, device=dev)
    r = torch.zeros(n, device=dev)
    grads = [student_t_dev(n, 10 + i, dev) for i in range(2)]
    fs = FusedSparseStep(n, segs, dev, values_dtype=torch.bfloat16,
                         max_k=k_for(n, 10.0) + 16)

    def events_ms(fn, reps=5):
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
        fn()
        ev[0].record()
        for _ in range(reps):
            fn()
        ev[1].record()
        torch.cuda.synchronize()
        return ev[0].elapsed_time(ev[1]) / reps

    calib = None
    if args.calib:
        cn = 1 << 30
        src = torch.ones(cn, device=dev)
        dst = torch.empty(cn, device=dev)
        ms = events_ms(lambda: L.bench_call("sga_calib_copy", L.ptr(dst), L.ptr(src), cn, L.stream()))
        calib = {"kernel": "k_calib_copy", "bytes": cn * 8, "avg_ms": ms,
                 "GBps": cn * 8 / ms / 1e6}
        del src, dst
        # the final sweep's own mix of streams without its math, on scratch arrays
        sg = torch.zeros(n, dtype=torch.bfloat16, device=dev)
        sc = [torch.zeros(n, device=dev) for _ in range(4)]
        sargs = [L.ptr(sg)] + [L.ptr(t) for t in sc] + [n, L.stream()]
        ms = events_ms(lambda: L.bench_call("sga_calib_streams", *sargs))
        calib["streams"] = {"kernel": "k_calib_streams", "bytes": n * 34, "avg_ms": ms,
                            "GBps": n * 34 / ms / 1e6}
        del sg, sc

    state = {"t": 0, "packed": None}
    max_steps = max(args.steps, 5)
    results = torch.zeros(max_steps, 8, dtype=torch.int32, device=dev)   # a result block per step

    def time_leg(layout, score, ratio, warmup, steps, single=False, oop=False, no_g=False):
        """`warmup` untimed + exactly `steps` timed steps of one configuration.  `oop`: the
        out-of-place single-sweep step on ping-pong state (flat tensors).  `no_g`: the
        reference's own buffer contract, resid already holds g + r and the step takes no
        separate gradient (backward's accumulation is not part of the step, so the buffer is
        not refreshed between the timed steps)."""
        gb = 0.0 if no_g else 2.0
        k = k_for(n, ratio)
        if layout == "packed" and state["packed"] is None:
            state["packed"] = PackedState(n, dev).pack(r, p, m, v)
        elif layout == "separate" and state["packed"] is not None:
            state["packed"].unpack(r, p, m, v)
            state["packed"] = None
        if oop and layout == "packed":
            sets = [state["packed"], PackedState(n, dev)]
        else:
            sets = [[r, p, m, v], [torch.empty_like(r) for _ in range(4)] if oop else None]

        def step_fn(t, res=None):
            if no_g:
                fs.step(None, r, p, m, v, t + 1, k=k, score=score, single_sweep=single,
                        check=False, result=res)
            elif oop and layout == "packed":
                fs.step_packed(grads[t % 2], sets[0], t + 1, k=k, score=score, single_sweep=True,
                               check=False, result=res, out=sets[1])
                sets.reverse()
                state["packed"] = sets[0]
            elif oop:
                fs.step(grads[t % 2], *sets[0], t + 1, k=k, score=score, single_sweep=True,
                        check=False, result=res, out=sets[1])
                sets.reverse()
            elif layout == "packed":
                fs.step_packed(grads[t % 2], state["packed"], t + 1, k=k, score=score,
                               single_sweep=single, check=False, result=res)
            else:
                fs.step(grads[t % 2], r, p, m, v, t + 1, k=k, score=score, single_sweep=single,
                        check=False, result=res)
        for _ in range(warmup):
            step_fn(state["t"])
            state["t"] += 1
        torch.cuda.synchronize()
        prof_enable(L, 1)
        t0 = time.perf_counter()
        for i in range(steps):
            step_fn(state["t"], results[i])
            state["t"] += 1
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        fin_ms, fin_n = prof_read(L, PROF_FINAL)
        sw_ms, sw_n = prof_read(L, PROF_SWEEP)
        prof_enable(L, 0)
        if oop and layout != "packed" and sets[0][0] is not r:   # leave the current state in r / p / m / v
            for dst, src in zip((r, p, m, v), sets[0]):
                dst.copy_(src)
        # every timed step must have ended as an exact top-k step (status word 0, k selected)
        rows = results[:steps].cpu()
        assert bool((rows[:, 6] == 0).all()) and bool((rows[:, 4] == k).all()), rows.tolist()
        from sga_amd.selection import read_result
        res = read_result(results[steps - 1])
        # dominant kernel: k_fused_final reads g, r, p, m, v, writes r, p, m, v and the pack
        # (4 + 2 B per selected coordinate); k_fused_spec (single sweep) the same state traffic
        # and one staged 2 B value per coordinate it takes as selected
        final_bytes = n * (ALG_BYTES_FINAL - 2.0 + gb) + k * (2.0 if single else 6.0)
        sweep_bytes = 0.0 if single else n * sweep_bytes_per_elem(score, gb)
        # bytes the step has to move: every array once (34 B per element + the pack) for the
        # single sweep; the score inputs once more for the two-sweep step's select
        once_bytes = n * (ALG_BYTES_FINAL - 2.0 + gb) + k * 6.0
        two_read_bytes = n * step_bytes_per_elem(score, gb) + k * 6.0
        moved = once_bytes if single else two_read_bytes
        fin_avg, sw_avg = fin_ms / max(fin_n, 1), sw_ms / max(sw_n, 1)
        return {"layout": layout, "single_sweep": single, "out_of_place": oop,
                "separate_gradient": not no_g, "score": score,
                "ratio_percent": ratio,
                "k": k, "steps": steps, "seconds": dt, "ms_per_step": dt / steps * 1e3,
                "elem_per_s": n * steps / dt,
                "moved_bytes_per_elem": moved / n, "moved_bytes_per_step": moved,
                "step_frac": moved * steps / dt / HBM_PEAK,
                # not a roofline fraction: the rate this step would need under the two-read
                # byte model (52 B per element for `update`, 40 for |g + r|), relative to peak
                "speedup_vs_two_read_model": two_read_bytes * steps / dt / HBM_PEAK,
                "final_avg_ms": fin_avg, "final_bytes": final_bytes,
                "final_frac": final_bytes / (fin_avg * 1e-3) / HBM_PEAK if fin_avg > 0 else None,
                "sweep_avg_ms": sw_avg, "sweep_bytes": sweep_bytes,
                "sweep_frac": sweep_bytes / (sw_avg * 1e-3) / HBM_PEAK if sw_avg > 0 else None,
                "other_kernels_ms": dt / steps * 1e3 - fin_avg - sw_avg,
                "select": {"thresh": res.thresh, "n_gt": res.n_gt, "n_eq": res.n_eq,
                           "path": res.path}}

    # the headline single-sweep step runs out of place on ping-pong state unless --in-place
    head_oop = bool(args.single_sweep and not args.in_place)
    head = time_leg(args.layout, args.score, args.ratio, args.warmup, args.steps, args.single_sweep,
                    oop=head_oop)
    stream_mix = None
    if args.layout == "separate" and not args.headline_only:
        # What the same five read and four write streams reach WITHOUT the math, on the very
        # tensors the headline ran on: the ceiling this placement of four flat tensors gives a
        # kernel of that stream mix.  (It scribbles over r / p / m / v: they are reset below.)
        sargs = [L.ptr(grads[0]), L.ptr(r), L.ptr(p), L.ptr(m), L.ptr(v), n, L.stream()]
        ms = events_ms(lambda: L.bench_call("sga_calib_streams", *sargs))
        stream_mix = {"kernel": "k_calib_streams (same five read / four write streams, no math), "
                                "same tensors as the headline",
                      "avg_ms": ms, "frac": n * ALG_BYTES_FINAL / (ms * 1e-3) / HBM_PEAK}
        gen = torch.Generator(device=dev).manual_seed(0)
        p.copy_(torch.randn(n, generator=gen, device=dev) * 0.02)
        m.zero_(); v.zero_(); r.zero_()
        state["t"] = 0
    # the other step variant and the other layout of the headline configuration
    other = packed_leg = oop_leg = nog_leg = None
    if not args.headline_only:
        other = time_leg(args.layout, args.score, args.ratio, 2, 5, not args.single_sweep)
        oop_leg = time_leg(args.layout, args.score, args.ratio, 2, 5, True, oop=not head_oop)
        if args.score != "abs_g_blind":
            # the buffer must hold a gradient's worth of values for the first of these steps
            r.add_(grads[0].float())
            nog_leg = time_leg("separate", args.score, args.ratio, 2, 5, args.single_sweep, no_g=True)
        packed_leg = time_leg("packed" if args.layout == "separate" else "separate", args.score,
                              args.ratio, 2, 5, args.single_sweep, oop=head_oop)
    two = head if not args.single_sweep else other
    sweep = []
    if args.sweep:
        for single in (False, True):
            for layout in ("separate", "packed"):
                for score in ("update", "abs_g"):
                    for ratio in (0.1, 1.0, 10.0):
                        sweep.append(time_leg(layout, score, ratio, 1, 5, single))
    if state["packed"] is not None:
        state["packed"].unpack(r, p, m, v)
        state["packed"] = None
    traffic, traffic_src = load_traffic(args.layout, args.score, args.ratio, args.single_sweep)
    k = head["k"]
    value = n * args.steps / head["seconds"]
    entry = ("sga_fused_sparse_step" + ("_single_sweep" if args.single_sweep else "")
             + ("_packed" if args.layout == "packed" else "") + ("_out" if head_oop else ""))
    out = {
        "metric": "grad elems/s (score+top-k+resid AdamW)",
        "value": value, "unit": "elem/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": head["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "Llama-3.2-1B-shaped set (BASELINE cfg 3), 1,235,814,400 elems / "
                               "146 tensors, bf16 Student-t(3) grads, fp32 p/m/v/residual, score "
                               f"{args.score}, exact top-k {args.ratio}%, index pack int32+bf16, "
                               f"residual-aware AdamW; entry point {entry}"
                               + (" (new state written to a second set of arrays: a missed "
                                  "bracket is redone on the device, never lost)" if head_oop else ""),
                   "ratio_percent": args.ratio, "score": args.score, "k": k,
                   "single_sweep": bool(args.single_sweep), "out_of_place": head_oop,
                   "state_layout": args.layout},
        "roofline": {"bound": "hbm",
                     "kernel": "k_fused_spec" if args.single_sweep else "k_fused_final",
                     "avg_ms": head["final_avg_ms"],
                     "alg_bytes_per_launch": head["final_bytes"],
                     "achieved": head["final_bytes"] / (head["final_avg_ms"] * 1e-3) / 1e9,
                     "peak": HBM_PEAK / 1e9, "unit": "GB/s", "frac": head["final_frac"],
                     "traffic": traffic,
                     "stream_mix_copy_frac": stream_mix["frac"] if stream_mix else None},
        # the whole step against the bytes this step variant has to move
        "step_roofline": {"bytes_per_elem": head["moved_bytes_per_elem"],
                          "frac": head["step_frac"],
                          "other_kernels_ms": head["other_kernels_ms"]},
    }
    if two is not None:
        out["two_sweep"] = {
            "ms_per_step": two["ms_per_step"], "elem_per_s": two["elem_per_s"],
            "bytes_per_elem": two["moved_bytes_per_elem"], "frac": two["step_frac"],
            "k_fused_final_ms": two["final_avg_ms"], "k_fused_final_frac": two["final_frac"],
            "k_bracket_sweep_ms": two["sweep_avg_ms"], "k_bracket_sweep_frac": two["sweep_frac"]}
    if packed_leg is not None:
        out["packed_layout" if args.layout == "separate" else "separate_layout"] = {
            "ms_per_step": packed_leg["ms_per_step"], "elem_per_s": packed_leg["elem_per_s"],
            "frac": packed_leg["step_frac"], "dominant_kernel_ms": packed_leg["final_avg_ms"],
            "dominant_kernel_frac": packed_leg["final_frac"]}
    if oop_leg is not None:
        out["in_place" if head_oop else "out_of_place"] = {
            "what": ("single-sweep step in place (a missed bracket ends in status 3)" if head_oop else
                     "single-sweep step on ping-pong state (a missed bracket is redone, never lost)"),
            "ms_per_step": oop_leg["ms_per_step"], "elem_per_s": oop_leg["elem_per_s"],
            "frac": oop_leg["step_frac"], "dominant_kernel_ms": oop_leg["final_avg_ms"],
            "dominant_kernel_frac": oop_leg["final_frac"]}
    if nog_leg is not None:
        out["single_buffer"] = {
            "what": "same step, no separate gradient: the fp32 buffer already holds g + r (the "
                    "reference's own contract)",
            "ms_per_step": nog_leg["ms_per_step"], "elem_per_s": nog_leg["elem_per_s"],
            "bytes_per_elem": nog_leg["moved_bytes_per_elem"], "frac": nog_leg["step_frac"],
            "dominant_kernel_ms": nog_leg["final_avg_ms"],
            "dominant_kernel_frac": nog_leg["final_frac"]}
    detail = {"headline_leg": head, "other_variant_leg": other, "other_layout_leg": packed_leg,
              "single_buffer_leg": nog_leg,
              "out_of_place_leg": oop_leg,
              "select": head["select"], "traffic_source": traffic_src,
              "stream_mix_copy": stream_mix}
    if sweep:
        detail["sweep"] = sweep
    if calib:
        detail["copy_calibration"] = calib
    del p, m, v, r, grads, fs
    torch.cuda.empty_cache()
    if not args.no_rows:
        row = qwen_mask_layout_row()
        detail["qwen06b_mask_layout"] = row
        out["cfg2"] = {"what": "Qwen3-0.6B set, 8 buckets, abs_g 1 %, mask layout, two-sweep step",
                       "ms_per_step": row["ms_per_step"], "elem_per_s": row["elem_per_s"],
                       "bytes_per_elem": row["alg_bytes_per_step"] / row["n"],
                       "frac": row["step_frac"]}
        torch.cuda.empty_cache()
        row = stress_row()
        detail["stress_1e9"] = row
        out["cfg5"] = {"what": "1e9 fp32, 5 % duplicated magnitudes: select_topk_flat alone "
                               "(5 B/elem) at 0.01 % | 1 %, then the fused two-sweep step at 1 %",
                       "select_ms": [row["select_only"]["0.01"]["ms"], row["select_only"]["1.0"]["ms"]],
                       "select_frac": [row["select_only"]["0.01"]["frac"],
                                       row["select_only"]["1.0"]["frac"]],
                       "step_ms": row["fused_step"]["ms_per_step"],
                       "step_frac": row["fused_step"]["step_frac"]}
        torch.cuda.empty_cache()
    if not args.no_replay:
        draws = replay_bench([("seed 4", replay_draw()), ("stress", REPLAY_STRESS_DRAW)])
        rp = draws[0]
        detail["replay"] = rp
        detail["replay_stress_draw"] = draws[1]
        out["replay"] = {"value": rp["value"], "unit": rp["unit"],
                         "ms_per_window": rp["ms_per_window"], "G": rp["G"], "W": rp["W"],
                         "alg_bytes": rp["alg_bytes"], "frac": rp["frac"],
                         "roofline": {"kernel": "k_replay_pass3", "avg_ms": rp["roofline"]["avg_ms"],
                                      "frac": rp["roofline"]["frac"]},
                         "stress_draw": {"value": draws[1]["value"], "frac": draws[1]["frac"]}}
        torch.cuda.empty_cache()
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(args.cpu_sample, 3, args.ratio, args.score)
        if "replay" in out:
            cb = replay_cpu_baseline()
            detail["replay"]["cpu_baseline"] = cb
            out["replay"]["cpu_baseline"] = {"value": cb["value"], "unit": cb["unit"],
                                             "cores": cb["cores"], "kind": cb["kind"]}
    else:
        out["cpu_baseline"] = None
    if args.detail:
        try:
            os.makedirs(os.path.dirname(args.detail) or ".", exist_ok=True)
            with open(args.detail, "w") as f:
                json.dump(dict(out, detail=detail), f, indent=1)
            out["detail_file"] = os.path.relpath(args.detail, ROOT)
        except OSError as e:
            out["detail_file"] = f"not written ({e.strerror})"
    # the last line stays compact whatever happens: optional summaries go first if it ever grew
    line = json.dumps(out, separators=(",", ":"))
    for key in ("cfg5", "cfg2", "single_buffer", "out_of_place", "in_place", "packed_layout", "separate_layout",
                "two_sweep"):
        if len(line) < 6000:
            break
        out.pop(key, None)
        line = json.dumps(out, separators=(",", ":"))
    print(line)


if __name__ == "__main__":
    main()
