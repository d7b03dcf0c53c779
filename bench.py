#!/usr/bin/env python3
"""Benchmark of the fused per-rank sparse step on one MI355X.

One "step" = score |g+r| -> exact top-k (1 %, lowest-index ties) -> index pack
(int32 idx + bf16 values) -> residual update -> residual-aware AdamW over the
Llama-3.2-1B-shaped gradient set (1,235,814,400 elements, 146 tensors, bf16
Student-t(3) gradients, fp32 p/m/v/residual) with every input resident in HBM.

The step is timed on both state layouts: the library-owned packed layout
(resid/p/m/v interleaved in 64 KiB records -- the headline) and the drop-in
one (four flat tensors, as the reference's buffers are); both run the same
arithmetic and produce the same bits.

Prints ONE JSON line: whole-job elements/s, the roofline of the dominant
kernel (the final sweep, timed live with HIP events on its launch stream),
both layouts under "layouts", the fused replay leg and the CPU oracle timed on
a bounded sample of the same workload.
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
ALG_BYTES_STEP = 40.0      # 2*(2+4) + 4 + 24  (bf16 g, two-buffer contract)
ALG_BYTES_FINAL = 34.0     # final sweep: read g,r,p,m,v (18) + write r,p,m,v (16)


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


def cpu_baseline(sample_n, steps, ratio):
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
    OF.fused_sparse_step(grads[0], r, p, m, v, segs, 1, ratio_percent=ratio,
                         values_dtype=torch.bfloat16)             # warm-up step
    t0 = time.perf_counter()
    for s in range(steps):
        OF.fused_sparse_step(grads[s], r, p, m, v, segs, s + 2, ratio_percent=ratio,
                             values_dtype=torch.bfloat16)
    dt = time.perf_counter() - t0
    return {"value": n * steps / dt, "unit": "elem/s", "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": f"{len(shapes)} layer tensors of the Llama-3.2-1B list "
                      f"({n} elements), {steps} steps at {ratio}% after 1 warm-up step, "
                      f"{dt:.1f} s; host cpu_count={os.cpu_count()}"}


def replay_bench(G=8, W=32, seed=4):
    """Fused offline replay on the Qwen3-0.6B shapes: a window of W recorded
    bf16 gradient steps resident in HBM, G configs drawn with a fixed seed from
    score x ratio x cycle length; per-config fp32 w/m/v/residual + byte mask."""
    import random
    import torch
    from sga_amd import _lib as L
    from sga_amd.replay import select_topk_flat
    from sga_amd.replay_group import Config, ReplayGroup
    from sga_amd.shapes import qwen3_06b, segments_for
    dev = torch.device("cuda:0")
    segs, n = segments_for(qwen3_06b())
    entries = [{"a": s["start"], "n": s["n"], "b1": s["b1"], "b2": s["b2"], "eps": s["eps"],
                "wd": s["wd"]} for s in segs]
    rnd = random.Random(seed)
    axes = [(sc, r, t) for sc in ("abs_g", "update", "coi") for r in (0.1, 1.0, 10.0)
            for t in (1, 4, 16)]
    picks = rnd.sample(axes, G)
    cfgs = [Config(*p) for p in picks]
    gen = torch.Generator(device=dev).manual_seed(1)
    w0 = torch.randn(n, generator=gen, device=dev) * 0.02
    m0 = torch.randn(n, generator=gen, device=dev) * 1e-4
    v0 = torch.rand(n, generator=gen, device=dev) * 1e-8
    # slowly drifting per-tensor scale: one scale vector per step applied on the fly
    window = []
    for s in range(W):
        g = student_t_dev(n, 500 + s, dev, scale=1e-3 * (1.0 + 0.02 * s))
        window.append(g)
    sel0 = []
    base = window[0].float().abs()
    for c in cfgs:                       # branch selection on |g0| (cheap stand-in for the front block)
        sel0.append(select_topk_flat(base, max(1, int(round(c.ratio / 100.0 * n))))[0])
    del base
    grp = ReplayGroup(entries, w0, m0, v0, sel0, cfgs, t0=100, window=W)
    del sel0
    meta = {"clip_grad": 1.0, "grad_norm": float("nan"), "lr": 1e-4}
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for s in range(W):
        grp.step(window[s], meta)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    # algorithmic bytes of this calendar (bf16 g read once per pass for the group)
    alg = 0.0
    n_resel = 0
    for s in range(W):
        alg += 2 * 2.0 * n                                   # g in pass 1 and pass 3
        for c in cfgs:
            bnd = s % c.T == 0
            rz = s == 0 or (s - 1) % c.T == 0                # res is all zeros: no traffic for it
            alg += ((0.0 if rz else 4.0) if bnd else 0.125) * n  # pass 1: res | sel (1 bit)
            # pass 3: m, v, w read+write; res read unless zero, written unless it stays zero
            alg += (24.0 + (0.0 if rz else 4.0) + (0.0 if (bnd and rz) else 4.0)
                    + (0.0 if bnd else 0.125)) * n
            if bnd and s > 0 and s + 1 < W:
                per = (6.0 if c.score == "abs_g" else 18.0) - (4.0 if rz else 0.0)
                alg += (per + 0.125) * n                     # one score sweep + the new mask bits
                n_resel += 1
    return {"metric": "replay config-steps/s", "value": G * W / dt, "unit": "config-steps/s",
            "ms_per_window": dt * 1e3, "G": G, "W": W, "n": n, "reselects": n_resel,
            "configs": [list(p) for p in picks],
            "alg_bytes": alg, "achieved_GBps": alg / dt / 1e9, "frac": alg / dt / HBM_PEAK,
            "workload": "Qwen3-0.6B shapes (596,049,920 elems, 310 tensors), bf16 Student-t(3) "
                        "window, per-config fp32 w/m/v/res + u8 mask resident, clip 1.0"}


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
    rnd = random.Random(seed)
    axes = [(sc, r, t) for sc in ("abs_g", "update", "coi") for r in (0.1, 1.0, 10.0)
            for t in (1, 4, 16)]
    cfgs = [OR.Config(*p) for p in rnd.sample(axes, G)]
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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--ratio", type=float, default=1.0)
    ap.add_argument("--score", default="abs_g")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-sample", type=int, default=1 << 29)
    ap.add_argument("--calib", action="store_true",
                    help="also launch one plain copy of 2^30 fp32 (k_calib_copy) so counter "
                         "runs can be scaled against a kernel of known traffic")
    ap.add_argument("--no-replay", action="store_true", help="skip the fused replay leg")
    ap.add_argument("--layout", choices=("both", "packed", "separate"), default="both",
                    help="state layout(s) to time; the headline is the packed layout unless "
                         "only the separate one runs")
    ap.add_argument("--trace-io", action="store_true",
                    help="run just the recorded-trace leg (writes a temporary trace, streams it "
                         "back through the pread reader and the dense pass) and print its JSON")
    ap.add_argument("--primitives", action="store_true",
                    help="time the drop-in primitives on their own and print their JSON")
    ap.add_argument("--only-replay", action="store_true",
                    help="run just the fused replay leg (for profiling) and print its JSON")
    ap.add_argument("--sweep", action="store_true",
                    help="also time ratios 0.1/1/10 % and the update score")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs one data-parallel rank's share on ONE GPU; "
              "there are no collectives, so --gpus must be 1", file=sys.stderr)
        sys.exit(2)

    import torch
    from sga_amd import _lib as L
    from sga_amd.fused_step import FusedSparseStep, k_for
    from sga_amd.shapes import llama32_1b, segments_for

    L.load()
    if args.only_replay:
        torch.cuda.set_device(0)
        print(json.dumps(replay_bench()))
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

    calib = None
    if args.calib:
        cn = 1 << 30
        src = torch.ones(cn, device=dev)
        dst = torch.empty(cn, device=dev)
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
        L.call("sga_calib_copy", L.ptr(dst), L.ptr(src), cn, L.stream())
        ev[0].record()
        for _ in range(5):
            L.call("sga_calib_copy", L.ptr(dst), L.ptr(src), cn, L.stream())
        ev[1].record()
        torch.cuda.synchronize()
        ms = ev[0].elapsed_time(ev[1]) / 5
        calib = {"kernel": "k_calib_copy", "bytes": cn * 8, "avg_ms": ms,
                 "GBps": cn * 8 / ms / 1e6}
        del src, dst
        # the final sweep's own mix of streams without its math, on scratch arrays
        sg = torch.zeros(n, dtype=torch.bfloat16, device=dev)
        sc = [torch.zeros(n, device=dev) for _ in range(4)]
        sargs = [L.ptr(sg)] + [L.ptr(t) for t in sc] + [n, L.stream()]
        L.call("sga_calib_streams", *sargs)
        ev[0].record()
        for _ in range(5):
            L.call("sga_calib_streams", *sargs)
        ev[1].record()
        torch.cuda.synchronize()
        ms = ev[0].elapsed_time(ev[1]) / 5
        calib["streams"] = {"kernel": "k_calib_streams", "bytes": n * 34, "avg_ms": ms,
                            "GBps": n * 34 / ms / 1e6}
        del sg, sc
    k = k_for(n, args.ratio)
    final_bytes = n * ALG_BYTES_FINAL + k * 6.0

    def time_leg(step_fn, step0):
        """W warm-up + K timed steps of one layout; returns (seconds, final-sweep ms)."""
        for s in range(args.warmup):
            step_fn(step0 + s)
        torch.cuda.synchronize()
        L.raw("sga_prof_enable", 1)
        t0 = time.perf_counter()
        for s in range(args.steps):
            step_fn(step0 + args.warmup + s)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        tot_ms, cnt = ctypes.c_double(0), ctypes.c_int(0)
        L.call("sga_prof_read", ctypes.byref(tot_ms), ctypes.byref(cnt))
        L.raw("sga_prof_enable", 0)
        res = fs.read_result()
        assert res.status == 0 and res.n_selected == k, vars(res)
        return dt, tot_ms.value / max(cnt.value, 1), res

    def leg_summary(dt, final_ms):
        return {"value": n * args.steps / dt, "ms_per_step": dt / args.steps * 1e3,
                "step_frac": n * args.steps / dt * ALG_BYTES_STEP / HBM_PEAK,
                "final_avg_ms": final_ms,
                "final_frac": final_bytes / (final_ms * 1e-3) / HBM_PEAK}

    legs, step0 = {}, 0
    if args.layout in ("separate", "both"):
        # the drop-in entry point: resid / p / m / v are the caller's four flat tensors
        dt_s, ms_s, res = time_leg(
            lambda t: fs.step(grads[t % 2], r, p, m, v, t + 1, k=k, score=args.score), step0)
        legs["separate"] = (dt_s, ms_s)
        step0 += args.warmup + args.steps
    if args.layout in ("packed", "both"):
        # the library-owned state layout: the same four arrays interleaved in 64 KiB
        # records; identical arithmetic and outputs (asserted bitwise by the tests)
        from sga_amd.fused_step import PackedState
        st = PackedState(n, dev).pack(r, p, m, v)
        dt_p, ms_p, res = time_leg(
            lambda t: fs.step_packed(grads[t % 2], st, t + 1, k=k, score=args.score), step0)
        legs["packed"] = (dt_p, ms_p)
        step0 += args.warmup + args.steps
    head = "packed" if "packed" in legs else "separate"
    dt, final_ms = legs[head]
    achieved = final_bytes / (final_ms * 1e-3) if final_ms > 0 else 0.0
    traffic = None
    tpath = os.path.join(ROOT, "profiles", "fused_final_llama1b_traffic.json")
    if os.path.exists(tpath):
        try:
            traffic = json.load(open(tpath)).get("hbm_bytes_per_launch")
        except Exception:
            traffic = None
    value = n * args.steps / dt
    layout_txt = ("resid/p/m/v interleaved in 64 KiB records (sga_fused_sparse_step_packed)"
                  if head == "packed" else
                  "resid/p/m/v as four flat tensors (sga_fused_sparse_step)")
    out = {
        "metric": "grad elems/s (score+top-k+resid AdamW)",
        "value": value, "unit": "elem/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": dt / args.steps * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "Llama-3.2-1B-shaped set, 1,235,814,400 elems / 146 tensors, "
                               "bf16 Student-t(3) grads, fp32 p/m/v/residual, score "
                               f"{args.score}, exact top-k {args.ratio}% (k={k}), index pack "
                               "int32+bf16, residual-aware AdamW; state layout: " + layout_txt,
                   "ratio_percent": args.ratio, "score": args.score, "k": k,
                   "state_layout": head},
        "roofline": {"bound": "hbm", "achieved": achieved / 1e9, "peak": HBM_PEAK / 1e9,
                     "unit": "GB/s", "frac": achieved / HBM_PEAK, "traffic": traffic,
                     "kernel": "k_fused_final", "avg_ms": final_ms,
                     "alg_bytes_per_launch": final_bytes},
        "step_roofline": {"alg_bytes_per_elem": ALG_BYTES_STEP,
                          "achieved_GBps": value * ALG_BYTES_STEP / 1e9,
                          "frac": value * ALG_BYTES_STEP / HBM_PEAK},
        "select": {"thresh": res.thresh, "n_gt": res.n_gt, "n_eq": res.n_eq, "path": res.path},
        "layouts": {name: leg_summary(*v) for name, v in legs.items()},
    }
    if calib:
        out["copy_calibration"] = calib
    if args.sweep:
        sw = []
        def run(steps, t0_, ratio, score):          # on the headline layout
            kk = k_for(n, ratio)
            for t in range(t0_, t0_ + steps):
                if head == "packed":
                    fs.step_packed(grads[t % 2], st, t + 1, k=kk, score=score)
                else:
                    fs.step(grads[t % 2], r, p, m, v, t + 1, k=kk, score=score)
        for score, ratio in (("abs_g", 0.1), ("abs_g", 10.0), ("update", 0.1),
                             ("update", 1.0), ("update", 10.0)):
            run(1, step0, ratio, score)
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            run(3, step0 + 1, ratio, score)
            torch.cuda.synchronize()
            d = (time.perf_counter() - t1) / 3
            step0 += 4
            sw.append({"score": score, "ratio_percent": ratio, "elem_per_s": n / d,
                       "ms_per_step": d * 1e3})
        out["sweep"] = sw
    if head == "packed":
        st.unpack(r, p, m, v)
        del st
    if not args.no_replay:
        del p, m, v, r, grads, fs
        torch.cuda.empty_cache()
        out["replay"] = replay_bench()
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(args.cpu_sample, 3, args.ratio)
        if "replay" in out:
            out["replay"]["cpu_baseline"] = replay_cpu_baseline()
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))


if __name__ == "__main__":
    main()
