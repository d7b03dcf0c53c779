"""Writes a small synthetic trace directory in the reference writer's layout
(catalog + branch state + per-step gradient dumps)."""
import torch

from sga_amd import trace_io as T

SIZES = [("embed.weight", (300, 40)), ("layers.0.w", (257, 33)), ("layers.0.b", (33,)),
         ("layers.1.w", (128, 65)), ("norm.weight", (7,))]


def make_trace(tmp, steps=6, t0=10, g_dtype=None, seed=2026, clip=0.3, absent=(2, 3),
               with_groups=True):
    gen = torch.Generator().manual_seed(seed)
    groups = [{"adam_beta1": 0.9, "adam_beta2": 0.95, "adam_eps": 1e-8, "weight_decay": 0.1},
              {"adam_beta1": 0.9, "adam_beta2": 0.999, "adam_eps": 1e-8, "weight_decay": 0.0}]
    cat = {}
    for name, shape in SIZES:
        cat[name] = {"shape": list(shape), "dtype": "torch.float32"}
        if with_groups:
            cat[name]["param_group"] = 0 if len(shape) > 1 else 1

    def meta(step, norm):
        m = {"step": step, "phase": "shadow", "lr": [5e-5, 2e-5], "grad_norm": norm,
             "clip_grad": clip, "weight_decay": 0.1, "adam_beta1": 0.9, "adam_beta2": 0.95,
             "adam_eps": 1e-8}
        if with_groups:
            m["param_groups"] = groups
        return m

    T.write_catalog(tmp, cat, meta(t0, float("nan")),
                    "bf16" if g_dtype is torch.bfloat16 else "fp32")
    w = {n: torch.randn(s, generator=gen) * 0.02 for n, s in SIZES}
    m = {n: torch.randn(s, generator=gen) * 1e-3 for n, s in SIZES}
    v = {n: torch.rand(s, generator=gen) * 1e-6 for n, s in SIZES}
    g0 = {n: torch.randn(s, generator=gen) * 1e-2 for n, s in SIZES}
    T.write_state(tmp, t0, meta(t0, 0.2), w, m, v, g0)
    for si in range(steps):
        grads = {n: torch.randn(s, generator=gen) * 1e-2 for n, s in SIZES}
        if si in absent:
            del grads["layers.0.b"]
        norm = float(torch.sqrt(sum((t.double() ** 2).sum() for t in grads.values())))
        # recorded gradients are post-clip
        coef = min(1.0, clip / (norm + 1e-6)) if clip > 0 else 1.0
        grads = {n: t * coef for n, t in grads.items()}
        T.write_grad(tmp, t0 + si, meta(t0 + si, norm), grads, g_dtype)
    return cat
