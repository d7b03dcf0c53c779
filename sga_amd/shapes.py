"""Parameter-set shapes of the benchmark configurations (tensor name, numel),
in catalog order.  Shapes come from the model families the reference's
examples train (``examples/llama3``, ``examples/qwen3``)."""


def llama32_1b():
    """Llama-3.2-1B: 146 tensors, 1,235,814,400 elements."""
    out = [("embed", 128256 * 2048)]
    for i in range(16):
        out += [(f"l{i}.in_norm", 2048), (f"l{i}.q", 2048 * 2048), (f"l{i}.k", 512 * 2048),
                (f"l{i}.v", 512 * 2048), (f"l{i}.o", 2048 * 2048),
                (f"l{i}.post_norm", 2048), (f"l{i}.gate", 8192 * 2048),
                (f"l{i}.up", 8192 * 2048), (f"l{i}.down", 2048 * 8192)]
    out.append(("final_norm", 2048))
    return out


def qwen3_06b():
    """Qwen3-0.6B: 310 tensors, 596,049,920 elements."""
    out = [("embed", 151936 * 1024)]
    for i in range(28):
        out += [(f"l{i}.in_norm", 1024), (f"l{i}.q", 2048 * 1024), (f"l{i}.k", 1024 * 1024),
                (f"l{i}.v", 1024 * 1024), (f"l{i}.q_norm", 128), (f"l{i}.k_norm", 128),
                (f"l{i}.o", 1024 * 2048), (f"l{i}.post_norm", 1024),
                (f"l{i}.gate", 3072 * 1024), (f"l{i}.up", 3072 * 1024),
                (f"l{i}.down", 1024 * 3072)]
    out.append(("final_norm", 1024))
    return out


def segments_for(shapes, lr=1e-4, b1=0.9, b2=0.95, eps=1e-8, wd=0.1):
    """One segment per tensor; norm gains (1-D tensors) take no weight decay,
    as in the trainer's param groups."""
    segs, off = [], 0
    for name, n in shapes:
        segs.append(dict(name=name, start=off, n=n, lr=lr, b1=b1, b2=b2, eps=eps,
                         wd=0.0 if "norm" in name else wd))
        off += n
    return segs, off
