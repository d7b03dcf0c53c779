"""ctypes binding of libsga_hip.so (the C ABI declared in include/sga_hip.h).

There is no CPU fallback anywhere in this package: if the shared library is
missing, or a tensor is not on a HIP device, the call raises.
"""
import ctypes as C
import os
import struct

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libsga_hip.so")

SGA_F32, SGA_BF16 = 0, 1
TIE_ALL, TIE_LOWEST_INDEX = 0, 1
GC_HAS_MASK, GC_APPLY_COEFF, GC_CLEAR, GC_FOLD, GC_LR_SPLIT, GC_ADAMS = 1, 2, 4, 8, 16, 32
RP_HAS_LAB, RP_ADAMS, RP_SPLIT = 1, 2, 4

P, I64, I32, F, SZ = C.c_void_p, C.c_int64, C.c_int, C.c_float, C.c_size_t
U32 = C.c_uint32


class Segment(C.Structure):
    """struct sga_segment"""
    _fields_ = [("start", C.c_int64), ("n", C.c_int64), ("lr", C.c_float),
                ("beta1", C.c_float), ("om1", C.c_float), ("beta2", C.c_float),
                ("om2", C.c_float), ("eps", C.c_float), ("wd", C.c_float),
                ("bc1", C.c_float), ("bc2", C.c_float), ("pad_", C.c_float)]


class FusedBucket(C.Structure):
    """struct sga_fused_bucket"""
    _fields_ = [("g", C.c_void_p), ("resid", C.c_void_p), ("p", C.c_void_p), ("m", C.c_void_p),
                ("v", C.c_void_p), ("n", C.c_int64), ("k", C.c_int64), ("segs", C.c_void_p),
                ("n_segs", C.c_int), ("pad_", C.c_int), ("idx_out", C.c_void_p),
                ("values_out", C.c_void_p), ("mask_out", C.c_void_p), ("result", C.c_void_p),
                ("ws", C.c_void_p), ("ws_bytes", C.c_size_t)]


class ReselectJob(C.Structure):
    """struct sga_reselect_job"""
    _fields_ = [("res", C.c_void_p), ("w", C.c_void_p), ("m", C.c_void_p), ("v", C.c_void_p),
                ("k", C.c_int64), ("score_id", C.c_int), ("adams", C.c_int),
                ("res_zero", C.c_int), ("pad_", C.c_int), ("coef_f", C.c_void_p),
                ("sel_out", C.c_void_p), ("result", C.c_void_p), ("ws", C.c_void_p),
                ("ws_bytes", C.c_size_t)]


# name -> (restype, argtypes); must list every symbol of include/sga_hip.h
SIGNATURES = {
    "sga_version": (I32, []),
    "sga_last_error": (C.c_char_p, []),
    "sga_scatter_selected": (I32, [P, P, P, I64, I64, P]),
    "sga_pack_selected": (I32, [P, P, P, I32, F, I64, I64, P]),
    "sga_norm_partials": (I64, [I64]),
    "sga_compact_norm_sq": (I32, [P, I64, P, P, P]),
    "sga_compact_norm_sq_noalloc": (I32, [P, I64, P, P]),
    "sga_masked_norm_sq": (I32, [P, P, I64, P, P, P]),
    "sga_gather_selected_blocks": (I32, [P, P, P, P, I64, I32, F, I64, P]),
    "sga_scatter_selected_blocks": (I32, [P, P, P, P, I64, I32, I64, P]),
    "sga_block_reduce": (I32, [P, I64, I32, I32, P, P]),
    "sga_block_any": (I32, [P, I64, I32, P, P]),
    "sga_expand_blocks": (I32, [P, I32, I64, P, P]),
    "sga_mask_chunks": (I64, [I64]),
    "sga_mask_count": (I32, [P, I64, P, P, P]),
    "sga_mask_fill": (I32, [P, I64, P, P, I64, P]),
    "sga_adamw_grad_correct": (I32, [P, P, P, P, P, I64] + [F] * 12 + [I32, I32, P]),
    "sga_adamw_grad_correct_multi": (I32, [P, I32, I64, F, F, I32, P]),
    "sga_adamw_grad_correct_compact_multi": (I32, [P, I32, I64, I32, F, F, P]),
    "sga_adamw_grad_correct_compact": (I32, [P, P, P, P, P, P, I32, I64, I64, I64]
                                       + [F] * 11 + [I32, P, I64, P]),
    "sga_build_dir_table": (I32, [P, I64, P, I64, P]),
    "sga_select_workspace_bytes": (SZ, [I64]),
    "sga_select_topk": (I32, [P, I64, I64, I32, P, P, P, SZ, P]),
    "sga_sel_begin": (I32, [I64, P, SZ, P]),
    "sga_sel_hist": (I32, [P, I64, I32, P, SZ, P]),
    "sga_sel_scan": (I32, [I32, P, SZ, P]),
    "sga_sel_count": (I32, [P, I64, I64, P, SZ, P]),
    "sga_sel_tile_scan": (I32, [I64, I32, P, SZ, P]),
    "sga_sel_mask": (I32, [P, I64, I64, I32, P, P, SZ, P]),
    "sga_sel_result": (I32, [P, P, SZ, P]),
    "sga_hist_topbits": (I32, [P, I64, I32, I32, I32, P, I32, P, P]),
    "sga_mask_topbits_ge": (I32, [P, I64, I32, I32, P, P]),
    "sga_scale_masked": (I32, [P, P, I64, F, P]),
    "sga_mask_abs_ge": (I32, [P, I64, F, P, P, P]),
    "sga_cand_extract_count": (I32, [P, I64, I32, P, P, P]),
    "sga_cand_extract_fill": (I32, [P, I64, I32, P, P, I64, P]),
    "sga_gt_eq": (I32, [P, I64, F, P, P, P, P]),
    "sga_score_formula": (I32, [I32, P, P, P, P, P, I64] + [F] * 8 + [I32, I32, P]),
    "sga_opt_step_inplace": (I32, [P, P, P, P, P, P, I64] + [F] * 13 + [I32, P]),
    "sga_replay_partials": (I64, []),
    "sga_replay_pass1": (I32, [P, I32, I64, F, C.c_double, P, I32, P, P, P, P, P]),
    "sga_replay_reselect": (I32, [P, I32, P, P, P, P, I64, I64, P, I32, I32, P, F, I32, I32, I32,
                                  P, P, P, SZ, P]),
    "sga_replay_reselect_multi": (I32, [P, I32, I64, P, I32, F, I32, P, I32, P]),
    "sga_balanced_hist_words": (I64, []),
    "sga_replay_reselect_balanced": (I32, [P, I32, P, P, P, P, I64, I64, P, I32, P, I32, P, F, I32,
                                           I32, I32, P, P, P, P, SZ, P]),
    "sga_replay_pass3": (I32, [P, I32, I64, F, P, I32, P, P, I32, P]),
    "sga_branch_score_f64": (I32, [I32, P, P, P, P, P, I64] + [C.c_double] * 6 + [I32, I32, P]),
    "sga_dense_replay_step": (I32, [P, I32, P, P, P, P, I64, P, I32, I32, C.c_double, P, P, P]),
    "sga_plane_words": (I64, [I64]),
    "sga_mask_to_planes": (I32, [P, I64, P, P]),
    "sga_planes_to_mask": (I32, [P, I64, P, P]),
    "sga_div_inplace": (I32, [P, I64, F, I32, P]),
    "sga_sq_dist": (I32, [P, I32, P, I64, P, P, P]),
    "sga_fused_workspace_bytes": (SZ, [I64]),
    "sga_fused_sparse_step": (I32, [P, I32, P, P, P, P, I64, I64, P, I32, I32, P, P,
                                    I32, P, F, F, I32, I32, F, P, P, SZ, P]),
    "sga_fused_sparse_step_multi": (I32, [P, I32, I32, I32, I32, F, F, I32, I32, F, P]),
    "sga_packed_state_elems": (I64, [I64]),
    "sga_fused_sparse_step_packed": (I32, [P, I32, P, I64, I64, P, I32, I32, P, P,
                                           I32, P, F, F, I32, I32, F, P, P, SZ, P]),
    "sga_state_repack": (I32, [P, P, P, P, P, I64, I32, P]),
    "sga_fused_single_sweep_workspace_bytes": (SZ, [I64, I32]),
    "sga_fused_sparse_step_single_sweep": (I32, [P, I32, P, P, P, P, I64, I64, P, I32, I32, P, P,
                                                 I32, P, F, F, I32, F, U32, P, P, SZ, P, SZ, P]),
    "sga_fused_sparse_step_single_sweep_packed": (I32, [P, I32, P, I64, I64, P, I32, I32, P, P,
                                                        I32, P, F, F, I32, F, U32, P, P, SZ, P,
                                                        SZ, P]),
    "sga_fused_sparse_step_single_sweep_out": (I32, [P, I32, P, P, P, P, P, P, P, P, I64, I64, P, I32,
                                                     I32, P, P, I32, P, F, F, I32, F, U32, P, P, SZ,
                                                     P, SZ, P]),
    "sga_fused_sparse_step_single_sweep_packed_out": (I32, [P, I32, P, P, I64, I64, P, I32, I32, P, P,
                                                            I32, P, F, F, I32, F, U32, P, P, SZ, P,
                                                            SZ, P]),
}

# include/sga_hip_bench.h: libsga_hip_bench.so, the benchmark-only companion
BENCH_SIGNATURES = {
    "sga_calib_copy": (I32, [P, P, I64, P]),
    "sga_calib_streams": (I32, [P, P, P, P, P, I64, P]),
    "sga_prof_enable": (I32, [I32]),
    "sga_prof_read": (I32, [I32, P, P]),
    "sga_bench_prof_begin": (P, [I32, P]),
    "sga_bench_prof_end": (None, [P, P]),
    "sga_bench_last_error": (C.c_char_p, []),
}
BENCH_LIB_PATH = os.path.join(_HERE, "libsga_hip_bench.so")

_lib = None
_bench = None


def load_bench():
    """Load the benchmark companion (timing observer + calibration kernels).
    libsga_hip.so binds its two weak observer references when it is loaded,
    so this has to come first and into the global symbol scope."""
    global _bench
    if _bench is not None:
        return _bench
    if _lib is not None:
        raise RuntimeError("load_bench() must run before the first use of libsga_hip.so")
    if not os.path.exists(BENCH_LIB_PATH):
        raise RuntimeError(f"{BENCH_LIB_PATH} is missing (run `python -m sga_amd.build`)")
    lib = C.CDLL(BENCH_LIB_PATH, mode=C.RTLD_GLOBAL)
    for name, (res, args) in BENCH_SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _bench = lib
    return lib


def bench_call(name, *args):
    lib = load_bench()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        raise RuntimeError(f"{name} failed ({rc}): "
                           f"{lib.sga_bench_last_error().decode(errors='replace')}")


def load():
    """Load the shared library once; raise loudly when it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: the HIP extension is not built "
            "(run `python -m sga_amd.build`). sga_amd has no CPU fallback.")
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def call(name, *args):
    """Invoke an int-returning entry point; raise with the library's text."""
    lib = load()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        raise RuntimeError(f"{name} failed ({rc}): "
                           f"{lib.sga_last_error().decode(errors='replace')}")


def raw(name, *args):
    return getattr(load(), name)(*args)


def f32(x):
    """Round a Python float to fp32 (nearest-even), back as a Python float."""
    return struct.unpack("f", struct.pack("f", float(x)))[0]


def require_dev(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError(
                "sga_amd operates on HIP device tensors only (got a "
                f"{t.device} tensor); there is no CPU fallback")


def require_contig(**named):
    for name, t in named.items():
        if t is not None and not t.is_contiguous():
            raise ValueError(f"sga_amd requires contiguous tensors ({name} is not)")


def ptr(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def dtype_code(t):
    if t.dtype == torch.float32:
        return SGA_F32
    if t.dtype == torch.bfloat16:
        return SGA_BF16
    raise TypeError(f"unsupported dtype {t.dtype} (fp32 or bf16)")


class TableUploader:
    """Ships small per-step parameter tables (ctypes struct arrays) to one
    device buffer without stalling the host: the bytes go through a ring of
    pinned staging buffers and an asynchronous copy on the current stream, so
    the copy is ordered after the kernels that still read the previous table
    and before the ones launched next."""

    def __init__(self, nbytes, device, slots=4):
        import torch
        self.nbytes = int(nbytes)
        self.dev = torch.empty(self.nbytes, dtype=torch.uint8, device=device)
        self._host = [torch.empty(self.nbytes, dtype=torch.uint8, pin_memory=True)
                      for _ in range(slots)]
        self._done = [None] * slots
        self._i = 0

    def upload(self, struct_array):
        import torch
        if C.sizeof(struct_array) != self.nbytes:
            raise ValueError("table size changed")
        slot = self._i % len(self._host)
        self._i += 1
        if self._done[slot] is not None:
            self._done[slot].synchronize()
        C.memmove(self._host[slot].data_ptr(), C.addressof(struct_array), self.nbytes)
        self.dev.copy_(self._host[slot], non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        self._done[slot] = ev
        return self.dev
