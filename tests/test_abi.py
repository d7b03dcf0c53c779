"""CPU-side checks of the boundary: the shared library loads, exports every
symbol declared in include/sga_hip.h, the Python table lists the same set,
and the product refuses CPU tensors (no fallback)."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared(header):
    txt = open(os.path.join(ROOT, "include", header)).read()
    txt = re.sub(r"/\*.*?\*/", "", txt, flags=re.S)
    return sorted(set(re.findall(r"\b(sga_[a-z0-9_]+)\s*\(", txt)))


def _exported(path):
    """The C symbols (``sga_*``) a shared library defines and exports."""
    import subprocess
    out = subprocess.run(["nm", "-D", "--defined-only", path], check=True, capture_output=True,
                         text=True).stdout
    return sorted(l.split()[-1] for l in out.splitlines()
                  if l.split() and l.split()[-1].startswith("sga_"))


def test_library_exports_exactly_the_declared_symbols():
    """libsga_hip.so exports the entry points of include/sga_hip.h and no other
    C symbol (no timing or calibration hook); the ctypes table lists the same set."""
    from sga_amd import _lib as L
    assert os.path.exists(L.LIB_PATH), "run python -m sga_amd.build"
    names = _declared("sga_hip.h")
    assert len(names) >= 30
    assert _exported(L.LIB_PATH) == names
    assert sorted(L.SIGNATURES) == names
    assert L.load().sga_version() >= 1


def test_bench_companion_exports_its_header():
    from sga_amd import _lib as L
    assert os.path.exists(L.BENCH_LIB_PATH), "run python -m sga_amd.build"
    names = _declared("sga_hip_bench.h")
    assert _exported(L.BENCH_LIB_PATH) == names
    assert sorted(L.BENCH_SIGNATURES) == names


def test_struct_layouts_match_header():
    from sga_amd import _lib as L
    from sga_amd.selection import SelectResult
    assert ctypes.sizeof(L.Segment) == 56
    assert ctypes.sizeof(SelectResult) == 32


def test_no_cpu_fallback():
    from sga_amd import adamw, kernels, replay, support
    z = torch.zeros(8)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        kernels.pack_selected(z, torch.zeros(2, dtype=torch.int32), torch.zeros(2), 1.0)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        adamw.adamw_grad_correct(z, z.clone(), z.clone(), z.clone(), 1e-3, .9, .95, 1e-8, 0., 1)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        support.compact_mask_u8(torch.zeros(8, dtype=torch.uint8))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        replay.select_topk_flat(z, 2)


def test_host_refusals_before_launch():
    from sga_amd import adamw
    z = torch.zeros(4)
    mk = torch.ones(4, dtype=torch.uint8)
    for kw, sub in ((dict(coeff=0.5), "requires a sparse step"),
                    (dict(mask=mk, emit_score="update"), "masked-commit full step"),
                    (dict(mask=mk, inactive_lr_scale=0.5), "requires a full step"),
                    (dict(mask=mk, emit_score="update", inactive_lr_scale=float("inf")),
                     "inactive_lr_scale"),
                    (dict(emit_score="bogus"), "no _grad_correct_kernel branch")):
        with pytest.raises(ValueError) as ei:
            adamw.adamw_grad_correct(z, z.clone(), z.clone(), z.clone(), 1e-3, .9, .95,
                                     1e-8, 0., 1, **kw)
        assert sub in str(ei.value)
    from sga_amd.scores import get_score_spec, score_names
    assert score_names() == ["abs_g", "abs_m", "coi", "update"]
    with pytest.raises(ValueError) as ei:
        get_score_spec("nope")
    assert "nope" in str(ei.value) and "abs_g" in str(ei.value)
    from sga_amd.fused_step import k_for
    assert k_for(4194304, 1.0) == 41943 and k_for(250, 1.0) == 2


def test_oracle_is_not_imported_by_the_product():
    pkg = os.path.join(ROOT, "sga_amd")
    for dp, _, fs in os.walk(pkg):
        for f in fs:
            if f.endswith((".py", ".hip", ".hpp")):
                src = open(os.path.join(dp, f)).read()
                assert "oracle" not in src.replace("# oracle", ""), f


def test_header_is_plain_c_and_struct_sizes_agree(tmp_path):
    """include/sga_hip.h compiles as C99 on its own, and the struct sizes a C
    caller sees are the ones the ctypes mirrors use."""
    import subprocess
    from sga_amd import _lib as L
    from sga_amd.adamw import GcRecord, GccRecord
    from sga_amd.replay_group import ReplayCfg, ReplaySegment
    from sga_amd.selection import SelectResult
    src = tmp_path / "sizes.c"
    src.write_text('#include <stdio.h>\n#include "sga_hip.h"\n'
                   'int main(void) { printf("%zu %zu %zu %zu ", sizeof(sga_segment), '
                   'sizeof(sga_select_result), sizeof(sga_replay_cfg), '
                   'sizeof(sga_replay_segment)); printf("%zu %zu\\n", sizeof(sga_gc_record), '
                   'sizeof(sga_gcc_record)); return 0; }\n')
    exe = tmp_path / "sizes"
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-pedantic",
                    "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
    got = [int(x) for x in subprocess.run([str(exe)], check=True, capture_output=True,
                                          text=True).stdout.split()]
    assert got == [ctypes.sizeof(L.Segment), ctypes.sizeof(SelectResult),
                   ctypes.sizeof(ReplayCfg), ctypes.sizeof(ReplaySegment),
                   ctypes.sizeof(GcRecord), ctypes.sizeof(GccRecord)]


def test_result_block_decoding():
    """The eight words of ``sga_select_result``: the path is the low byte of
    the last word, bit 8 says that an fp32 score array held a value below
    zero (what ``sga/replay.py:545-547`` rejects)."""
    import struct
    import torch
    from sga_amd.selection import read_result
    th = struct.unpack("i", struct.pack("f", 0.75))[0]
    r = read_result(torch.tensor([th, 3, 10, 5, 13, 0, 0, 1 | 0x100], dtype=torch.int32))
    assert (r.thresh, r.need, r.n_gt, r.n_eq, r.n_selected) == (0.75, 3, 10, 5, 13)
    assert r.path == 1 and r.negative and r.status == 0 and r.nonfinite == 0
    r = read_result(torch.tensor([th, 3, 10, 5, 13, 2, 3, 2], dtype=torch.int32))
    assert r.path == 2 and not r.negative and r.status == 3 and r.nonfinite == 2


def test_step_counter_helpers():
    """``sga_peek_step`` / ``sga_advance_step`` on the two counter styles of
    ``sga/kernels.py:305-367``: a group counter (int or tensor), and per-param
    state counters that seed the group counter once per wrapper."""
    from types import SimpleNamespace
    from sga_amd.kernels import sga_advance_step, sga_peek_step
    p1, p2 = object(), object()
    w = SimpleNamespace(optimizer=SimpleNamespace(state={}))
    g = {'params': [p1, p2]}
    assert sga_peek_step(w, g) == 1 and 'step' not in g              # nothing anywhere: first commit
    g['step'] = torch.tensor(6)
    assert sga_peek_step(w, g) == 7 and int(g['step']) == 6          # read-only
    assert sga_advance_step(w, g) == 7 and g['step'] == 7 and isinstance(g['step'], int)
    # torch-AdamW style: per-param state['step'], seeded once, shared by every group
    w = SimpleNamespace(optimizer=SimpleNamespace(state={p2: {'step': torch.tensor(41.0)}}))
    ga, gb = {'params': [p1, p2]}, {'params': [p1]}
    assert sga_peek_step(w, ga) == 42 and 'step' not in ga
    assert sga_advance_step(w, ga) == 42 and sga_advance_step(w, ga) == 43
    assert sga_advance_step(w, gb) == 42                              # the wrapper's one seed
    w = SimpleNamespace(optimizer=SimpleNamespace(state={}))
    assert sga_advance_step(w, {'params': [p1]}) == 1                 # fresh moments seed 0


def test_replay_dtype_guards():
    from sga_amd.replay import require_scan_dtypes, resolve_replay_dtype
    assert resolve_replay_dtype("fp32") is torch.float32
    with pytest.raises(ValueError, match="--replay-dtype must be one of"):
        resolve_replay_dtype("bf16")
    with pytest.raises(ValueError, match="--norm-dtype must be one of"):
        require_scan_dtypes("fp32", "half")
    with pytest.raises(ValueError, match="reserved for --self-check"):
        require_scan_dtypes("fp64", "fp32")
    require_scan_dtypes("fp32", "fp32")


def test_plugins_read_the_args_singleton():
    """``SgaAdamW()`` / ``TopkSelection()`` take no arguments and read the
    ``sga_*`` flags from the args singleton (``sga/config/__init__.py:36-51``,
    ``adamw.py:798-799``, ``topk.py:59-60``); unset, they fail loudly."""
    from types import SimpleNamespace
    from sga_amd import config
    from sga_amd.adams import SgaAdamS
    from sga_amd.adamw import SgaAdamW
    from sga_amd.selection import TopkSelection
    config.set_args(None)
    with pytest.raises(RuntimeError, match="sga args not set"):
        SgaAdamW()
    config.set_args(SimpleNamespace(sga_score="coi", sga_optimizer_residual_mean=True,
                                    sga_optimizer_compact_search="bisection",
                                    sga_optimizer_full_sync_inactive_lr_scale=0.25,
                                    sga_selection_method="histogram",
                                    sga_selection_ratio_percent=2.5,
                                    sga_selection_histogram_mode="balanced"))
    for cls in (SgaAdamW, SgaAdamS):
        o = cls()
        assert (o.residual_mean, o.compact_search, o.full_sync_inactive_lr_scale, o.emit_score) == (
            True, "bisection", 0.25, "coi")
    s = TopkSelection()
    assert s.method == "histogram" and s.ratio_percent == 2.5 and s.k_for(1000) == 25
    config.set_args(SimpleNamespace(sga_score="nope"))
    with pytest.raises(ValueError, match="no EMIT_MODE branch"):
        SgaAdamW()
