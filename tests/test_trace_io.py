"""Trace index / pread reader against torch.load on files in the writer's
layout (no GPU)."""
import os
import pickle

import pytest
import torch

from oracle import trace as OT
from sga_amd import trace_io as T
from trace_fixture import SIZES, make_trace


@pytest.mark.parametrize("g_dtype", [None, torch.bfloat16])
def test_index_matches_torch_load(tmp_path, g_dtype):
    d = str(tmp_path)
    make_trace(d, g_dtype=g_dtype)
    catalog, names, offsets, N, state_files, g_files = T.discover_trace(d)
    assert names == [n for n, _ in SIZES]
    assert N == sum(torch.Size(s).numel() for _, s in SIZES)
    assert offsets["layers.0.w"] == 300 * 40 and sorted(g_files) == list(range(10, 16))
    assert list(state_files) == [10]
    for step, path in g_files.items():
        ref = OT.load_file(path)
        tf = T.TraceFile(path)
        assert tf.meta == ref["meta"]
        assert set(tf.payload) == set(ref["payload"])
        for name, t in ref["payload"].items():
            card = tf.payload[name]
            assert card.dtype == t.dtype and card.shape == tuple(t.shape)
            assert torch.equal(tf.read_tensor(card).view(torch.uint8),
                               t.reshape(-1).view(torch.uint8))
            lo, cnt = 5, min(11, t.numel() - 5)
            assert torch.equal(tf.read_tensor(card, lo, cnt).view(torch.uint8),
                               t.reshape(-1)[lo:lo + cnt].contiguous().view(torch.uint8))
    sref = OT.load_file(state_files[10])
    stf = T.TraceFile(state_files[10])
    for which in ("w", "m", "v", "g"):
        for name, t in sref["payload"][which].items():
            assert torch.equal(stf.read_tensor(stf.payload[which][name]), t.reshape(-1))


def test_window_steps_and_hp(tmp_path):
    d = str(tmp_path)
    make_trace(d)
    catalog, names, _o, N, state_files, g_files = T.discover_trace(d)
    assert T.window_steps_for(g_files, 10, 4) == [10, 11, 12, 13]
    assert T.window_steps_for(g_files, 14, 8) == [14, 15]
    assert T.window_steps_for(g_files, 99, 8) == []
    meta = T.TraceFile(state_files[10]).meta
    assert T.param_hp(meta, catalog["embed.weight"]) == (0.9, 0.95, 1e-8, 0.1, 0)
    assert T.param_hp(meta, catalog["norm.weight"]) == (0.9, 0.999, 1e-8, 0.0, 1)
    legacy = {k: v for k, v in meta.items() if k != "param_groups"}
    assert T.param_hp(legacy, {"shape": [1]}) == (0.9, 0.95, 1e-8, 0.1, None)
    with pytest.raises(ValueError):
        T.param_hp(meta, {"param_group": 7})
    assert T.lr_for_step(meta, 1) == 2e-5 and T.lr_for_step(meta) == (5e-5 + 2e-5) / 2
    # shard slices tile the flat index space like the oracle's
    for lo, hi in [(0, N), (11_000, 21_000), (12_000, 12_001)]:
        sp = T.ShardParams(names, catalog, meta, lo, hi)
        ref = OT.entries_for(catalog, names, {n: catalog[n]["numel"] for n in names}, meta,
                             lo, hi)
        keys = ("name", "p_off", "a", "n", "b1", "b2", "eps", "wd", "group")
        assert [{k: e[k] for k in keys} for e in sp.entries] == \
            [{k: e[k] for k in keys} for e in ref]
        assert sum(e["n"] for e in sp.entries) == hi - lo


@pytest.mark.parametrize("g_dtype", [None, torch.bfloat16])
@pytest.mark.parametrize("span", [None, (11_000, 21_500)])
def test_window_reader_host(tmp_path, g_dtype, span):
    d = str(tmp_path)
    make_trace(d, g_dtype=g_dtype)
    catalog, names, _o, N, state_files, g_files = T.discover_trace(d)
    meta = T.TraceFile(state_files[10]).meta
    lo, hi = span or (0, N)
    sp = T.ShardParams(names, catalog, meta, lo, hi)
    steps = T.window_steps_for(g_files, 10, 6)
    got = list(T.WindowReader(g_files, steps, sp, "cpu", depth=2))
    assert [s for s, _, _ in got] == steps
    for gstep, gmeta, g in got:
        ref = OT.load_file(g_files[gstep])
        assert gmeta == ref["meta"]
        assert g.dtype == (g_dtype or torch.float32)
        assert torch.equal(g.float(), OT.flat_slice(ref["payload"], sp.entries, sp.n))
    w0, m0, v0, smeta = T.load_branch_state(state_files[10], sp, "cpu")
    sref = OT.load_file(state_files[10])
    for t, which in ((w0, "w"), (m0, "m"), (v0, "v")):
        assert torch.equal(t, OT.flat_slice(sref["payload"][which], sp.entries, sp.n))
    assert smeta == sref["meta"]


def test_index_rejects_foreign_content(tmp_path):
    d = str(tmp_path)
    make_trace(d)
    bad = os.path.join(d, "step_000099_g.pt")
    torch.save({"meta": {}, "payload": {"x": torch.nn.Linear(2, 2)}}, bad)
    with pytest.raises(pickle.UnpicklingError):
        T.TraceFile(bad)
    _c, names, _o, N, s_files, g_files = T.discover_trace(d)
    tf = T.TraceFile(g_files[10])
    card = tf.payload["embed.weight"]
    with pytest.raises(ValueError):
        tf.byte_range(card, 0, card.numel() + 1)
    strided = T.TensorCard(card.key, card.dtype, 0, (10, 10), (1, 10))
    with pytest.raises(ValueError):
        tf.byte_range(strided)
    with pytest.raises(ValueError):
        T.discover_trace(os.path.join(d, "missing"))


def test_reader_surfaces_errors(tmp_path):
    d = str(tmp_path)
    make_trace(d)
    catalog, names, _o, N, s_files, g_files = T.discover_trace(d)
    sp = T.ShardParams(names, catalog, T.TraceFile(s_files[10]).meta, 0, N)
    g_files = dict(g_files)
    g_files[11] = os.path.join(d, "nope.pt")
    with pytest.raises(RuntimeError):
        list(T.WindowReader(g_files, [10, 11], sp, "cpu"))


def test_replay_switches_validate_like_the_reference():
    """Same names and allowed values as replay_fused.py:1137-1198; an unknown
    value raises (a typo must not leave a switch a silent no-op); an arm that
    needs the reference's CPU / eager / mmap path is refused."""
    import pytest
    from sga_amd.replay_run import replay_switches
    assert replay_switches({}) == {"REPLAY_FUSED_FRONT_SORT": "auto", "REPLAY_FUSED_SELECT": "auto",
                                   "REPLAY_FUSED_FRONT_RANK_BG": "auto",
                                   "REPLAY_FUSED_KERNEL": "auto", "REPLAY_FUSED_P1_READ": "pread"}
    assert replay_switches({"REPLAY_FUSED_FRONT_RANK_BG": "off"})["REPLAY_FUSED_FRONT_RANK_BG"] == "off"
    for name, bad in (("REPLAY_FUSED_FRONT_SORT", "CPU"), ("REPLAY_FUSED_SELECT", "1"),
                      ("REPLAY_FUSED_KERNEL", "on"), ("REPLAY_FUSED_P1_READ", "read")):
        with pytest.raises(ValueError, match="is not one of the allowed values"):
            replay_switches({name: bad})
    for name, arm in (("REPLAY_FUSED_FRONT_SORT", "cpu"), ("REPLAY_FUSED_SELECT", "cpu"),
                      ("REPLAY_FUSED_KERNEL", "off"), ("REPLAY_FUSED_P1_READ", "mmap")):
        with pytest.raises(RuntimeError, match="HIP kernels only"):
            replay_switches({name: arm})
