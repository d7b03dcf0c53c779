"""Recorded-trace files for the offline replay: layout, index and streaming.

A trace directory holds ``catalog.pt``, branch-point ``step_NNNNNN_state.pt``
files and per-step ``step_NNNNNN_g.pt`` gradient dumps, each a ``torch.save``
zip of ``{"meta": ..., "payload": ...}`` (writer ``sga/trace.py:756-864``;
discovery ``sga/replay.py:174-212``; pread index ``sga/replay_fused.py:779-892``;
prefetcher ``sga/replay_fused.py:895-1104``).

The reader here never materialises a payload tensor on the host heap.  It
parses the zip directory and the pickled index card of every tensor, then
``preadv``s exactly the shard's byte ranges into a ring of flat host staging
buffers (pinned when a device is given) and ships them to the device in the
recorded dtype: a bf16 trace crosses PCIe at 2 B/element and is widened in
registers by the replay kernels, instead of being upcast on the host.
"""
import glob
import io
import os
import pickle
import queue
import re
import struct
import threading
import zipfile

import torch

_STORAGE_DTYPES = {
    "DoubleStorage": torch.float64, "FloatStorage": torch.float32,
    "HalfStorage": torch.float16, "BFloat16Storage": torch.bfloat16,
    "LongStorage": torch.int64, "IntStorage": torch.int32,
    "ShortStorage": torch.int16, "CharStorage": torch.int8,
    "ByteStorage": torch.uint8, "BoolStorage": torch.bool,
}
_ITEMSIZE = {torch.float64: 8, torch.float32: 4, torch.float16: 2, torch.bfloat16: 2,
             torch.int64: 8, torch.int32: 4, torch.int16: 2, torch.int8: 1,
             torch.uint8: 1, torch.bool: 1}
_G_RE = re.compile(r"step_(\d+)_g\.pt$")
_STATE_RE = re.compile(r"step_(\d+)_state\.pt$")
_LOCAL_SIG = 0x04034B50


class TensorCard:
    """Where one payload tensor's bytes live: storage record key, dtype,
    element offset inside the record, shape and strides."""
    __slots__ = ("key", "dtype", "offset", "shape", "stride")

    def __init__(self, key, dtype, offset, shape, stride):
        self.key, self.dtype, self.offset = key, dtype, int(offset)
        self.shape, self.stride = tuple(shape), tuple(stride)

    def numel(self):
        n = 1
        for d in self.shape:
            n *= d
        return n

    def is_contiguous(self):
        want = 1
        for d, s in zip(reversed(self.shape), reversed(self.stride)):
            if d != 1 and s != want:
                return False
            want *= d
        return True


def _card_from_rebuild(storage, offset, size, stride, *unused):
    key, dtype = storage
    return TensorCard(key, dtype, offset, size, stride)


class _CardUnpickler(pickle.Unpickler):
    """Reads ``data.pkl`` into plain containers and ``TensorCard``s.  Only the
    trace writer's vocabulary resolves; any other global is an error, so
    nothing in the file is ever executed."""

    def find_class(self, module, name):
        if (module, name) == ("torch._utils", "_rebuild_tensor_v2"):
            return _card_from_rebuild
        if module == "torch" and name in _STORAGE_DTYPES:
            return _STORAGE_DTYPES[name]
        if (module, name) == ("collections", "OrderedDict"):
            return dict
        raise pickle.UnpicklingError(f"unexpected {module}.{name} in trace index")

    def persistent_load(self, pid):
        ok = (isinstance(pid, tuple) and len(pid) == 5 and pid[0] == "storage"
              and pid[3] == "cpu")
        if not ok:
            raise pickle.UnpicklingError(f"unexpected persistent id {pid!r}")
        return (pid[2], pid[1])


class TraceFile:
    """Index of one trace file: ``meta``, ``payload`` (names -> TensorCard,
    possibly nested one level for state files) and, per storage record, the
    absolute file offset and byte length of its data.

    The data offset is taken from each record's LOCAL zip header: the writer
    pads a record's start to the storage alignment through the local extra
    field, which the central directory does not describe
    (``replay_fused.py:859-892``)."""

    def __init__(self, path):
        self.path = path
        pkl, members = None, {}
        with zipfile.ZipFile(path) as zf:
            for info in zf.infolist():
                parts = info.filename.split("/")
                if parts[-1] == "data.pkl":
                    pkl = zf.read(info)
                elif len(parts) == 3 and parts[1] == "data":
                    if info.compress_type != zipfile.ZIP_STORED:
                        raise ValueError(f"{path}: compressed storage record {info.filename}")
                    members[parts[2]] = (info.header_offset, info.file_size)
        if pkl is None:
            raise ValueError(f"{path}: no data.pkl record")
        self.records = {}
        fd = os.open(path, os.O_RDONLY)
        try:
            for key, (hdr_off, size) in members.items():
                hdr = os.pread(fd, 30, hdr_off)
                if len(hdr) != 30:
                    raise ValueError(f"{path}: short local header read @{hdr_off} "
                                     f"({len(hdr)}/30)")
                sig, = struct.unpack_from("<I", hdr, 0)
                name_len, extra_len = struct.unpack_from("<HH", hdr, 26)
                if sig != _LOCAL_SIG:
                    raise ValueError(f"{path}: bad local header sig @{hdr_off}")
                self.records[key] = (hdr_off + 30 + name_len + extra_len, size)
        finally:
            os.close(fd)
        top = _CardUnpickler(io.BytesIO(pkl)).load()
        self.meta = top.get("meta")
        self.payload = top.get("payload", {})
        self.top = top

    def byte_range(self, card, first=0, count=None):
        """Absolute (offset, nbytes) of elements [first, first+count) of a
        contiguous tensor; raises when the range leaves its storage record."""
        if not card.is_contiguous():
            raise ValueError(f"{self.path}: non-contiguous payload stride={card.stride}")
        count = card.numel() - first if count is None else count
        size = _ITEMSIZE[card.dtype]
        base, rec_bytes = self.records[card.key]
        if (card.offset + card.numel()) * size > rec_bytes:
            raise ValueError(f"{self.path}: storage record {card.key} too short")
        if first < 0 or count < 0 or (card.offset + first + count) * size > rec_bytes \
                or first + count > card.numel():
            raise ValueError(f"{self.path}: slice [{first}, {first + count}) outruns "
                             f"storage record {card.key}")
        return base + (card.offset + first) * size, count * size

    def read_into(self, fd, card, first, count, out_bytes):
        """preadv elements [first, first+count) into ``out_bytes`` (a writable
        byte view of exactly the right length)."""
        off, nbytes = self.byte_range(card, first, count)
        mv = memoryview(out_bytes).cast("B")
        if len(mv) != nbytes:
            raise ValueError("read_into: destination size mismatch")
        got = 0
        while got < nbytes:
            r = os.preadv(fd, [mv[got:]], off + got)
            if r == 0:
                raise OSError(f"short pread {self.path} @{off + got} ({got}/{nbytes})")
            got += r

    def read_tensor(self, card, first=0, count=None, out=None):
        """One tensor slice as a flat host tensor of the recorded dtype."""
        count = card.numel() - first if count is None else count
        if out is None:
            out = torch.empty(count, dtype=card.dtype)
        fd = os.open(self.path, os.O_RDONLY)
        try:
            self.read_into(fd, card, first, count, _bytes_of(out))
        finally:
            os.close(fd)
        return out


def _bytes_of(t):
    """Writable byte view over a contiguous host tensor's memory."""
    return t.view(torch.uint8).numpy()


# ----------------------------------------------------------------- discovery
def discover_trace(trace_dir):
    """(catalog, names, offsets, N, state_files, g_files) of a trace
    directory (``sga/replay.py:174-212``)."""
    if not os.path.isdir(trace_dir):
        raise ValueError(f"--trace-dir does not exist: {trace_dir}")
    cat_path = os.path.join(trace_dir, "catalog.pt")
    if not os.path.isfile(cat_path):
        raise ValueError(f"no catalog.pt in {trace_dir}")
    catalog = TraceFile(cat_path).top["catalog"]
    names = list(catalog)
    if not names:
        raise ValueError(f"catalog.pt has no params in {trace_dir}")
    offsets, total = {}, 0
    for name in names:
        offsets[name] = total
        numel = 1
        for s in catalog[name]["shape"]:
            numel *= int(s)
        catalog[name]["numel"] = numel
        total += numel
    state_files, g_files = {}, {}
    for f in sorted(glob.glob(os.path.join(trace_dir, "*.pt"))):
        base = os.path.basename(f)
        mg, ms = _G_RE.match(base), _STATE_RE.match(base)
        if mg:
            g_files[int(mg.group(1))] = f
        elif ms:
            state_files[int(ms.group(1))] = f
    if not state_files:
        raise ValueError(f"no step_*_state.pt files in {trace_dir}")
    return catalog, names, offsets, total, state_files, g_files


def window_steps_for(g_files, t0, window):
    """Logged steps t0, t0+1, ... up to ``window`` long, ending before the
    first missing g file (``sga/replay.py:215-224``)."""
    steps = []
    for s in range(t0, t0 + window):
        if s not in g_files:
            break
        steps.append(s)
    return steps


def param_hp(meta, catalog_entry):
    """(beta1, beta2, eps, weight_decay, group) of one param: per-group values
    when the trace carries them, else the global scalars
    (``sga/replay.py:268-293``)."""
    groups = meta.get("param_groups") if isinstance(meta, dict) else None
    gi = catalog_entry.get("param_group") if catalog_entry else None
    if groups is not None and gi is not None:
        gi = int(gi)
        if not 0 <= gi < len(groups):
            raise ValueError(f"trace catalog param_group index {gi} outside the step meta "
                             f"param_groups (0..{len(groups) - 1}); catalog and meta come "
                             "from different runs")
        g = groups[gi]
        return (float(g["adam_beta1"]), float(g["adam_beta2"]), float(g["adam_eps"]),
                float(g["weight_decay"]), gi)
    return (float(meta["adam_beta1"]), float(meta["adam_beta2"]), float(meta["adam_eps"]),
            float(meta["weight_decay"]), None)


def lr_for_step(gmeta, group=None):
    """Recorded learning rate of a param group, or the mean over groups when
    the group is unknown (``sga/replay.py:248-257``)."""
    lrs = [float(x) for x in gmeta.get("lr", [0.0])]
    if not lrs:
        return 0.0
    if group is not None and group < len(lrs):
        return lrs[group]
    return sum(lrs) / len(lrs)


class ShardParams:
    """Params overlapping the flat-index slice [lo, hi): per-param offsets
    ``p_off`` (inside the param), ``a`` (inside the shard), length ``n`` and
    hyper-parameters (``sga/replay_fused.py:251-271``)."""

    def __init__(self, names, catalog, meta, lo, hi):
        self.lo, self.hi, self.n = lo, hi, hi - lo
        self.entries = []
        start = 0
        for name in names:
            numel = int(catalog[name]["numel"])
            a, b = max(start, lo), min(start + numel, hi)
            if b > a:
                b1, b2, eps, wd, group = param_hp(meta, catalog.get(name))
                self.entries.append({"name": name, "p_off": a - start, "a": a - lo, "n": b - a,
                                     "b1": b1, "b2": b2, "eps": eps, "wd": wd, "group": group})
            start += numel


# ------------------------------------------------------------------- reading
def load_branch_state(path, sp, device):
    """Flat fp32 device tensors (w0, m0, v0) of the shard from a branch-point
    state file, plus its meta.  Each param slice is read straight into its
    place in one flat host buffer and uploaded once."""
    tf = TraceFile(path)
    pin = torch.device(device).type == "cuda"
    out = []
    fd = os.open(path, os.O_RDONLY)
    try:
        for which in ("w", "m", "v"):
            host = torch.zeros(sp.n, dtype=torch.float32, pin_memory=pin)
            hb = _bytes_of(host)
            for e in sp.entries:
                card = tf.payload[which].get(e["name"])
                if card is None:
                    raise ValueError(f"{path}: state payload {which!r} lacks {e['name']}")
                if card.dtype != torch.float32:
                    raise ValueError(f"{path}: state {which}/{e['name']} is {card.dtype}")
                tf.read_into(fd, card, e["p_off"], e["n"], hb[4 * e["a"]:4 * (e["a"] + e["n"])])
            out.append(host.to(device))
    finally:
        os.close(fd)
    return out[0], out[1], out[2], tf.meta


class WindowReader:
    """Streams the shard's slice of each window step's recorded gradient to
    the device, reading ahead on a background thread.

    Iterating yields ``(gstep, meta, g_flat)``: ``g_flat`` is a flat device
    tensor of the shard's length in the recorded dtype (bf16 or fp32), zeros
    where a param has no entry in that step.  It stays valid until the next
    iteration step re-uses its slot, so consume it before advancing.

    ``depth`` host staging buffers (pinned on a GPU) bound the read-ahead;
    ``read_threads`` threads copy disjoint pieces of a step out of the page
    cache side by side (positional reads release the GIL); the upload runs on
    its own stream and the consumer's current stream is made to wait on it.
    """

    def __init__(self, g_files, window_steps, sp, device, depth=2, index_cache=None,
                 read_threads=8):
        self.g_files, self.steps, self.sp = g_files, list(window_steps), sp
        self.read_threads = max(1, int(read_threads))
        self.device = torch.device(device)
        self.index_cache = {} if index_cache is None else index_cache
        self.depth = max(1, int(depth))
        self._pin = self.device.type == "cuda"
        self._free = queue.Queue()
        self._ready = queue.Queue()
        self._host = {}
        self._dev = {}
        self._exc = None
        for slot in range(self.depth):
            self._free.put(slot)
        self._copy_stream = torch.cuda.Stream(self.device) if self._pin else None
        self._thread = threading.Thread(target=self._read_loop, daemon=True)
        self._thread.start()

    def _buffers(self, slot, dtype):
        key = (slot, dtype)
        if key not in self._host:
            self._host[key] = torch.zeros(self.sp.n, dtype=dtype, pin_memory=self._pin)
        return self._host[key]

    def _read_loop(self):
        from concurrent.futures import ThreadPoolExecutor
        piece = 32 << 20                       # elements per read task
        pool = ThreadPoolExecutor(self.read_threads) if self.read_threads > 1 else None
        try:
            for gstep in self.steps:
                path = self.g_files[gstep]
                tf = self.index_cache.get(path)
                if tf is None:
                    tf = self.index_cache[path] = TraceFile(path)
                cards = [(e, tf.payload.get(e["name"])) for e in self.sp.entries]
                dtypes = {c.dtype for _, c in cards if c is not None}
                if len(dtypes) > 1:
                    raise ValueError(f"{path}: mixed payload dtypes {sorted(map(str, dtypes))}")
                dtype = dtypes.pop() if dtypes else torch.float32
                if dtype not in (torch.float32, torch.bfloat16):
                    raise ValueError(f"{path}: unsupported gradient dtype {dtype}")
                slot = self._free.get()
                if slot is None:
                    return
                host = self._buffers(slot, dtype)
                hb, size = _bytes_of(host), _ITEMSIZE[dtype]
                fd = os.open(path, os.O_RDONLY)
                try:
                    # positional reads release the GIL and are independent, so a few
                    # threads copy disjoint pieces out of the page cache side by side
                    jobs = []
                    for e, card in cards:
                        if card is None:
                            hb[size * e["a"]:size * (e["a"] + e["n"])] = 0
                            continue
                        for lo in range(0, e["n"], piece):
                            cnt = min(piece, e["n"] - lo)
                            dst = hb[size * (e["a"] + lo):size * (e["a"] + lo + cnt)]
                            jobs.append((card, e["p_off"] + lo, cnt, dst))
                    if pool is None:
                        for card, first, cnt, dst in jobs:
                            tf.read_into(fd, card, first, cnt, dst)
                    else:
                        for fut in [pool.submit(tf.read_into, fd, *j) for j in jobs]:
                            fut.result()
                finally:
                    os.close(fd)
                self._ready.put((gstep, tf.meta, slot, dtype))
            self._ready.put(None)
        except BaseException as exc:          # surface in the consumer
            self._exc = exc
            self._ready.put(None)
        finally:
            if pool is not None:
                pool.shutdown(wait=False)

    def __iter__(self):
        cur = torch.cuda.current_stream(self.device) if self._pin else None
        ends = []          # ends[i]: consumer work of iterations < i is enqueued before it
        in_flight = None   # (host slot, upload-done event) of the previous step
        for i, _ in enumerate(self.steps):
            if self._pin:
                ev = torch.cuda.Event()
                ev.record(cur)
                ends.append(ev)
            if in_flight is not None:
                in_flight[1].synchronize()             # host buffer may be refilled
                self._free.put(in_flight[0])
                in_flight = None
            item = self._ready.get()
            if item is None:
                raise RuntimeError("trace read-ahead failed") from self._exc
            gstep, meta, slot, dtype = item
            host = self._host[(slot, dtype)]
            if not self._pin:
                g = host.clone()
                self._free.put(slot)
                yield gstep, meta, g
                continue
            # two device buffers alternate: buffer i % 2 was last read by the
            # consumer's work of iteration i - 2, all enqueued before ends[i - 1]
            dev = self._dev.get((i & 1, dtype))
            if dev is None:
                dev = self._dev[(i & 1, dtype)] = torch.empty(self.sp.n, dtype=dtype,
                                                              device=self.device)
            if i >= 2:
                self._copy_stream.wait_event(ends[i - 1])
            done = torch.cuda.Event()
            with torch.cuda.stream(self._copy_stream):
                dev.copy_(host, non_blocking=True)
                done.record(self._copy_stream)
            cur.wait_event(done)
            in_flight = (slot, done)
            yield gstep, meta, dev
        if in_flight is not None:
            in_flight[1].synchronize()
            self._free.put(in_flight[0])

    def close(self):
        self._free.put(None)


class ResidentWindow:
    """Keeps a window's gradients on the device after the first pass over a
    ``WindowReader`` so that later passes (the dense reference pass, then one
    streaming pass per optimizer family) re-read HBM instead of the trace: a
    32-step bf16 window of a 0.6 B-element shard is 38 GB of the 288 GB.
    Falls back to re-reading when the window would not fit ``budget_bytes``."""

    def __init__(self, make_reader, n_steps, shard_elems, budget_bytes=96 << 30):
        self._make_reader = make_reader
        self._keep = n_steps * shard_elems * 4 <= budget_bytes      # worst case fp32
        self._held = None

    def __iter__(self):
        if self._held is not None:
            yield from self._held
            return
        held = []
        for gstep, meta, g in self._make_reader():
            if self._keep:
                g = g.clone()
                held.append((gstep, meta, g))
            yield gstep, meta, g
        if self._keep:
            self._held = held


# ------------------------------------------------------------------- writing
def write_catalog(trace_dir, catalog, meta, g_dtype="fp32"):
    """``catalog.pt`` in the writer's layout (``sga/trace.py:770-799``):
    ``catalog`` maps name -> {"shape", "dtype", "param_group"}."""
    os.makedirs(trace_dir, exist_ok=True)
    torch.save({"meta": meta, "catalog": catalog, "g_dtype": g_dtype},
               os.path.join(trace_dir, "catalog.pt"))


def write_state(trace_dir, step, meta, w, m, v, g=None):
    """``step_NNNNNN_state.pt`` (``sga/trace.py:810-833``); ``w/m/v/g`` map
    name -> host tensor."""
    payload = {"w": dict(w), "m": dict(m), "v": dict(v), "g": dict(g or {})}
    torch.save({"meta": dict(meta), "payload": payload},
               os.path.join(trace_dir, f"step_{step:06d}_state.pt"))


def write_grad(trace_dir, step, meta, grads, g_dtype=None):
    """``step_NNNNNN_g.pt`` (``sga/trace.py:835-852``); with
    ``g_dtype=torch.bfloat16`` each tensor is stored round-to-nearest bf16."""
    payload = {k: (t.detach().cpu().to(g_dtype) if g_dtype is not None else t.detach().cpu())
               for k, t in grads.items()}
    torch.save({"meta": dict(meta), "payload": payload},
               os.path.join(trace_dir, f"step_{step:06d}_g.pt"))
