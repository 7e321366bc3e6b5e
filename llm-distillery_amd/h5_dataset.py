"""`distributions.hdf5` without h5py: the storage half of the reference's dataset manager.

Mirrors what `H5DataManager` (classes/data_manager.py) does to the file — the per-conversation
group layout of `_save_data` (:287-312), `_load_id` (:315-329), `_make_outgoing_batch` (:332-353),
the id / sha / attribute queries (:143-156, :271-284) and `_clear_dataset` / `_rename_ids`
(:355-376) — as plain synchronous methods of `DistributionStore`.  The child process, queues and
shared-memory shell around them are not rebuilt: `packed_batch` decodes conversations on a thread
pool (zlib releases the GIL) straight into pinned host memory in the storage dtypes, which is what
the loss kernels read.

Writing is append-only: new datasets go to the end of the file as they are saved; `flush()`
appends fresh copies of the groups that changed and of the root group, then repoints the
superblock (the only bytes rewritten in place), so a crash between flushes leaves the previous
consistent state.  Space of replaced objects is not reused; `compact()` writes a tight copy.
Files keep the format h5py/libhdf5 produce and read (see `h5_format`).
"""
from __future__ import annotations

import mmap
import os
import struct
from concurrent.futures import ThreadPoolExecutor
from typing import Iterable, Sequence

import numpy as np

from . import h5_format as F
from .h5_format import H5FormatError

DISTR_KEY, INDICES_KEY = "distributions", "indices"


def _to_numpy(x) -> np.ndarray:
    return x.detach().cpu().numpy() if hasattr(x, "detach") else np.asarray(x)


class _Group:
    __slots__ = ("address", "attrs", "members", "loaded", "dirty")

    def __init__(self, address: int | None):
        self.address = address          # object header in the file (None: not written yet)
        self.attrs: dict[str, object] = {}
        self.members: dict[str, int] = {}
        self.loaded = address is None
        self.dirty = address is None


class DistributionStore:
    """One `distributions.hdf5`.  `mode`: 'r' read-only, 'a' read/append (created when missing),
    'w' start empty."""

    def __init__(self, path: str, mode: str = "a", compression_level: int = 6, workers: int = 8,
                 chunk_bytes: int = 1 << 20):
        if mode not in ("r", "a", "w"):
            raise ValueError("mode must be 'r', 'a' or 'w'")
        self.path, self.mode, self.level = path, mode, compression_level
        self.workers = max(1, workers)
        self.chunk_bytes = chunk_bytes
        self._pool: ThreadPoolExecutor | None = None
        self._map = None
        self._reader: F.H5Reader | None = None
        self._groups: dict[str, _Group] = {}
        self._file_attrs: dict[str, object] = {}
        self._root_dirty = False
        exists = os.path.exists(path) and os.path.getsize(path) > 0
        if mode == "r":
            if not exists:
                raise FileNotFoundError(path)
            self._fd = os.open(path, os.O_RDONLY)
        else:
            self._fd = os.open(path, os.O_RDWR | os.O_CREAT | (os.O_TRUNC if mode == "w" else 0), 0o644)
        if exists and mode != "w":
            self._end = os.fstat(self._fd).st_size
            self._mapped = 0
            self._remap()
            root = self._reader.object(self._reader.root_address)
            self._file_attrs = self._reader.attributes(root)
            for name, addr in self._reader.links(root).items():
                self._groups[name] = _Group(addr)
            self._end = max(self._end, self._reader.eof_address)
        else:
            self._end = 96                                  # room for the superblock
            self._root_dirty = True
            self.flush()                                    # an empty, valid file from the start

    # -- plumbing -------------------------------------------------------------------------------
    def _remap(self):
        if self._reader is not None:
            self._reader.buf.release()
            self._reader = None
        if self._map is not None:
            self._map.close()
        self._map = mmap.mmap(self._fd, 0, access=mmap.ACCESS_READ)
        self._mapped = len(self._map)
        self._reader = F.H5Reader(self._map)

    def _rd(self, upto: int) -> F.H5Reader:
        """The reader over a mapping that covers the file up to `upto` (objects are addressed
        absolutely, so a mapping made before later appends stays valid for everything it covers)."""
        if self._reader is None or self._mapped < upto:
            self._remap()
        return self._reader

    def _append(self, blob: bytes) -> int:
        if self.mode == "r":
            raise PermissionError("store opened read-only")
        addr = self._end
        view, done = memoryview(blob), 0
        while done < len(view):
            done += os.pwrite(self._fd, view[done:], addr + done)
        self._end = addr + len(blob)
        return addr

    def _group(self, name: str) -> _Group:
        g = self._groups[name]
        if not g.loaded:
            rd = self._rd(g.address + 16)
            obj = rd.object(g.address)
            g.attrs = rd.attributes(obj)
            g.members = rd.links(obj)
            g.loaded = True
        return g

    @staticmethod
    def _key(convo_id: int) -> str:
        return f"convo_{int(convo_id)}"

    # -- queries ---------------------------------------------------------------------------------
    def get_available_ids(self) -> list[int]:
        """classes/data_manager.py:103: the ids of all conversation groups."""
        return [int(k.split("_")[1]) for k in self._groups]

    def has_data(self) -> bool:
        return len(self._groups) > 0

    def get_available_shas(self) -> dict[int, str]:
        """classes/data_manager.py:271-275 (a group without `content_sha` raises KeyError there too)."""
        return {int(k.split("_")[1]): self._group(k).attrs["content_sha"] for k in self._groups}

    def update_shas(self, shas: dict[int, str]):
        for cid, sha in shas.items():
            k = self._key(cid)
            if k in self._groups:
                g = self._group(k)
                g.attrs["content_sha"] = str(sha)
                g.dirty = True

    def get_dataset_attr(self, name: str):
        return self._file_attrs.get(name, None)

    def set_dataset_attr(self, name: str, value):
        if self.mode == "r":
            raise PermissionError("store opened read-only")
        self._file_attrs[name] = value
        self._root_dirty = True

    def get_vocab_family(self):
        return self.get_dataset_attr("vocab_family")

    def set_vocab_family(self, family: str):
        self.set_dataset_attr("vocab_family", family)

    def get_topk(self):
        return self.get_dataset_attr("topk")

    def set_topk(self, topk: int):
        self.set_dataset_attr("topk", int(topk))

    def group_attrs(self, convo_id: int) -> dict[str, object]:
        return dict(self._group(self._key(convo_id)).attrs)

    # -- loading ---------------------------------------------------------------------------------
    def _dataset(self, convo_id: int, key: str):
        name = self._key(convo_id)
        if name not in self._groups:
            raise ValueError(f"Convo ID {convo_id} not found in dataset.")
        g = self._group(name)
        if key not in g.members:
            return None
        rd = self._rd(g.members[key] + 16)
        obj = rd.object(g.members[key])
        return rd, obj, rd.dataset_info(obj)

    def shape_of(self, convo_id: int) -> tuple[tuple[int, int], bool]:
        """((rows, width) of the conversation's distributions, has indices) without decoding."""
        d = self._dataset(convo_id, DISTR_KEY)
        if d is None:
            raise ValueError(f"Convo ID {convo_id} has no distributions in dataset.")
        return tuple(d[2].shape), INDICES_KEY in self._group(self._key(convo_id)).members

    def load_id(self, convo_id: int, storage: bool = False):
        """`_load_id` (classes/data_manager.py:315-329): (distributions float32, indices int64 or
        None); `storage=True` returns what the file holds (float16, uint32) without the casts."""
        d = self._dataset(convo_id, DISTR_KEY)
        if d is None:
            raise ValueError(f"Convo ID {convo_id} has no distributions in dataset.")
        i = self._dataset(convo_id, INDICES_KEY)
        rd = self._reader                                   # the latest mapping covers both datasets
        dist = rd.read_dataset(d[1], d[2])
        idx = rd.read_dataset(i[1], i[2]) if i is not None else None
        if storage:
            return dist, idx
        return dist.astype(np.float32), (idx.astype(np.int64) if idx is not None else None)

    def make_outgoing_batch(self, batch_ids: Sequence[int]):
        """`_make_outgoing_batch` (classes/data_manager.py:332-353) minus the shared-memory handle:
        (padded_batch float32 [B, max_len, width] zero-padded, batch_indices, batch_padding)."""
        loaded = [self.load_id(c) for c in batch_ids]
        max_len = max(len(d) for d, _ in loaded)
        padded = np.stack([np.pad(d, ((0, max_len - len(d)), (0, 0))) for d, _ in loaded])
        return padded, [i for _, i in loaded], [len(d) for d, _ in loaded]

    def packed_batch(self, batch_ids: Sequence[int], pin: bool = True):
        """The rows of the conversations back to back, decoded straight into (pinned) host tensors in
        the storage dtypes: (log-probs float16 [sum N_b, K], ids int32 [sum N_b, K], counts).  uint32
        ids are reinterpreted as int32 (token ids are far below 2^31; checked).  The tensors go to
        the device in two copies and are split per conversation by `counts`."""
        import torch
        metas = []
        for c in batch_ids:
            d = self._dataset(c, DISTR_KEY)
            i = self._dataset(c, INDICES_KEY)
            if d is None:
                raise ValueError(f"Convo ID {c} has no distributions in dataset.")
            if i is None:
                raise ValueError(f"Convo ID {c} has no indices (dense-mode data): use load_id")
            if d[2].shape != i[2].shape or d[2].dtype.numpy != np.float16 or i[2].dtype.numpy.kind not in "iu" \
                    or i[2].dtype.numpy.itemsize != 4:
                raise H5FormatError(f"Convo ID {c}: distributions {d[2].shape} {d[2].dtype.numpy}, "
                                    f"indices {i[2].shape} {i[2].dtype.numpy}")
            metas.append((d[1:], i[1:]))
        widths = {m[0][1].shape[1] for m in metas}
        if len(widths) > 1:
            raise ValueError(f"conversations of different top-K in one batch: {sorted(widths)}")
        K = widths.pop() if widths else 0
        counts = [m[0][1].shape[0] for m in metas]
        total = int(sum(counts))
        pin = pin and torch.cuda.is_available()
        vals = torch.empty((total, K), dtype=torch.float16, pin_memory=pin)
        ids = torch.empty((total, K), dtype=torch.int32, pin_memory=pin)
        nv, ni = vals.numpy(), ids.numpy()
        cuts = np.cumsum([0] + counts)
        rd = self._reader

        # one task per stored chunk (about 1 MiB of rows each), so that a batch of a few long
        # conversations still spreads over all workers
        tasks = []
        for b, pair in enumerate(metas):
            for which, (obj, info) in enumerate(pair):
                dst = (nv if which == 0 else ni)[cuts[b]:cuts[b + 1]]
                if info.layout != 2:
                    rd.read_dataset(obj, info, out=dst)
                    continue
                dst = dst.view(info.dtype.numpy.newbyteorder("="))
                dst[...] = 0
                tasks += [(info, ch, dst) for ch in rd.chunk_list(info)]

        def job(t):
            rd.decode_chunk(*t)

        if self.workers > 1 and len(tasks) > 1:
            if self._pool is None:
                self._pool = ThreadPoolExecutor(self.workers)
            list(self._pool.map(job, tasks))
        else:
            for t in tasks:
                job(t)
        if total and K and int(ni.min()) < 0:
            raise ValueError("token ids outside int32")
        return vals, ids, counts

    def teachers_for_batch(self, batch_ids: Sequence[int], device):
        """`packed_batch` uploaded: [(log-probs [N_b, K], ids [N_b, K])] device views per conversation,
        the form `distill_loss_batch_indexed` takes."""
        vals, ids, counts = self.packed_batch(batch_ids)
        dv, di = vals.to(device, non_blocking=True), ids.to(device, non_blocking=True)
        cuts = np.cumsum([0] + counts)
        return [(dv[cuts[b]:cuts[b + 1]], di[cuts[b]:cuts[b + 1]]) for b in range(len(counts))]

    # -- saving ----------------------------------------------------------------------------------
    def save_data(self, data: np.ndarray, convo_id: int, indices: np.ndarray | None = None,
                  content_sha: str | None = None, sample: str | None = None):
        """`_save_data` (classes/data_manager.py:287-312): create the group if missing, set the two
        attributes when given, replace `distributions` (stored float16) and, when given, `indices`
        (stored uint32)."""
        name = self._key(convo_id)
        if name not in self._groups:
            if self.mode == "r":
                raise PermissionError("store opened read-only")
            self._groups[name] = _Group(None)
            self._root_dirty = True
        g = self._group(name)
        if content_sha is not None:
            g.attrs["content_sha"] = str(content_sha)
        if sample is not None:
            g.attrs["sample"] = str(sample)
        data = np.asarray(data)
        if data.ndim != 2:
            raise ValueError("distributions are [rows, width]")
        blob, addr = F.chunked_dataset(data.astype(np.float16, copy=False), self._end, self.level, self.chunk_bytes)
        self._append(blob)
        g.members[DISTR_KEY] = addr
        if indices is not None:
            indices = np.asarray(indices)
            if indices.shape != data.shape:
                raise ValueError(f"indices {indices.shape} for distributions {data.shape}")
            if indices.size and (indices.min() < 0 or indices.max() > 0xFFFFFFFF):
                raise ValueError("token ids outside uint32")
            blob, addr = F.chunked_dataset(indices.astype(np.uint32, copy=False), self._end, self.level, self.chunk_bytes)
            self._append(blob)
            g.members[INDICES_KEY] = addr
        g.dirty = True

    def put_distribution(self, data, convo_id: int, indices, content_sha: str | None = None,
                         sample: str | None = None, *, vocab: int, device="cuda:0"):
        """One item of `_process_distributions` (classes/data_manager.py:180-195): a conversation that
        is new is saved as it comes; one that is already stored is merged with what the file holds
        (`_merge_data`, :198-261 — probabilities of shared ids add, the K largest stay, rows beyond
        the shorter input pass through) by the GPU merge kernel, and the result replaces the stored
        datasets while the group's attributes stay.  `data` / `indices`: [rows, K] log-probs and ids
        (numpy or torch); `vocab`: the teachers' vocabulary size (ids must lie below it).
        Dense-mode conversations (no `indices`) cannot be merged: the reference's own dense merge
        fails too (it returns an unbound name), so this raises instead of guessing."""
        import torch
        from . import teacher_prep
        name = self._key(convo_id)
        if name not in self._groups:
            self.save_data(_to_numpy(data), convo_id, None if indices is None else _to_numpy(indices), content_sha, sample)
            return
        if indices is None or INDICES_KEY not in self._group(name).members:
            raise ValueError(f"Convo ID {convo_id}: dense-mode data cannot be merged")
        disk_v, disk_i = self.load_id(convo_id, storage=True)
        if int(disk_i.max(initial=0)) >= vocab:
            raise ValueError(f"Convo ID {convo_id}: stored ids reach beyond a vocabulary of {vocab}")
        dev = torch.device(device)
        dv = torch.from_numpy(disk_v).to(dev).float()
        di = torch.from_numpy(disk_i.view(np.int32)).to(dev)
        nv = torch.as_tensor(_to_numpy(data)).to(dev).float()
        ni = torch.as_tensor(_to_numpy(indices).astype(np.int32)).to(dev)
        logmass, ids = teacher_prep.merge_topk_pair(dv, di, nv, ni, vocab)
        self.save_data(logmass.cpu().numpy(), convo_id, ids.cpu().numpy())

    def clear_ids(self, ids: Iterable[int]):
        """`_clear_dataset` (classes/data_manager.py:355-367): drops the groups (missing ones are
        skipped) and, as there, the file attributes `vocab_family` and `topk`."""
        if self.mode == "r":
            raise PermissionError("store opened read-only")
        for cid in ids:
            self._groups.pop(self._key(cid), None)
        if "vocab_family" not in self._file_attrs or "topk" not in self._file_attrs:
            raise KeyError("vocab_family / topk")           # `del attrs[...]` raises there as well
        del self._file_attrs["vocab_family"]
        del self._file_attrs["topk"]
        self._root_dirty = True

    def clear_dataset(self):
        self.clear_ids(self.get_available_ids())

    def rename_ids(self, ids_to_rename: dict[int, int]):
        """`_rename_ids` (classes/data_manager.py:370-376): all moves happen at once, so chains and
        swaps (1->2, 2->1) work; a target that exists and is not itself renamed raises."""
        if self.mode == "r":
            raise PermissionError("store opened read-only")
        olds = {self._key(o) for o in ids_to_rename}
        moving = {}
        for old, new in ids_to_rename.items():
            if self._key(old) not in self._groups:
                raise KeyError(self._key(old))
            if self._key(new) in moving or (self._key(new) in self._groups and self._key(new) not in olds):
                raise ValueError(f"{self._key(new)} already exists")
            moving[self._key(new)] = self._groups[self._key(old)]
        for k in olds:                                      # nothing is touched before every move is known to work
            del self._groups[k]
        self._groups.update(moving)
        self._root_dirty = True

    # -- flushing --------------------------------------------------------------------------------
    def _attr_messages(self, attrs: dict[str, object]) -> list[bytes]:
        """Attribute messages for `attrs`; strings go to a global heap collection appended first."""
        strings = [(k, v.encode("utf-8")) for k, v in attrs.items() if isinstance(v, str)]
        coll_addr = None
        if strings:
            coll_addr = self._append(F.global_heap_collection([s for _, s in strings]))
        msgs, si = [], 0
        for k, v in attrs.items():
            if isinstance(v, str):
                si += 1
                raw = v.encode("utf-8")
                msgs.append(F.attribute_message(k, F.VLEN_UTF8_MESSAGE, (), struct.pack("<IQI", len(raw), coll_addr, si)))
                continue
            arr = np.asarray(v)
            if arr.dtype.kind == "b":
                arr = arr.astype(np.int8)
            if arr.dtype.kind not in "iuf":
                raise TypeError(f"attribute {k!r} of type {type(v).__name__} cannot be stored")
            msgs.append(F.attribute_message(k, F.datatype_message(arr.dtype), arr.shape, arr.tobytes()))   # tobytes: C order
        return msgs

    def _write_group(self, attrs: dict[str, object], members: dict[str, int]) -> tuple[int, int, int]:
        msgs = self._attr_messages(attrs)
        blob, btree, heap = F.group_structures(members, self._end)
        self._append(blob)
        header = F.object_header([F._message(F.MSG_SYMBOL_TABLE, struct.pack("<QQ", btree, heap))] + msgs)
        header += b"\0" * (F._pad8(len(header)) - len(header))
        return self._append(header), btree, heap

    def flush(self):
        if self.mode == "r":
            return
        changed = self._root_dirty
        for g in self._groups.values():
            if g.dirty:
                g.address, _, _ = self._write_group(g.attrs, g.members)
                g.dirty = False
                changed = True
        if not changed:
            return
        root, btree, heap = self._write_group(self._file_attrs, {k: g.address for k, g in self._groups.items()})
        os.fsync(self._fd)                                  # everything new is on disk before the superblock points at it
        os.pwrite(self._fd, F.superblock(root, btree, heap, self._end), 0)
        os.fsync(self._fd)
        self._root_dirty = False
        self._mapped = 0                                    # the next read maps the file afresh

    def close(self):
        if self._fd is None:
            return
        self.flush()
        if self._pool is not None:
            self._pool.shutdown()
            self._pool = None
        if self._reader is not None:
            self._reader.buf.release()
            self._reader = None
        if self._map is not None:
            self._map.close()
            self._map = None
        os.close(self._fd)
        self._fd = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def compact(self, dst_path: str):
        """A tight copy (no superseded objects) at `dst_path`: every conversation re-encoded."""
        with DistributionStore(dst_path, "w", self.level, self.workers, self.chunk_bytes) as out:
            for k, v in self._file_attrs.items():
                out.set_dataset_attr(k, v)
            for cid in self.get_available_ids():
                g = self._group(self._key(cid))
                if DISTR_KEY in g.members:
                    d, i = self.load_id(cid, storage=True)
                    out.save_data(d, cid, i)
                else:
                    out._groups[self._key(cid)] = _Group(None)
                og = out._group(self._key(cid))
                og.attrs = dict(g.attrs)
                og.dirty = True


class BatchPrefetcher:
    """`enqueue_get_batches` / `read_next_batch` / `read_only_mode` (classes/data_manager.py:379-398)
    without the child process: a worker thread inflates the coming batches into pinned memory and
    uploads them on a copy stream of its own (default priority) while the current batch trains; at
    most `depth` batches wait.  Iterating yields, per batch, the list `teachers_for_batch` returns;
    the consumer's current stream is made to wait for the upload, so the tensors can be used at once.
    `loop=True` goes round the batches until `close()` (the reference's read-only mode).  The store
    must not be written to while a prefetcher reads it."""

    _END = object()

    def __init__(self, store: DistributionStore, batches: Sequence[Sequence[int]], device, depth: int = 2, loop: bool = False):
        import queue
        import threading
        import torch
        self._torch = torch
        self.store, self.batches, self.loop = store, [list(b) for b in batches], loop
        self.device = torch.device(device)
        self._queue: "queue.Queue" = queue.Queue(max(1, depth))
        self._closing = threading.Event()
        self._stream = torch.cuda.Stream(self.device) if self.device.type == "cuda" else None
        self._thread = threading.Thread(target=self._work, name="distribution-prefetch", daemon=True)
        self._thread.start()

    def _put(self, item) -> bool:
        import queue
        while not self._closing.is_set():
            try:
                self._queue.put(item, timeout=0.05)
                return True
            except queue.Full:
                continue
        return False

    def _work(self):
        torch = self._torch
        try:
            while True:
                for ids in self.batches:
                    if self._closing.is_set():
                        return
                    vals, idx, counts = self.store.packed_batch(ids)
                    if self._stream is not None:
                        with torch.cuda.stream(self._stream):
                            dv, di = vals.to(self.device, non_blocking=True), idx.to(self.device, non_blocking=True)
                            ready = self._stream.record_event()
                    else:
                        dv, di, ready = vals, idx, None
                    # the pinned staging tensors travel along: they must outlive the copies
                    if not self._put((dv, di, counts, ready, (vals, idx))):
                        return
                if not self.loop:
                    break
            self._put(self._END)
        except BaseException as e:                          # handed to the consumer, which re-raises it
            self._put(e)

    def __iter__(self):
        return self

    def __next__(self):
        item = self._queue.get()
        if item is self._END:
            self._queue.put(item)                           # further calls keep ending
            raise StopIteration
        if isinstance(item, BaseException):
            self._queue.put(item)
            raise item
        dv, di, counts, ready, _staging = item
        if ready is not None:
            cur = self._torch.cuda.current_stream(self.device)
            cur.wait_event(ready)
            dv.record_stream(cur)
            di.record_stream(cur)
            # the pinned staging tensors may go now: torch's host allocator holds a pinned block back
            # until the copies that read it have finished
        cuts = np.cumsum([0] + list(counts))
        return [(dv[cuts[b]:cuts[b + 1]], di[cuts[b]:cuts[b + 1]]) for b in range(len(counts))]

    def close(self):
        self._closing.set()
        while self._thread.is_alive():
            try:
                self._queue.get_nowait()
            except Exception:
                pass
            self._thread.join(0.05)

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()
