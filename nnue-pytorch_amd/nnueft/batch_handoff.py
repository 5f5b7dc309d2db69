"""Loader -> device hand-off: the step before the feature transformer.

`SparseBatch` is the struct the reference's C++ loader returns (declared for ctypes in
data_loader/_native.py:33-46; C++ side data_loader/cpp/training_data_loader_internal.h:32-62): a float
block (is_white, outcome, score: 3*size floats, contiguous from `is_white`) and an int block (white,
black, piece_count: 2*size*max_active + size ints, contiguous from `white`).  `get_tensors` returns
what the reference's returns (data_loader/_native.py:48-96): (us, them, white_indices, black_indices,
outcome, score, piece_count), with the same shapes and dtypes.

On a GPU the way there differs from the reference's two pinned allocations, two copies and two
elementwise ops per batch:
  * both blocks are copied into ONE pinned staging buffer taken from a small ring that is reused batch
    after batch (pinned allocations cost far more than the copy they serve),
  * ONE asynchronous copy moves it to the device; white/black/us/outcome/score are views of that block
    (the int block first, so the index lists start on the 256-byte boundary of the allocation),
  * one kernel of libnnueft.so writes `them` and the int64 `piece_count`.
`DevicePrefetcher` runs this on a thread and stream of its own, one or more batches ahead, and orders the
consumer's stream after each copy with an event, like the reference's prefetch worker
(data_loader/dataset.py:291-371).
"""
import ctypes
import queue
import threading

import numpy as np
import torch

from . import _native


class _StagingRing:
    """Pinned host buffers, reused in turn.  A buffer is handed out again only after the copy that last
    read it has finished (its event), so `depth` bounds how many copies can be in flight."""

    def __init__(self, depth: int = 4):
        self.depth = depth
        self._bufs = [None] * depth
        self._events = [None] * depth
        self._next = 0
        self._lock = threading.Lock()

    def take(self, nwords: int):
        with self._lock:
            slot = self._next
            self._next = (slot + 1) % self.depth
        if self._events[slot] is not None:
            self._events[slot].synchronize()
            self._events[slot] = None
        buf = self._bufs[slot]
        if buf is None or buf.numel() < nwords:
            buf = torch.empty(nwords, dtype=torch.int32, device="cpu", pin_memory=True)
            self._bufs[slot] = buf
        return slot, buf[:nwords]

    def sent(self, slot: int, stream) -> None:
        ev = torch.cuda.Event()
        ev.record(stream)
        self._events[slot] = ev


_RINGS = {}
_RINGS_LOCK = threading.Lock()


def _ring(device: torch.device) -> _StagingRing:
    key = (threading.get_ident(), device.index)
    with _RINGS_LOCK:
        if key not in _RINGS:
            _RINGS[key] = _StagingRing()
        return _RINGS[key]


def _blocks(batch):
    size, k = int(batch.size), int(batch.max_active_features)
    floats = np.ctypeslib.as_array(batch.is_white, shape=(3 * size,))
    ints = np.ctypeslib.as_array(batch.white, shape=(2 * size * k + size,))
    return size, k, torch.from_numpy(floats), torch.from_numpy(ints)


def _get_tensors_cpu(batch, use_pinned_memory: bool):
    size, k, floats, ints = _blocks(batch)
    pin = bool(use_pinned_memory) and torch.cuda.is_available()
    # the loader frees its memory with the batch: everything returned is a copy
    fb = torch.empty(floats.shape, dtype=torch.float32, pin_memory=pin).copy_(floats)
    ib = torch.empty(ints.shape, dtype=torch.int32, pin_memory=pin).copy_(ints)
    us = fb[0:size].view(size, 1)
    outcome = fb[size:2 * size].view(size, 1)
    score = fb[2 * size:3 * size].view(size, 1)
    white = ib[0:size * k].view(size, k)
    black = ib[size * k:2 * size * k].view(size, k)
    them = torch.empty(us.shape, dtype=torch.float32, pin_memory=pin).fill_(1.0).sub_(us)
    piece_count = torch.empty(size, dtype=torch.int64, pin_memory=pin).copy_(ib[2 * size * k:])
    return us, them, white, black, outcome, score, piece_count


def _get_tensors_gpu(batch, device: torch.device):
    lib = _native.load()      # raises when libnnueft.so is missing: no other path to a GPU
    size, k, floats, ints = _blocks(batch)
    if size <= 0:
        raise ValueError("empty batch")
    n_int, n_float = ints.numel(), floats.numel()
    ring = _ring(device)
    slot, stage = ring.take(n_int + n_float)
    stage[:n_int].copy_(ints)
    stage[n_int:].view(torch.float32).copy_(floats)
    with torch.cuda.device(device):
        stream = torch.cuda.current_stream(device)
        block = torch.empty(n_int + n_float, dtype=torch.int32, device=device)
        block.copy_(stage, non_blocking=True)
        ring.sent(slot, stream)
        white = block[0:size * k].view(size, k)
        black = block[size * k:2 * size * k].view(size, k)
        piece_count32 = block[2 * size * k:n_int]
        fb = block[n_int:].view(torch.float32)
        us = fb[0:size].view(size, 1)
        outcome = fb[size:2 * size].view(size, 1)
        score = fb[2 * size:3 * size].view(size, 1)
        them = torch.empty(size, 1, dtype=torch.float32, device=device)
        piece_count = torch.empty(size, dtype=torch.int64, device=device)
        rc = lib.nnueft_batch_unpack(us.data_ptr(), piece_count32.data_ptr(), them.data_ptr(),
                                     piece_count.data_ptr(), size, stream.cuda_stream)
        _native.check(rc, "nnueft_batch_unpack")
    return us, them, white, black, outcome, score, piece_count


def get_tensors(batch, device, use_pinned_memory: bool = False):
    """(us, them, white_indices, black_indices, outcome, score, piece_count) of a SparseBatch on `device`.

    us/them/outcome/score f32 [size, 1]; the index lists int32 [size, max_active_features], -1 padded;
    piece_count int64 [size].  Nothing returned aliases the loader's memory.  For a GPU the copy is
    asynchronous on the current stream of that device and always goes through pinned staging
    (use_pinned_memory only matters for a CPU device, where it selects pinned result tensors)."""
    device = torch.device(device)
    if device.type == "cpu":
        return _get_tensors_cpu(batch, use_pinned_memory)
    if device.type != "cuda":
        raise ValueError(f"unsupported device {device}")
    if device.index is None:
        device = torch.device("cuda", torch.cuda.current_device())
    return _get_tensors_gpu(batch, device)


class SparseBatch(ctypes.Structure):
    """Field for field the reference's struct (data_loader/_native.py:33-46): a pointer the reference's
    loader library returns can be cast to POINTER(SparseBatch)."""

    _fields_ = [
        ("num_inputs", ctypes.c_int),
        ("size", ctypes.c_int),
        ("is_white", ctypes.POINTER(ctypes.c_float)),
        ("outcome", ctypes.POINTER(ctypes.c_float)),
        ("score", ctypes.POINTER(ctypes.c_float)),
        ("num_active_white_features", ctypes.c_int),
        ("num_active_black_features", ctypes.c_int),
        ("max_active_features", ctypes.c_int),
        ("white", ctypes.POINTER(ctypes.c_int)),
        ("black", ctypes.POINTER(ctypes.c_int)),
        ("piece_count", ctypes.POINTER(ctypes.c_int)),
    ]

    def get_tensors(self, device, use_pinned_memory: bool = False):
        return get_tensors(self, device, use_pinned_memory)

    @classmethod
    def from_arrays(cls, num_inputs, is_white, outcome, score, white, black, piece_count):
        """A SparseBatch over numpy memory laid out like the loader's (one float block, one int block);
        for tests and synthetic data.  The arrays are copied; the result keeps its blocks alive."""
        white = np.ascontiguousarray(white, dtype=np.int32)
        black = np.ascontiguousarray(black, dtype=np.int32)
        size, k = white.shape
        assert black.shape == (size, k)
        fb = np.concatenate([np.asarray(a, dtype=np.float32).reshape(size) for a in (is_white, outcome, score)])
        ib = np.concatenate([white.reshape(-1), black.reshape(-1), np.asarray(piece_count, dtype=np.int32).reshape(size)])
        self = cls()
        self._keep = (fb, ib)
        fp = fb.ctypes.data_as(ctypes.POINTER(ctypes.c_float))
        ip = ib.ctypes.data_as(ctypes.POINTER(ctypes.c_int))
        self.num_inputs, self.size, self.max_active_features = int(num_inputs), size, k
        self.is_white = fp
        self.outcome = ctypes.cast(ctypes.addressof(fp.contents) + 4 * size, ctypes.POINTER(ctypes.c_float))
        self.score = ctypes.cast(ctypes.addressof(fp.contents) + 8 * size, ctypes.POINTER(ctypes.c_float))
        self.white = ip
        self.black = ctypes.cast(ctypes.addressof(ip.contents) + 4 * size * k, ctypes.POINTER(ctypes.c_int))
        self.piece_count = ctypes.cast(ctypes.addressof(ip.contents) + 8 * size * k, ctypes.POINTER(ctypes.c_int))
        self.num_active_white_features = int((white >= 0).sum())
        self.num_active_black_features = int((black >= 0).sum())
        return self


class _Ready:
    __slots__ = ("item", "event")

    def __init__(self, item, event):
        self.item, self.event = item, event


class DevicePrefetcher:
    """Iterates over `source` (an iterator of SparseBatch-like objects, or of tuples of host tensors) and
    yields tuples of tensors on `device`, staged up to `depth` batches ahead by a worker thread on a
    stream of its own (default priority).  `release(batch)`, if given, is called as soon as a batch has
    been copied off the loader's memory (the reference calls destroy_sparse_batch there).

    The consumer's current stream is ordered after each batch's copy with an event, and every tensor is
    recorded on it, so its memory is not reused while the consumer's kernels may still read it.  An
    exception in the worker is re-raised by the consumer; `close()` stops the worker."""

    def __init__(self, source, device, depth: int = 4, release=None, timeout: float = 300.0):
        self.device = torch.device(device)
        if self.device.type == "cuda" and self.device.index is None:
            self.device = torch.device("cuda", torch.cuda.current_device())
        self._source = iter(source)
        self._release = release
        self._timeout = timeout
        self._queue = queue.Queue(maxsize=max(1, depth))
        self._stop = threading.Event()
        self._thread = threading.Thread(target=self._work, daemon=True)
        self._thread.start()

    def _put(self, item) -> None:
        while not self._stop.is_set():
            try:
                self._queue.put(item, timeout=0.2)
                return
            except queue.Full:
                continue

    def _stage(self, batch):
        if hasattr(batch, "get_tensors") or hasattr(batch, "max_active_features"):
            out = get_tensors(batch, self.device, use_pinned_memory=True)
            if self._release is not None:
                self._release(batch)
            return out
        return tuple(t.to(self.device, non_blocking=True) if isinstance(t, torch.Tensor) else t for t in batch)

    def _work(self) -> None:
        try:
            on_gpu = self.device.type == "cuda"
            stream = None
            if on_gpu:
                torch.cuda.set_device(self.device)
                stream = torch.cuda.Stream(device=self.device)
            for batch in self._source:
                if self._stop.is_set():
                    return
                if on_gpu:
                    with torch.cuda.stream(stream):
                        item = self._stage(batch)
                        event = torch.cuda.Event()
                        event.record(stream)
                    self._put(_Ready(item, event))
                else:
                    self._put(_Ready(self._stage(batch), None))
            self._put(None)
        except Exception as e:  # noqa: BLE001  (handed to the consumer)
            self._put(e)

    def __iter__(self):
        return self

    def __next__(self):
        try:
            got = self._queue.get(timeout=self._timeout)
        except queue.Empty:
            raise RuntimeError("prefetch timeout: the loader produced no batch") from None
        if got is None:
            self._queue.put(None)      # stays exhausted
            raise StopIteration
        if isinstance(got, Exception):
            raise got
        if got.event is not None:
            cur = torch.cuda.current_stream(self.device)
            cur.wait_event(got.event)
            for t in got.item:
                if isinstance(t, torch.Tensor) and t.is_cuda:
                    t.record_stream(cur)
        return got.item

    def close(self) -> None:
        self._stop.set()
        try:
            while True:
                self._queue.get_nowait()
        except queue.Empty:
            pass
        self._thread.join(timeout=2.0)

    def __del__(self):
        try:
            self._stop.set()
        except Exception:  # noqa: BLE001
            pass
