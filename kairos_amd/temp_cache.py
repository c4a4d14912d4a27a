"""Bounded temp cache for on-demand converted weights.

The reference allocates a fresh `torch.empty(self.shape)` for every converted weight
(kairos/dynamic_linear.py:145,159).  Here one device buffer is shared by all layers of a process:
it grows to the largest converted weight ever requested (one layer's largest format) and never
beyond `capacity_limit`; a tag remembers what it currently holds so that back-to-back calls of the
same layer in the same format skip the conversion.  ResidentCache is the many-entry variant (LRU under a byte
cap) for processes that can spare HBM for converted copies of their hottest layers.
"""
import torch


# ---- what the caches need to know about streams (module-level so that host-logic tests can replace them) ------------
def _is_capturing(device):
    """True while the current stream of a GPU device records a graph."""
    return device.type == "cuda" and torch.cuda.is_current_stream_capturing()


def _current_stream(device):
    """The current stream object of a GPU device, None for a CPU 'device' (host-logic tests)."""
    return torch.cuda.current_stream(device) if device.type == "cuda" else None


def _order_after(stream, earlier):
    """Everything queued on `earlier` so far happens before whatever is queued on `stream` from now on."""
    ev = torch.cuda.Event()
    ev.record(earlier)
    stream.wait_event(ev)


def _nbytes(shape, dtype):
    n = int(torch.empty((), dtype=dtype).element_size())
    for s in shape:
        n *= int(s)
    return n


class _StreamOrder:
    """Remembers the stream a buffer was last handed out on.  A request from another stream is ordered behind all
    work queued on that stream so far (the conversion that filled the buffer and the GEMM that reads it were both
    queued there before this request was made), so a hit never reads a half-written copy and a miss never
    overwrites a copy that is still being read."""

    def __init__(self):
        self.last = None

    def handover(self, device):
        """-> True when the buffer changed streams (the caller may want to tell the allocator)."""
        stream = _current_stream(device)
        if stream is None:
            return False
        moved = self.last is not None and self.last != stream
        if moved:
            _order_after(stream, self.last)
        self.last = stream
        return moved


class TempCache:
    """One shared buffer.  Stream rules: requests from different streams are ordered through events (see
    _StreamOrder).  Graph capture: a request made while the current stream is capturing is always a miss -- the
    conversion becomes part of the graph, because on replay the buffer holds whatever ran last -- and it leaves the
    tag cleared; the buffer must already be large enough (run the step once eagerly first), since a buffer whose
    address a graph has recorded is never freed: if a later eager request outgrows it, it is kept aside for the
    graph and a new one is allocated."""

    def __init__(self, capacity_limit=None):
        self.capacity_limit = capacity_limit    # bytes, None = unbounded growth to the largest request
        self._buf = None
        self._tag = None
        self._order = _StreamOrder()
        self._captured = False                  # a graph has recorded the current buffer's address
        self._retired = []                      # outgrown buffers that graphs still point to
        self.peak_bytes = 0                     # high-water mark of bytes handed out
        self.hits = 0
        self.misses = 0

    def clear(self):
        """Drops every buffer.  Only when no captured graph that used this cache is still alive."""
        self._buf = None
        self._tag = None
        self._captured = False
        self._retired = []
        self._order = _StreamOrder()

    def invalidate(self):
        self._tag = None

    def touch(self, device):
        """The buffer was just used on the current stream behind the cache's back (a graph replay)."""
        self._order.handover(torch.device(device))

    def prepare_for_capture(self, device, nbytes=0):
        """Before capturing a step that was run eagerly at least once: the buffer is as large as that step needs
        already; `nbytes` asks for more."""
        if nbytes > self.capacity:
            self.get(None, None, (nbytes,), torch.uint8, device)
            self._tag = None

    @property
    def capacity(self):
        return 0 if self._buf is None else self._buf.numel()

    def get(self, owner, fmt, shape, dtype, device):
        """owner: a key unique to the layer.  Returns (view of `shape`/`dtype`, hit); on a miss the caller fills it."""
        nbytes = _nbytes(shape, dtype)
        device = torch.device(device)
        capturing = _is_capturing(device)
        if self.capacity_limit is not None and nbytes > self.capacity_limit:
            raise MemoryError(f"temp cache: request of {nbytes} B exceeds the limit of {self.capacity_limit} B")
        if self._buf is None or self._buf.numel() < nbytes or self._buf.device != device:
            if capturing:
                raise RuntimeError(f"temp cache: a request of {nbytes} B during graph capture does not fit the buffer of "
                                   f"{self.capacity} B; run the step once eagerly (or call prepare_for_capture) before "
                                   "capturing it")
            if self._captured:
                self._retired.append(self._buf)
            self._buf = None                    # release before growing: peak stays at one buffer
            self._buf = torch.empty(nbytes, dtype=torch.uint8, device=device)
            self._tag = None
            self._captured = False
        self.peak_bytes = max(self.peak_bytes, nbytes)
        view = self._buf[:nbytes].view(dtype).view(*shape)
        if capturing:
            self._captured = True
            self._tag = None
            self._order.last = None             # no events across a capturing stream; replays call touch()
            self.misses += 1
            return view, False
        self._order.handover(device)
        tag = (owner, fmt)
        hit = self._tag == tag
        self._tag = tag
        if hit:
            self.hits += 1
        else:
            self.misses += 1
        return view, hit


class ResidentCache:
    """Several converted weights at once, least recently used out first, never more than `capacity_bytes` in total.

    With 288 GB of HBM a serving process can afford to keep the int8 (or fp16) copies of its hottest layers next to
    the resident int4 tensors: a layer whose copy is still here skips the conversion, exactly as with the
    single-buffer TempCache when the same layer is called twice in a row.  The bound is the caller's: capacity 0
    behaves like no cache, the size of all converted weights like the reference's keep-everything SwitchLinear.
    Same interface as TempCache (`get`, `invalidate`, `clear`, `peak_bytes`, `hits`, `misses`).
    """

    def __init__(self, capacity_bytes):
        from collections import OrderedDict
        self.capacity_limit = int(capacity_bytes)
        self._entries = OrderedDict()           # (owner, fmt) -> [uint8 buffer, holds a valid copy, _StreamOrder]
        self._bytes = 0
        self._scratch = TempCache()             # requests larger than the whole capacity, or made during graph
        self._largest = 0                       # capture: converted, never kept
        self.peak_bytes = 0
        self.hits = 0
        self.misses = 0

    def clear(self):
        self._entries.clear()
        self._bytes = 0
        self._scratch.clear()

    def invalidate(self):
        """Every copy becomes stale (the next request of its layer converts again); the buffers stay allocated."""
        for entry in self._entries.values():
            entry[1] = False

    @property
    def capacity(self):
        return self._bytes + self._scratch.capacity

    def touch(self, device):
        self._scratch.touch(device)

    def prepare_for_capture(self, device, nbytes=0):
        """Sizes the buffer that serves requests made during graph capture (they convert inside the graph and keep
        nothing): the largest request seen so far, or `nbytes`."""
        self._scratch.prepare_for_capture(device, max(nbytes, self._largest))

    def get(self, owner, fmt, shape, dtype, device):
        nbytes = _nbytes(shape, dtype)
        device = torch.device(device)
        self._largest = max(self._largest, nbytes)
        if _is_capturing(device):
            # A hit decided now would be baked into the graph while the copy can be evicted before a replay: inside
            # a capture every request converts into the scratch buffer (sized by an eager run, never freed while
            # a graph points to it), and nothing is kept.
            self.misses += 1
            out, _ = self._scratch.get(owner, fmt, shape, dtype, device)
            return out, False
        key = (owner, fmt)
        entry = self._entries.get(key)
        if entry is not None and entry[0].numel() == nbytes and entry[0].device == device:
            self._entries.move_to_end(key)
            if entry[2].handover(device):
                entry[0].record_stream(entry[2].last)   # freed later: not reused before this stream is done with it
            hit, entry[1] = entry[1], True
            self.hits += hit
            self.misses += not hit
            return entry[0].view(dtype).view(*shape), hit
        self.misses += 1
        if entry is not None:
            self._bytes -= self._entries.pop(key)[0].numel()
        if nbytes > self.capacity_limit:
            self._scratch.invalidate()
            out, _ = self._scratch.get(owner, fmt, shape, dtype, device)
            self._scratch.invalidate()          # never report a hit for a buffer other layers overwrite
            self.peak_bytes = max(self.peak_bytes, self._bytes + nbytes)
            return out, False
        while self._bytes + nbytes > self.capacity_limit:
            _, old = self._entries.popitem(last=False)
            self._bytes -= old[0].numel()
            del old
        buf = torch.empty(nbytes, dtype=torch.uint8, device=device)
        order = _StreamOrder()
        order.handover(device)
        self._entries[key] = [buf, True, order]
        self._bytes += nbytes
        self.peak_bytes = max(self.peak_bytes, self._bytes)
        return buf.view(dtype).view(*shape), False


_default = TempCache()


def set_default_cache(cache):
    """Replace the process-wide cache used by layers that have no cache of their own (e.g. a ResidentCache)."""
    global _default
    _default = cache
    return cache


def default_cache():
    return _default
