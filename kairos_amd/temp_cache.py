"""Bounded temp cache for on-demand converted weights.

The reference allocates a fresh `torch.empty(self.shape)` for every converted weight
(kairos/dynamic_linear.py:145,159).  Here one device buffer is shared by all layers of a process:
it grows to the largest converted weight ever requested (one layer's largest format) and never
beyond `capacity_limit`; a tag remembers what it currently holds so that back-to-back calls of the
same layer in the same format skip the conversion.  ResidentCache is the many-entry variant (LRU under a byte
cap) for processes that can spare HBM for converted copies of their hottest layers.
"""
import torch


class TempCache:
    def __init__(self, capacity_limit=None):
        self.capacity_limit = capacity_limit    # bytes, None = unbounded growth to the largest request
        self._buf = None
        self._tag = None
        self.peak_bytes = 0                     # high-water mark of bytes handed out
        self.hits = 0
        self.misses = 0

    def clear(self):
        self._buf = None
        self._tag = None

    def invalidate(self):
        self._tag = None

    @property
    def capacity(self):
        return 0 if self._buf is None else self._buf.numel()

    def get(self, owner, fmt, shape, dtype, device):
        """owner: a key unique to the layer.  Returns (view of `shape`/`dtype`, hit); on a miss the caller fills it."""
        nbytes = int(torch.empty((), dtype=dtype).element_size())
        for s in shape:
            nbytes *= int(s)
        if self.capacity_limit is not None and nbytes > self.capacity_limit:
            raise MemoryError(f"temp cache: request of {nbytes} B exceeds the limit of {self.capacity_limit} B")
        if self._buf is None or self._buf.numel() < nbytes or self._buf.device != torch.device(device):
            self._buf = None                    # release before growing: peak stays at one buffer
            self._buf = torch.empty(nbytes, dtype=torch.uint8, device=device)
            self._tag = None
        self.peak_bytes = max(self.peak_bytes, nbytes)
        tag = (owner, fmt)
        hit = self._tag == tag
        self._tag = tag
        if hit:
            self.hits += 1
        else:
            self.misses += 1
        return self._buf[:nbytes].view(dtype).view(*shape), hit


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
        self._entries = OrderedDict()           # (owner, fmt) -> [uint8 buffer, holds a valid copy]
        self._bytes = 0
        self._scratch = TempCache()             # requests larger than the whole capacity: converted, never kept
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

    def get(self, owner, fmt, shape, dtype, device):
        nbytes = int(torch.empty((), dtype=dtype).element_size())
        for s in shape:
            nbytes *= int(s)
        key = (owner, fmt)
        entry = self._entries.get(key)
        if entry is not None and entry[0].numel() == nbytes and entry[0].device == torch.device(device):
            self._entries.move_to_end(key)
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
        self._entries[key] = [buf, True]
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
