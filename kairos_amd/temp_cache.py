"""Bounded temp cache for on-demand converted weights.

The reference allocates a fresh `torch.empty(self.shape)` for every converted weight
(kairos/dynamic_linear.py:145,159).  Here one device buffer is shared by all layers of a process:
it grows to the largest converted weight ever requested (one layer's largest format) and never
beyond `capacity_limit`; a tag remembers what it currently holds so that back-to-back calls of the
same layer in the same format skip the conversion.
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


_default = TempCache()


def default_cache():
    return _default
