"""Host-side cache for 0-dim scale buffers.

Upstream reads ``self.a.item()`` on every forward (``torch_int/nn/linear.py:40-41``,
``nn/bmm.py:15``), a blocking device-to-host copy per call.  The buffers stay
(state-dict compatibility); this mixin remembers the Python float and only
re-reads when the buffer object or its version counter changed.
"""
import torch


class ScalarCacheMixin:
    def _scalar(self, name):
        buf = getattr(self, name)
        if not torch.is_tensor(buf):
            return float(buf)
        cache = self.__dict__.setdefault("_scalar_cache", {})
        key = (id(buf), buf._version)
        hit = cache.get(name)
        if hit is None or hit[0] != key:
            hit = (key, float(buf.item()))
            cache[name] = hit
        return hit[1]
