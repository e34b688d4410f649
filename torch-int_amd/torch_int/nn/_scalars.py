"""Host-side cache for 0-dim scale buffers.

Upstream reads ``self.a.item()`` on every forward (``torch_int/nn/linear.py:40-41``,
``nn/bmm.py:15``), a blocking device-to-host copy per call.  The buffers stay
(state-dict compatibility); this mixin remembers the Python float and only
re-reads when the buffer object or its version counter changed.
"""
import torch


class ScalarCacheMixin:
    def _scalar(self, name):
        buf = self._buffers.get(name)  # skips nn.Module.__getattr__: this runs several times per kernel launch
        if buf is None:
            buf = getattr(self, name)
            if not torch.is_tensor(buf):
                return float(buf)
        cache = self.__dict__.get("_scalar_cache")
        if cache is None:
            cache = self.__dict__["_scalar_cache"] = {}
        hit = cache.get(name)
        if hit is not None and hit[0] is buf and hit[1] == buf._version:
            return hit[2]
        value = float(buf.item())
        cache[name] = (buf, buf._version, value)
        return value
