"""Common part of the host tensor providers: an object that owns some mapping
of host memory (a shared-memory segment, a memory-mapped file), exposes it as
`tensor_` and forwards the usual read-only tensor attributes to it. The
mapping is released by a finalizer that holds only plain values, never the
object or its tensor."""
import math
import weakref

import torch


class HostTensorView:
    tensor_ = None

    def _adopt(self, tensor, release, *release_args):
        """Install `tensor` as the view and arrange for `release(*release_args)`
        to run once when this object goes away (or at interpreter exit)."""
        self.tensor_ = tensor
        self._finalizer = weakref.finalize(self, release, *release_args)

    def pinned(self):
        """A staging copy of the mapped tensor in pinned host memory, which GPU
        kernels can read and write (uva_fetch / cache_fetch / uva_set ...). It is
        the way onto the GPU where the driver does not register an existing
        mapping in place (pin_memory=True raises there). Made on first use and
        kept; GPU writes land in the copy until flush() is called."""
        if getattr(self, "_staged", None) is None:
            self._staged = torch.empty(self.tensor_.shape, dtype=self.tensor_.dtype, pin_memory=True)
            self._staged.copy_(self.tensor_)
        return self._staged

    def flush(self):
        """Copy the staging copy back into the mapping (after GPU writes to it).
        The caller synchronises the GPU work first."""
        if getattr(self, "_staged", None) is not None:
            self.tensor_.copy_(self._staged)

    shape = property(lambda self: self.tensor_.shape)
    dtype = property(lambda self: self.tensor_.dtype)
    device = property(lambda self: self.tensor_.device)
    size = property(lambda self: self.tensor_.size)


def tensor_nbytes(shape, dtype):
    return math.prod(int(d) for d in shape) * torch.empty(0, dtype=dtype).element_size()
