"""DiskTensor: a tensor viewing a memory-mapped .npy file
(python/shmtensor/disk_tensor.py:8-47 in the reference)."""
import os
import weakref

from .. import install_aliases

capi = install_aliases()


def _close(size, ptr, fd, pin_memory):
    capi.close_mmap_tensor(size, ptr, fd, pin_memory)


class DiskTensor:

    def __init__(self, filename, pin_memory=False):
        if not os.path.exists(filename):
            raise FileNotFoundError(filename)
        if not filename.endswith(".npy"):
            raise ValueError("DiskTensor expects a .npy file, got %r" % filename)
        self.filename_ = filename
        self.pin_memory_ = pin_memory
        self.tensor_, self.size_, self.ptr_, self.fd_ = capi.open_mmap_tensor(filename, pin_memory)
        # the finalizer must not keep the object (or its tensor) alive
        self._disk_finalizer = weakref.finalize(self, _close, self.size_, self.ptr_, self.fd_,
                                                self.pin_memory_)

    @property
    def shape(self):
        return self.tensor_.shape

    @property
    def dtype(self):
        return self.tensor_.dtype

    @property
    def device(self):
        return self.tensor_.device

    @property
    def size(self):
        return self.tensor_.size
