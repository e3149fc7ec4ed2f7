"""DiskTensor: a tensor viewing a memory-mapped .npy file
(python/shmtensor/disk_tensor.py:8-47 in the reference)."""
import os

from .. import install_aliases
from ._host_view import HostTensorView

capi = install_aliases()


def _close(size, ptr, fd, pin_memory):
    capi.close_mmap_tensor(size, ptr, fd, pin_memory)


class DiskTensor(HostTensorView):

    def __init__(self, filename, pin_memory=False):
        if not os.path.exists(filename):
            raise FileNotFoundError(filename)
        if not filename.endswith(".npy"):
            raise ValueError("DiskTensor expects a .npy file, got %r" % filename)
        self.filename_, self.pin_memory_ = filename, pin_memory
        view, self.size_, self.ptr_, self.fd_ = capi.open_mmap_tensor(filename, pin_memory)
        self._adopt(view, _close, self.size_, self.ptr_, self.fd_, pin_memory)
