"""ShmTensor: a tensor living in a POSIX shared-memory segment that the local
rank 0 creates and the other local ranks open
(python/shmtensor/shm_tensor.py:20-88 in the reference)."""
import torch
import torch.distributed as dist

from .. import install_aliases
from ._host_view import HostTensorView, tensor_nbytes

capi = install_aliases()


def _release(name, size, ptr, fd, pin_memory):
    capi.release_shared_mem(name, size, ptr, fd, pin_memory)


class ShmTensor(HostTensorView):
    """Protocol between the ranks of one node (same as the reference's): nobody
    may find a segment of that name beforehand; rank 0 creates and sizes it while
    the others wait at a barrier; then the others open it. Attribute names
    (`tensor_`, `ptr_`, `fd_`, `size_`, ...) are the reference's."""

    def __init__(self, name, shape, local_rank, local_world_size, local_group=None,
                 dtype=torch.float32, pin_memory=False):
        self.name, self.shape_, self.dtype_, self.pin_memory_ = name, tuple(shape), dtype, pin_memory
        self.cur_rank, self.cur_world_size, self.cur_group = local_rank, local_world_size, local_group
        self.size_ = tensor_nbytes(self.shape_, dtype)
        if self.size_ <= 0:
            raise Exception("Invalid shape")
        # a segment of that name left over by someone else is an error, not something to adopt
        if capi.file_exist(name):
            raise Exception("File name is already exist")
        self._barrier()                    # everybody has looked before anybody creates
        creator = local_rank == 0
        if not creator:
            self._barrier()                # wait for rank 0's segment
        attach = capi.create_shared_mem if creator else capi.open_shared_mem
        self.ptr_, self.fd_ = attach(name, self.size_, pin_memory)
        if creator:
            self._barrier()                # release the waiting ranks
        self._adopt(capi.open_shared_tensor(self.ptr_, dtype, list(self.shape_)), _release, name, self.size_,
                    self.ptr_, self.fd_, pin_memory)

    def _barrier(self):
        if self.cur_world_size > 1 and dist.is_available() and dist.is_initialized():
            dist.barrier(self.cur_group)
