"""ShmTensor: a tensor living in a POSIX shared-memory segment that the local
rank 0 creates and the other local ranks open
(python/shmtensor/shm_tensor.py:20-88 in the reference)."""
import weakref

import torch
import torch.distributed as dist

from .. import install_aliases

capi = install_aliases()


def _release(name, size, ptr, fd, pin_memory):
    capi.release_shared_mem(name, size, ptr, fd, pin_memory)


class ShmTensor:

    def __init__(self, name, shape, local_rank, local_world_size, local_group=None,
                 dtype=torch.float32, pin_memory=False):
        self.name = name
        self.shape_ = tuple(shape)
        self.dtype_ = dtype
        self.pin_memory_ = pin_memory
        self.cur_rank = local_rank
        self.cur_world_size = local_world_size
        self.cur_group = local_group

        self.size_ = torch.empty(0, dtype=dtype).element_size()
        for d in self.shape_:
            self.size_ *= d
        if self.size_ <= 0:
            raise Exception("Invalid shape")

        distributed = dist.is_available() and dist.is_initialized() and local_world_size > 1
        # a segment of that name left over by someone else is an error, not something to adopt
        if capi.file_exist(name):
            raise Exception("File name is already exist")
        if distributed:
            dist.barrier(self.cur_group)

        if self.cur_rank == 0:
            self.ptr_, self.fd_ = capi.create_shared_mem(self.name, self.size_, self.pin_memory_)
            if distributed:
                dist.barrier(self.cur_group)
        else:
            if distributed:
                dist.barrier(self.cur_group)
            self.ptr_, self.fd_ = capi.open_shared_mem(self.name, self.size_, self.pin_memory_)

        self._shm_finalizer = weakref.finalize(self, _release, self.name, self.size_, self.ptr_,
                                               self.fd_, self.pin_memory_)
        self.tensor_ = capi.open_shared_tensor(self.ptr_, self.dtype_, list(self.shape_))

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
