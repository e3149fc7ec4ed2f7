"""Mirror of the reference's `shmtensor` Python package
(python/shmtensor/__init__.py:1-4): host tensor providers and the GPU
sampling dataloader on top of the `ShmTensorLib` operators."""
from .. import install_aliases as _install_aliases

capi = _install_aliases()

from .disk_tensor import DiskTensor  # noqa: E402
from .shm_tensor import ShmTensor  # noqa: E402
from .sampling import GPUSamplingDataloader  # noqa: E402

__all__ = ["DiskTensor", "ShmTensor", "GPUSamplingDataloader", "capi"]
