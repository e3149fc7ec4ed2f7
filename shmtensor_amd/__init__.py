"""MI355X-native GPU-cache hot path behind the ShmTensor operator surface.

    import shmtensor_amd
    capi = shmtensor_amd.ShmTensorLib      # or: shmtensor_amd.install_aliases();
                                           #     import ShmTensorLib as capi

`ShmTensorLib` is the compiled operator module (pybind11 over the C ABI of
libshmt.so); it is loaded on first use so that `python -m shmtensor_amd.build`
can run before anything is built. There is no fallback implementation: if the
native module is missing the import fails.
"""
import importlib
import sys

_MODULE = None


def _load_module():
    global _MODULE
    if _MODULE is None:
        import torch  # noqa: F401  (ShmTensorLib links against libtorch)
        if "ShmTensorLib" in sys.modules:
            # already imported top-level (this directory on PYTHONPATH): one
            # extension module must not be initialised twice
            _MODULE = sys.modules["ShmTensorLib"]
            return _MODULE
        try:
            _MODULE = importlib.import_module("shmtensor_amd.ShmTensorLib")
        except ImportError as exc:
            raise ImportError(
                "shmtensor_amd.ShmTensorLib is not built "
                "(run `python -m shmtensor_amd.build`): %s" % exc) from exc
    return _MODULE


_ALIASING = False


def install_aliases():
    """Register the operator module and the Python package under the names the
    reference scripts use (`import ShmTensorLib as capi`, `from shmtensor import
    GPUSamplingDataloader`). Returns the operator module."""
    global _ALIASING
    mod = _load_module()
    sys.modules.setdefault("ShmTensorLib", mod)
    if not _ALIASING and "shmtensor" not in sys.modules:
        _ALIASING = True
        try:
            sys.modules.setdefault("shmtensor", importlib.import_module("shmtensor_amd.shmtensor"))
        finally:
            _ALIASING = False
    return mod


def __getattr__(name):
    if name in ("ShmTensorLib", "capi"):
        return _load_module()
    raise AttributeError("module 'shmtensor_amd' has no attribute %r" % name)
