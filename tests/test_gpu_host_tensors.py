"""Host tensor providers in front of the GPU operators: a numpy-written .npy opened as
DiskTensor (example/test_disk_tensor.py:6-14) and a single-process ShmTensor
(example/test_shm_tensor.py:10-19, include/shm_memory.h:6-39), made GPU-addressable and
read / written by uva_fetch, cache_fetch and uva_set; rows compared with numpy bit for bit.

Registering an existing mapping in place (pin_memory=True) depends on the driver: where it is
refused the providers raise a RuntimeError that names the staging copy (`pinned()` / `flush()`),
and leave no mapping or segment behind."""
import os
import uuid
import warnings

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def shmtensor(capi):
    import shmtensor_amd.shmtensor as pkg
    return pkg


def _bits(t):
    return t.detach().cpu().contiguous().numpy().view(np.uint8)


def _exercise(capi, provider, expect):
    """uva_fetch, cache_fetch and uva_set on the provider's staging copy; `expect` is the numpy
    array the provider was filled from (2-D). Returns the rows written by uva_set."""
    rng = np.random.default_rng(5)
    n = expect.shape[0]
    staged = provider.pinned()
    assert staged.is_pinned() and staged.shape == provider.tensor_.shape and staged.dtype == provider.tensor_.dtype
    assert provider.pinned() is staged                                   # made once, kept
    q = rng.integers(0, n, size=777)
    out = capi.uva_fetch(staged, torch.from_numpy(q).cuda())
    assert out.is_cuda and np.array_equal(_bits(out), expect[q].view(np.uint8))
    # cache a third of the rows; cached rows are made different from the host rows so that routing shows
    ids = rng.choice(n, size=n // 3, replace=False)
    cache_np = expect[ids].copy()
    cache_np.view(np.uint8)[...] ^= 0x5A
    hmap = capi.CUCOStaticHashmap(torch.from_numpy(ids).cuda(), torch.arange(ids.size).cuda(), 0.8)
    out = capi.cache_fetch(staged, torch.from_numpy(cache_np).cuda(), torch.from_numpy(q).cuda(), hmap)
    slot = {int(k): i for i, k in enumerate(ids)}
    want = np.stack([cache_np[slot[int(v)]] if int(v) in slot else expect[v] for v in q])
    assert np.array_equal(_bits(out), want.view(np.uint8))
    # GPU writes: land in the staging copy, reach the mapping with flush()
    w = rng.choice(n, size=50, replace=False)
    upd = rng.integers(-100, 100, size=(50,) + expect.shape[1:]).astype(expect.dtype)
    capi.uva_set(staged, torch.from_numpy(w).cuda(), torch.from_numpy(upd).cuda())
    torch.cuda.synchronize()
    assert np.array_equal(staged.numpy()[w], upd)
    assert np.array_equal(provider.tensor_.numpy()[w], expect[w])       # not yet in the mapping
    provider.flush()
    after = expect.copy()
    after[w] = upd
    assert np.array_equal(provider.tensor_.numpy(), after)
    return after


@pytest.mark.parametrize("dtype", [np.float32, np.float16, np.int64])
def test_disk_tensor_rows_through_the_gpu_operators(capi, shmtensor, tmp_path, dtype):
    rng = np.random.default_rng(1)
    data = (rng.standard_normal((3000, 24)) * 50).astype(dtype)
    path = str(tmp_path / "features.npy")
    np.save(path, data)
    t = shmtensor.DiskTensor(path)
    assert np.array_equal(t.tensor_.numpy(), data)
    after = _exercise(capi, t, data)
    del t                                                                # unmaps; the file keeps the GPU's writes
    import gc
    gc.collect()
    assert np.array_equal(np.load(path), after)


def test_shm_tensor_rows_through_the_gpu_operators(capi, shmtensor):
    name = "shmt_gpu_%s" % uuid.uuid4().hex[:12]
    rng = np.random.default_rng(2)
    data = rng.integers(-30000, 30000, size=(2048, 40)).astype(np.int16)
    t = shmtensor.ShmTensor(name, data.shape, 0, 1, None, torch.int16)
    try:
        t.tensor_.copy_(torch.from_numpy(data))
        after = _exercise(capi, t, data)
        ptr, fd = capi.open_shared_mem(name, data.nbytes)               # a second mapping sees the flushed rows
        other = capi.open_shared_tensor(ptr, torch.int16, list(data.shape))
        assert np.array_equal(other.numpy(), after)
        del other
        import mmap as _mmap  # noqa: F401  (the second mapping is released by the OS at exit; close its fd)
        os.close(fd)
    finally:
        del t
    import gc
    gc.collect()
    assert not capi.file_exist(name)


def test_pin_memory_true_works_or_names_the_alternative(capi, shmtensor, tmp_path):
    """In-place registration is the reference's route (include/shm_memory.h:19-21,
    src/mmap_tensor.cc:42-45). It is asked of the driver only on request (SHMT_HOST_REGISTER=1 /
    set_host_register(True)): without the request pin_memory=True raises the error that names the
    staging copy, makes no runtime call and leaves nothing behind; with it, the mapping itself is
    fetched from where the driver provides registration, and the same error is raised where not."""
    asked = os.environ.get("SHMT_HOST_REGISTER", "0") not in ("", "0")
    data = np.arange(600, dtype=np.float32).reshape(100, 6)
    path = str(tmp_path / "p.npy")
    np.save(path, data)
    idx = torch.tensor([0, 99, 5]).cuda()
    name = "shmt_pin_%s" % uuid.uuid4().hex[:12]
    if not asked:
        with pytest.raises(RuntimeError, match="switched off") as exc:
            shmtensor.DiskTensor(path, pin_memory=True)
        assert "pinned()" in str(exc.value) and "pin_memory=False" in str(exc.value)
        with pytest.raises(RuntimeError, match="switched off") as exc:
            shmtensor.ShmTensor(name, (100, 6), 0, 1, None, torch.float32, pin_memory=True)
        assert "pinned()" in str(exc.value)
        assert not capi.file_exist(name)                                 # the refused segment was removed
    else:
        try:
            t = shmtensor.DiskTensor(path, pin_memory=True)
        except RuntimeError as exc:
            assert "pinned()" in str(exc) and "pin_memory=False" in str(exc)
        else:
            assert np.array_equal(capi.uva_fetch(t.tensor_, idx).cpu().numpy(), data[[0, 99, 5]])
            del t
        try:
            s = shmtensor.ShmTensor(name, (100, 6), 0, 1, None, torch.float32, pin_memory=True)
        except RuntimeError as exc:
            assert "pinned()" in str(exc)
            assert not capi.file_exist(name)
        else:
            s.tensor_.copy_(torch.from_numpy(data))
            assert np.array_equal(capi.uva_fetch(s.tensor_, idx).cpu().numpy(), data[[0, 99, 5]])
            del s
    # an unpinned mapping handed to a kernel is an error, not a fault
    t = shmtensor.DiskTensor(path)
    with pytest.raises(RuntimeError, match="pin_memory"):
        capi.uva_fetch(t.tensor_, idx)
    torch.cuda.synchronize()


def test_pin_memory_keeps_torch_aliases_and_warns_about_foreign_memory(capi):
    """capi.pin_memory(t) (src/cache_feature_fetch.cu:6-9) makes t's memory GPU-addressable.
    Every torch tensor that shares t's storage keeps aliasing it afterwards; memory that torch
    does not own (a numpy array) cannot follow when the storage is re-homed, which is reported."""
    idx = torch.tensor([1, 3]).cuda()
    upd = torch.full((2, 4), 7.0).cuda()
    base = torch.arange(40, dtype=torch.float32).reshape(10, 4)
    alias = base.view(40)                                                # shares base's storage
    tail = base[5:]                                                      # a view with an offset
    with warnings.catch_warnings():
        warnings.simplefilter("error")                                   # torch-owned memory: no warning
        capi.pin_memory(base)
    capi.uva_set(base, idx, upd)
    torch.cuda.synchronize()
    assert torch.equal(base[[1, 3]], upd.cpu())
    assert torch.equal(alias.view(10, 4), base) and alias.data_ptr() == base.data_ptr()
    assert tail.data_ptr() == base.data_ptr() + 5 * 4 * 4
    capi.uva_set(tail, torch.tensor([0]).cuda(), upd[:1])                # the view is addressable too
    torch.cuda.synchronize()
    assert torch.equal(base[5], upd[0].cpu())

    arr = np.arange(40, dtype=np.float32).reshape(10, 4)
    t = torch.from_numpy(arr)
    before = t.data_ptr()
    with warnings.catch_warnings(record=True) as seen:
        warnings.simplefilter("always")
        capi.pin_memory(t)
    capi.uva_set(t, idx, upd)
    torch.cuda.synchronize()
    assert torch.equal(t[[1, 3]], upd.cpu())
    if t.data_ptr() == before:                                           # registered in place: numpy sees the writes
        assert np.array_equal(arr[[1, 3]], upd.cpu().numpy())
    else:                                                                # re-homed: said so, numpy keeps the old rows
        assert any("no longer aliases" in str(w.message) for w in seen)
        assert np.array_equal(arr, np.arange(40, dtype=np.float32).reshape(10, 4))
