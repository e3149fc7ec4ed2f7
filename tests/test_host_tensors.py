"""Host tensor providers (DiskTensor, ShmTensor): the semantics of
example/test_disk_tensor.py:6-14 and example/test_shm_tensor.py:10-19, on the CPU."""
import gc
import os
import uuid

import numpy as np
import pytest
import torch


@pytest.fixture(scope="module")
def shmtensor(capi):
    import shmtensor as pkg      # registered by install_aliases()
    return pkg


@pytest.mark.parametrize("dtype", [np.float64, np.float32, np.float16, np.int64, np.int32, np.int16, np.int8, np.uint8])
def test_disk_tensor_matches_numpy(shmtensor, tmp_path, dtype):
    a = (np.random.default_rng(0).standard_normal((2, 3, 4)) * 50).astype(dtype)
    f = str(tmp_path / "a.npy")
    np.save(f, a)
    t = shmtensor.DiskTensor(f)
    assert t.shape == (2, 3, 4) and t.dtype == torch.from_numpy(a).dtype and t.device.type == "cpu"
    assert torch.equal(t.tensor_, torch.from_numpy(a))


def test_disk_tensor_is_a_writable_mapping(shmtensor, tmp_path):
    f = str(tmp_path / "b.npy")
    np.save(f, np.arange(1000, dtype=np.int64))
    t = shmtensor.DiskTensor(f)
    t.tensor_[7] = -5
    del t
    gc.collect()
    assert np.load(f)[7] == -5


def test_disk_tensor_large_header_and_errors(shmtensor, tmp_path, capi):
    # a shape with many dimensions still parses; version-2 headers (4-byte length) too
    a = np.zeros((1, 2, 1, 3, 1, 2, 1, 1, 2), dtype=np.float32)
    f = str(tmp_path / "c.npy")
    np.save(f, a)
    assert tuple(shmtensor.DiskTensor(f).shape) == a.shape
    f2 = str(tmp_path / "v2.npy")
    with open(f2, "wb") as fh:
        np.lib.format.write_array_header_2_0(fh, {"descr": "<i4", "fortran_order": False, "shape": (5,)})
        fh.write(np.arange(5, dtype=np.int32).tobytes())
    assert shmtensor.DiskTensor(f2).tensor_.tolist() == [0, 1, 2, 3, 4]
    np.save(str(tmp_path / "f.npy"), np.asfortranarray(np.ones((3, 4))))
    with pytest.raises(RuntimeError, match="fortran"):
        shmtensor.DiskTensor(str(tmp_path / "f.npy"))
    np.save(str(tmp_path / "c64.npy"), np.ones(3, dtype=np.complex64))
    with pytest.raises(RuntimeError, match="dtype"):
        shmtensor.DiskTensor(str(tmp_path / "c64.npy"))
    with pytest.raises(FileNotFoundError):
        shmtensor.DiskTensor(str(tmp_path / "missing.npy"))
    other = str(tmp_path / "raw.bin")
    open(other, "wb").write(b"0123")
    with pytest.raises(ValueError):
        shmtensor.DiskTensor(other)


def test_shm_tensor_single_process(shmtensor, capi):
    name = "shmt_" + uuid.uuid4().hex[:12]
    t = shmtensor.ShmTensor(name, (2, 3, 4), 0, 1, None, torch.int16)
    assert t.shape == (2, 3, 4) and t.dtype == torch.int16
    t.tensor_[:] = 1000
    assert capi.file_exist(name)
    ptr, fd = capi.open_shared_mem(name, 48)                 # a second mapping sees the data
    other = capi.open_shared_tensor(ptr, torch.int16, [2, 3, 4])
    assert int(other.sum()) == 24000
    with pytest.raises(Exception, match="already exist"):    # python/shmtensor/shm_tensor.py:44-45
        shmtensor.ShmTensor(name, (2,), 0, 1)
    with pytest.raises(Exception, match="Invalid shape"):
        shmtensor.ShmTensor(name + "x", (0, 3), 0, 1)
    del t, other
    gc.collect()
    assert not capi.file_exist(name)                         # released by the finalizer


def _shm_worker(rank, world, name, port, results):
    import torch.distributed as dist
    os.environ.update(MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port))
    dist.init_process_group("gloo", rank=rank, world_size=world)
    import shmtensor_amd
    shmtensor_amd.install_aliases()
    from shmtensor import ShmTensor
    t = ShmTensor(name, (2, 3, 4), rank, world, None, torch.int16)
    if rank == 0:
        t.tensor_[:] = 1000
    dist.barrier()
    results[rank] = int(t.tensor_.sum())
    dist.barrier()
    del t
    dist.destroy_process_group()


def test_shm_tensor_two_ranks_gloo():
    """rank 0 writes, rank 1 reads after a barrier (example/test_shm_tensor.py:10-19)."""
    import torch.multiprocessing as mp
    name = "shmt_" + uuid.uuid4().hex[:12]
    ctx = mp.get_context("spawn")
    results = ctx.Manager().dict()
    port = 29500 + os.getpid() % 2000
    procs = [ctx.Process(target=_shm_worker, args=(r, 2, name, port, results)) for r in range(2)]
    for p in procs:
        p.start()
    for p in procs:
        p.join(120)
        assert p.exitcode == 0
    assert dict(results) == {0: 24000, 1: 24000}


def test_pin_memory_true_needs_the_opt_in(shmtensor, capi, tmp_path):
    """Registering an existing mapping in place is only asked of the driver on request
    (set_host_register(True) / SHMT_HOST_REGISTER=1). Without it pin_memory=True raises an error
    that names the staging copy, before any runtime call (so this runs without a GPU), and takes
    the mapping and the segment it created down again."""
    capi.set_host_register(False)
    f = str(tmp_path / "p.npy")
    np.save(f, np.arange(12, dtype=np.float32))
    with pytest.raises(RuntimeError, match="switched off") as exc:
        shmtensor.DiskTensor(f, pin_memory=True)
    assert "pinned()" in str(exc.value) and "set_host_register" in str(exc.value)
    name = "shmt_cpu_pin_%s" % uuid.uuid4().hex[:12]
    with pytest.raises(RuntimeError, match="switched off"):
        shmtensor.ShmTensor(name, (4, 3), 0, 1, None, torch.float32, pin_memory=True)
    assert not capi.file_exist(name)
    assert shmtensor.DiskTensor(f).tensor_.tolist() == list(range(12))      # the file is still fine
