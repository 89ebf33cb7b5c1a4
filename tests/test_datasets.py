"""MNIST idx loading (dlgrad/nn/datasets.py:9-39): header parsing, shapes, uint8 -> fp32, errors.
The files are synthetic, written by the test in the idx format (big-endian magic / count /
rows / cols, then bytes); the real files need a download, which does not exist here."""
import gzip
import struct

import numpy as np
import pytest

import oracle.cpu_runtime  # noqa: F401  (test infrastructure: registers the cpu device)
from dlgrad_amd.buffer import Buffer
from dlgrad_amd.device import Device
from dlgrad_amd.nn import datasets
from dlgrad_amd.runtime import hip

RNG = np.random.default_rng(5)


def write_set(root, n_train=37, n_test=11, rows=28, cols=28, gz=()):
    arrays = {}
    for name, images, magic in datasets.MNIST_FILES:
        n = n_train if name.startswith("train") else n_test
        if images:
            data = RNG.integers(0, 256, (n, rows * cols), dtype=np.uint8)
            blob = struct.pack(">IIII", magic, n, rows, cols) + data.tobytes()
        else:
            data = RNG.integers(0, 10, (n, 1), dtype=np.uint8)
            blob = struct.pack(">II", magic, n) + data.tobytes()
        arrays[name] = data
        if name in gz:
            with gzip.open(root / (name + ".gz"), "wb") as f:
                f.write(blob)
        else:
            (root / name).write_bytes(blob)
    return arrays


def test_mnist_on_the_cpu_device(tmp_path):
    arrays = write_set(tmp_path, gz=("t10k-images-idx3-ubyte",))
    tensors = datasets.mnist(device="cpu", root=str(tmp_path))
    assert [t.shape for t in tensors] == [(37, 784), (37, 1), (11, 784), (11, 1)]
    for t, (name, _, _) in zip(tensors, datasets.MNIST_FILES):
        assert not t.requires_grad
        np.testing.assert_array_equal(t.numpy(), arrays[name].astype(np.float32))       # not normalised


def test_idx_errors(tmp_path):
    write_set(tmp_path)
    with pytest.raises(ValueError, match="magic"):
        datasets.read_idx(str(tmp_path / "train-images-idx3-ubyte"), False, 2049)
    p = tmp_path / "cut"
    p.write_bytes((tmp_path / "train-images-idx3-ubyte").read_bytes()[:-5])
    with pytest.raises(ValueError, match="EOF"):
        datasets.read_idx(str(p), True, 2051)
    p.write_bytes(b"\x00\x00")
    with pytest.raises(ValueError, match="header"):
        datasets.read_idx(str(p), True, 2051)
    (tmp_path / "t10k-labels-idx1-ubyte").unlink()
    with pytest.raises(FileNotFoundError, match="does not download"):
        datasets.mnist(device="cpu", root=str(tmp_path))


@pytest.mark.gpu
def test_mnist_bytes_are_widened_on_the_hip_device(tmp_path):
    if not (hip.available() or hip.COMPILE_ONLY):
        pytest.skip("no HIP device")
    arrays = write_set(tmp_path, n_train=1001, n_test=3, rows=5, cols=3, gz=("train-labels-idx1-ubyte",))
    tensors = datasets.mnist(device="hip", root=str(tmp_path))
    assert [t.shape for t in tensors] == [(1001, 15), (1001, 1), (3, 15), (3, 1)]      # 15015, 1001, 45, 3 bytes: tails of 3, 1, 1, 3
    if hip.COMPILE_ONLY:
        return
    for t, (name, _, _) in zip(tensors, datasets.MNIST_FILES):
        np.testing.assert_array_equal(t.numpy(), arrays[name].astype(np.float32))
    big = RNG.integers(0, 256, (60000, 784), dtype=np.uint8)                            # the real training-set size
    np.testing.assert_array_equal(Buffer.from_u8(big, Device.HIP).numpy(), big.astype(np.float32))
    batch = tensors[0][128:256]                                                         # a leading-dim slice is a view
    np.testing.assert_array_equal(batch.numpy(), arrays["train-images-idx3-ubyte"][128:256].astype(np.float32))
