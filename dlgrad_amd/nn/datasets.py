"""MNIST from the four idx files (dlgrad/nn/datasets.py:9-39 with the loaders of
cpu_kernel.py:876-1010): big-endian header -- magic 2051, count, rows, cols for images, magic
2049, count for labels -- then one unsigned byte per pixel or label.  Tensors come back as
fp32, not normalised: images (count, rows*cols), labels (count, 1).

The reference downloads the files; nothing here touches the network.  Put the files (plain
or .gz) into `root`, by default the `downloads` folder of the kernel cache directory, which is
where the reference's fetch() leaves them.  On the hip device the bytes are uploaded as bytes
and widened to fp32 by a kernel."""
from __future__ import annotations

import gzip
import os
import struct

import numpy as np

from dlgrad_amd.buffer import Buffer
from dlgrad_amd.device import Device
from dlgrad_amd.helpers import CACHE_DIR
from dlgrad_amd.tensor import Tensor

MNIST_FILES = (
    ("train-images-idx3-ubyte", True, 2051),
    ("train-labels-idx1-ubyte", False, 2049),
    ("t10k-images-idx3-ubyte", True, 2051),
    ("t10k-labels-idx1-ubyte", False, 2049),
)


def read_idx(path: str, images: bool, magic_number: int, empty=np.empty) -> np.ndarray:
    """uint8 array (count, rows*cols) or (count, 1) from an idx file, plain or gzip.  `empty`
    allocates the result (shape, dtype) -- page-locked memory when the bytes go to a GPU."""
    opener = gzip.open if path.endswith(".gz") else open
    nhead = 16 if images else 8
    with opener(path, "rb") as f:
        head = f.read(nhead)
        if len(head) < nhead:
            raise ValueError(f"{path}: shorter than an idx header")
        fields = struct.unpack(">" + "I" * (nhead // 4), head)
        if fields[0] != magic_number:
            raise ValueError(f"{path}: invalid magic number {fields[0]}, expected {magic_number}")
        count = fields[1]
        per = fields[2] * fields[3] if images else 1
        out = empty((count, per), np.uint8)
        view = memoryview(out).cast("B") if out.size else memoryview(b"")
        got = 0
        while got < len(view):
            n = f.readinto(view[got:])
            if not n:
                raise ValueError(f"{path}: read error or unexpected EOF ({got} data bytes, {len(view)} announced)")
            got += n
    return out


def _find(root: str, name: str) -> str:
    for cand in (os.path.join(root, name), os.path.join(root, name + ".gz")):
        if os.path.exists(cand):
            return cand
    raise FileNotFoundError(f"{name}[.gz] not found in {root}: this build does not download; place the MNIST idx files there")


def mnist(device: Device = Device.CPU, root: str | None = None) -> list[Tensor]:
    """[train_images, train_labels, test_images, test_labels]."""
    root = root or os.path.join(CACHE_DIR, "downloads")
    out = []
    from dlgrad_amd.device import as_device
    on_hip = as_device(device) is Device.HIP
    if on_hip:
        from dlgrad_amd.runtime import hip
    for name, images, magic in MNIST_FILES:
        # hip: file -> page-locked buffer -> DMA -> widened to fp32 by a kernel; the upload is only enqueued
        data = read_idx(_find(root, name), images, magic, empty=hip.pinned_empty if on_hip else np.empty)
        out.append(Tensor(Buffer.from_u8(data, device), requires_grad=False, device=device))
    if on_hip:
        hip.lib().sync()                   # the staging buffers are released when `data` goes out of scope
    return out
