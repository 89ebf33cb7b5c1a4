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


def read_idx(path: str, images: bool, magic_number: int) -> np.ndarray:
    """uint8 array (count, rows*cols) or (count, 1) from an idx file, plain or gzip."""
    opener = gzip.open if path.endswith(".gz") else open
    with opener(path, "rb") as f:
        raw = f.read()
    nhead = 16 if images else 8
    if len(raw) < nhead:
        raise ValueError(f"{path}: shorter than an idx header")
    fields = struct.unpack(">" + "I" * (nhead // 4), raw[:nhead])
    if fields[0] != magic_number:
        raise ValueError(f"{path}: invalid magic number {fields[0]}, expected {magic_number}")
    count = fields[1]
    per = fields[2] * fields[3] if images else 1
    if len(raw) - nhead < count * per:
        raise ValueError(f"{path}: read error or unexpected EOF ({len(raw) - nhead} data bytes, "
                         f"{count * per} announced)")
    return np.frombuffer(raw, dtype=np.uint8, count=count * per, offset=nhead).reshape(count, per)


def _find(root: str, name: str) -> str:
    for cand in (os.path.join(root, name), os.path.join(root, name + ".gz")):
        if os.path.exists(cand):
            return cand
    raise FileNotFoundError(f"{name}[.gz] not found in {root}: this build does not download; place the MNIST idx files there")


def mnist(device: Device = Device.CPU, root: str | None = None) -> list[Tensor]:
    """[train_images, train_labels, test_images, test_labels]."""
    root = root or os.path.join(CACHE_DIR, "downloads")
    out = []
    for name, images, magic in MNIST_FILES:
        data = read_idx(_find(root, name), images, magic)
        out.append(Tensor(Buffer.from_u8(data, device), requires_grad=False, device=device))
    return out
