"""save_model / load_model: the safetensors layout of dlgrad/nn/utils.py:54-132.

The format is pinned from outside by the `safetensors` library itself: a file written here
must load there with equal names, shapes and bits, and a file written there (with a
__metadata__ entry and its own header padding) must load here.  On the GPU the same files
cross devices: written from hip, read on the C oracle's cpu device and back, bit-exact, into
the tensors' existing allocations."""
import json
import os
import struct

import numpy as np
import pytest
from safetensors.numpy import load_file, save_file

import oracle.cpu_runtime  # noqa: F401  (test infrastructure: registers the cpu device)
from dlgrad_amd import Tensor, nn
from dlgrad_amd.runtime import hip
from examples import gpt as G

CFG = dict(vocab_size=20, block_size=12, n_layer=2, n_head=2, n_embd=16, batch_size=1)


def make(device, seed):
    m = G.GPT(G.GPTConfig(device=device, **CFG))
    G.init_weights_(m, seed)
    return m


def values(m):
    return {k: t.numpy() for k, t in nn.utils.get_state_dict(m).items()}


def test_written_file_is_read_by_the_safetensors_library(tmp_path):
    m = make("cpu", 0)
    path = str(tmp_path / "m.safetensors")
    assert nn.utils.save_model(m, path) == 20
    theirs, ours = load_file(path), values(m)
    assert list(theirs) and set(theirs) == set(ours)
    for k in ours:
        assert theirs[k].dtype == np.float32 and theirs[k].shape == ours[k].shape
        np.testing.assert_array_equal(theirs[k], ours[k])
    with open(path, "rb") as f:                                   # layout: u64 size, JSON, data in header order
        (hsize,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(hsize))
    assert list(header) == list(nn.utils.get_state_dict(m))
    first = header["wte.weight"]
    assert first == {"dtype": "F32", "shape": [20, 16], "data_offsets": [0, 20 * 16 * 4]}
    assert os.path.getsize(path) == 8 + hsize + sum(v.nbytes for v in ours.values())


def test_file_from_the_safetensors_library_loads_in_place(tmp_path):
    src, dst = make("cpu", 0), make("cpu", 1)
    path = str(tmp_path / "lib.safetensors")
    save_file({k: v * 2 for k, v in values(src).items()}, path, metadata={"written_by": "safetensors"})
    before = {k: t.data.ptr for k, t in nn.utils.get_state_dict(dst).items()}
    assert nn.utils.load_model(dst, path) == 20
    for k, t in nn.utils.get_state_dict(dst).items():
        assert t.data.ptr is before[k]                              # same allocation, new contents
        np.testing.assert_array_equal(t.numpy(), values(src)[k] * 2)


def test_unknown_names_wrong_shapes_and_other_dtypes_are_skipped(tmp_path, capsys):
    dst = make("cpu", 1)
    keep = values(dst)
    good = values(make("cpu", 0))
    path = str(tmp_path / "odd.safetensors")
    save_file({"wte.weight": good["wte.weight"], "not.in.model": np.zeros(3, np.float32),
               "wpe.weight": np.zeros((5, 5), np.float32), "ln_f.weight": np.ones((1, 16), np.float16)}, path)
    assert nn.utils.load_model(dst, path) == 1
    out = capsys.readouterr().out
    assert "not.in.model found in file but not in model" in out and "Shape mismatch for wpe.weight" in out
    got = values(dst)
    np.testing.assert_array_equal(got["wte.weight"], good["wte.weight"])
    np.testing.assert_array_equal(got["wpe.weight"], keep["wpe.weight"])
    np.testing.assert_array_equal(got["ln_f.weight"], keep["ln_f.weight"])


def test_missing_and_damaged_files_raise(tmp_path):
    m = make("cpu", 0)
    with pytest.raises(FileNotFoundError):
        nn.utils.load_model(m, str(tmp_path / "absent.safetensors"))
    path = str(tmp_path / "m.safetensors")
    nn.utils.save_model(m, path)
    data = open(path, "rb").read()
    short = str(tmp_path / "short.safetensors")
    open(short, "wb").write(data[:-64])                            # last tensor cut off
    with pytest.raises(ValueError):
        nn.utils.load_model(m, short)
    open(short, "wb").write(data[:5])
    with pytest.raises(ValueError):
        nn.utils.load_model(m, short)
    open(short, "wb").write(struct.pack("<Q", 1 << 40) + data[8:])
    with pytest.raises(ValueError):
        nn.utils.load_model(m, short)


@pytest.mark.gpu
def test_checkpoints_cross_devices_bit_exactly(tmp_path):
    if not (hip.available() or hip.COMPILE_ONLY):
        pytest.skip("no HIP device")
    on_hip, on_cpu = make("hip", 0), make("cpu", 1)
    path = str(tmp_path / "hip.safetensors")
    nn.utils.save_model(on_hip, path)
    assert nn.utils.load_model(on_cpu, path) == 20
    back = make("hip", 2)
    addrs = {k: t.data.ptr.addr for k, t in nn.utils.get_state_dict(back).items()}
    path2 = str(tmp_path / "cpu.safetensors")
    nn.utils.save_model(on_cpu, path2)
    assert nn.utils.load_model(back, path2) == 20
    assert {k: t.data.ptr.addr for k, t in nn.utils.get_state_dict(back).items()} == addrs
    if hip.COMPILE_ONLY:
        return
    want = values(make("cpu", 0))
    for m in (on_hip, on_cpu, back):
        got = values(m)
        for k in want:
            np.testing.assert_array_equal(got[k], want[k], err_msg=k)
    ids = Tensor(np.array([[1, 2, 3, 4]], np.float32), device="hip")
    a, _ = on_hip(ids)
    b, _ = back(ids)
    np.testing.assert_array_equal(a.numpy(), b.numpy())               # same weights, same kernels, same logits
