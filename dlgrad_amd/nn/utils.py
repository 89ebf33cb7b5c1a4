"""Parameter discovery by walking an object graph, in the order dlgrad/nn/utils.py:10-52
visits it: attributes in definition order, dict values, list/tuple elements; every Tensor
found is returned."""
from dlgrad_amd.tensor import Tensor


def _walk(o, path: str, visit, skip_private: bool) -> None:
    if isinstance(o, Tensor):
        visit(path, o)
        return
    if isinstance(o, dict):
        items = o.items()
    elif isinstance(o, (list, tuple)):
        items = enumerate(o)
    elif hasattr(o, "__dict__"):
        items = ((k, v) for k, v in vars(o).items() if not (skip_private and str(k).startswith("_")))
    else:
        return
    for k, v in items:
        _walk(v, f"{path}.{k}" if path else f"{k}", visit, skip_private)


def get_state_dict(obj, prefix: str = "") -> dict:
    """{'path.to.tensor': Tensor}; attributes starting with '_' are skipped."""
    out: dict = {}
    _walk(obj, prefix, out.__setitem__, True)
    return out


def get_parameters(obj) -> list:
    out: list = []
    _walk(obj, "", lambda _p, t: out.append(t), False)
    return out


# ---- checkpoints ---------------------------------------------------------------------------------
# The safetensors layout dlgrad/nn/utils.py:54-132 writes and reads: u64 little-endian header
# size, a JSON header {name: {"dtype": "F32", "shape": [...], "data_offsets": [begin, end]}}
# with offsets relative to the end of the header, then the raw little-endian fp32 data in
# header order.  Names are the attribute paths of get_state_dict.  Tensors on the hip device
# are staged through the host one at a time (D2H on save, H2D into the existing allocation
# on load), so a file written from one device loads on the other and peak host memory is
# one tensor, not the model.

def save_model(model, path: str) -> int:
    """Writes every Tensor of `model` to `path`; returns how many were written."""
    import json
    import struct
    state = get_state_dict(model)
    header, offset = {}, 0
    for name, t in state.items():
        header[name] = {"dtype": "F32", "shape": list(t.shape), "data_offsets": [offset, offset + t.nbytes]}
        offset += t.nbytes
    blob = json.dumps(header).encode("utf-8")
    blob += b" " * (-len(blob) % 8)                          # keeps the data 8-byte aligned; JSON ignores it
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for t in state.values():
            f.write(t.tobytes())
    print(f"Saved {len(state)} tensors to {path}")
    return len(state)


def load_model(model, path: str) -> int:
    """Copies the tensors of a safetensors file into the model's existing Tensors (same
    allocation, so captured graphs and optimizer state keep pointing at them).  Names the
    model does not have, shapes that differ and non-F32 entries are reported and skipped,
    as the reference does; returns how many tensors were loaded."""
    import json
    import os
    import struct

    import numpy as np
    if not os.path.exists(path):
        raise FileNotFoundError(f"Checkpoint {path} not found")
    current = get_state_dict(model)
    size = os.path.getsize(path)
    with open(path, "rb") as f:
        head = f.read(8)
        if len(head) != 8:
            raise ValueError(f"{path}: too short for a safetensors header")
        (hsize,) = struct.unpack("<Q", head)
        if hsize > size - 8:
            raise ValueError(f"{path}: header of {hsize} bytes exceeds the file")
        header = json.loads(f.read(hsize))
    base, loaded = 8 + hsize, 0
    for name, meta in header.items():
        if name == "__metadata__":
            continue
        if name not in current:
            print(f"Warning: {name} found in file but not in model. Skipping.")
            continue
        t = current[name]
        if meta.get("dtype") != "F32":
            print(f"Unsupported dtype {meta.get('dtype')} for {name}. Skipping.")
            continue
        if tuple(t.shape) != tuple(meta["shape"]):
            print(f"Shape mismatch for {name}: Model {t.shape} vs File {tuple(meta['shape'])}")
            continue
        begin, end = meta["data_offsets"]
        if end - begin != t.nbytes or base + end > size:
            raise ValueError(f"{path}: {name} claims bytes {begin}:{end}, the tensor needs {t.nbytes}")
        arr = np.fromfile(path, dtype="<f4", count=t.numel, offset=base + begin)
        t.data.upload_(arr)
        loaded += 1
    print(f"Successfully loaded {loaded} tensors.")
    return loaded
