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
