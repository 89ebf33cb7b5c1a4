"""dlgrad's Tensor/ops API with an MI355X-native `device="hip"` kernel backend."""
from dlgrad_amd.device import Device  # noqa: F401
from dlgrad_amd.runtime import hip as _hip_runtime  # registers every (op, Device.HIP) entry  # noqa: F401
from dlgrad_amd.tensor import Tensor  # noqa: F401
from dlgrad_amd import nn  # noqa: F401


def manual_seed(seed: int) -> None:
    """Seeds the PCG32 streams behind `uniform` (and so dropout and layer init) on the hip device."""
    _hip_runtime.HIP.manual_seed(seed)
