"""dlgrad's Tensor/ops API with an MI355X-native `device="hip"` kernel backend."""
from dlgrad_amd.device import Device  # noqa: F401
from dlgrad_amd.runtime import hip as _hip_runtime  # registers every (op, Device.HIP) entry  # noqa: F401
