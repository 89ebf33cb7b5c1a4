"""Device names of the dispatch table.

Mirrors dlgrad/device.py:4-13 and adds HIP beside CPU and METAL.  Only
HIP has a runtime in this package; the (op, Device.CPU) column is filled by
whoever imports a CPU runtime (the test oracle does), METAL by nobody here.
"""
from enum import Enum, auto


class Device(Enum):
    __hash__ = object.__hash__          # members are singletons; this keys the dispatch table on every op

    CPU = auto()
    METAL = auto()
    HIP = auto()

    @staticmethod
    def from_str(d: str) -> "Device":
        # Same observable behaviour as the reference for a bad name: a message
        # on stdout and None as the result (dlgrad/device.py:10-13).
        member = Device.__members__.get(str(d).upper())
        if member is None:
            print(f"Invalid device: {d}")
        return member


def as_device(d) -> "Device":
    """Accepts a Device, a name, or None (meaning CPU, the reference default)."""
    if d is None:
        return Device.CPU
    return d if isinstance(d, Device) else Device.from_str(d)
