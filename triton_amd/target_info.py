"""What the target is (target_info.py of the reference, which asks the Triton runtime): here the answer comes from
the HIP device itself, and the only target the kernels are built for is gfx950 (CDNA4)."""
import functools

import torch

__all__ = ["cuda_capability_geq", "get_cdna_version", "get_rdna_version", "has_tma_gather", "has_native_mxfp", "is_cuda",
           "is_hip", "is_hip_cdna3", "is_hip_cdna4", "is_hip_gfx1250", "num_sms"]


@functools.lru_cache(maxsize=None)
def _arch():
    """Architecture name of device 0 without its feature suffixes ('gfx950'), or '' without a HIP device."""
    if torch.version.hip is None or not torch.cuda.is_available():
        return ""
    return torch.cuda.get_device_properties(0).gcnArchName.split(":")[0]


def is_hip():
    return torch.version.hip is not None


def is_cuda():
    return False


def cuda_capability_geq(major, minor=0):
    return False


def is_hip_cdna3():
    return _arch() == "gfx942"


def is_hip_cdna4():
    return _arch() == "gfx950"


def is_hip_gfx1250():
    return _arch() == "gfx1250"


def get_cdna_version():
    """3 (gfx942), 4 (gfx950), or -1 for anything else (target_info.py:28-43 of the reference)."""
    return {"gfx942": 3, "gfx950": 4}.get(_arch(), -1)


def get_rdna_version():
    a = _arch()
    if a.startswith("gfx11"):
        return 3
    if a.startswith("gfx12") and not a.startswith("gfx125"):
        return 4
    return -1


def has_tma_gather():
    return False


def has_native_mxfp():
    """The reference answers for Blackwell's tensor-memory MMA only (target_info.py:69-71)."""
    return False


def num_sms():
    return torch.cuda.get_device_properties(0).multi_processor_count
