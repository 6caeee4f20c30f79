"""Target predicates (mirrors `triton_kernels/target_info.py`); this build targets gfx950 only."""
import torch


def is_hip():
    return True


def is_cuda():
    return False


def is_hip_cdna4():
    return True


def is_hip_cdna3():
    return False


def get_cdna_version():
    return 4


def cuda_capability_geq(major, minor=0):
    return False


def has_native_mxfp():
    return True


def num_sms():
    if torch.cuda.is_available():
        return torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count
    return 256
