"""Device facts and CU-partition helpers shared by the benchmark drivers (reference benchmarks/common.py)."""
import torch

from ..origami import hardware_for_device


def get_cu_info(device_id: int = 0):
    """(total_cus, num_xcds, cus_per_xcd) of a device (reference benchmarks/common.py:26-31)."""
    hw = hardware_for_device(device_id)
    return hw.N_CU, hw.NUM_XCD, hw.CU_per_L2


def build_balanced_hex_mask(remove_per_xcd: int, num_xcds: int, cus_per_xcd: int) -> str:
    """Hex CU mask that switches off the first ``remove_per_xcd`` CUs of every XCD; CU bit ``i`` belongs
    to XCD ``i % num_xcds`` (reference benchmarks/common.py:34-45).  Empty string: nothing removed."""
    if remove_per_xcd == 0:
        return ""
    keep = 0
    for bit in range(num_xcds * cus_per_xcd):
        if bit // num_xcds >= remove_per_xcd:
            keep |= 1 << bit
    return f"0x{keep:x}"


def workgroup_mask(total_cus: int, active_cus: int, device) -> torch.Tensor:
    """int32[total_cus] work-stealing mask with the first ``active_cus`` workgroups enabled
    (reference config.py:117-121)."""
    mask = torch.ones(total_cus, dtype=torch.int32, device=device)
    mask[active_cus:] = 0
    return mask
