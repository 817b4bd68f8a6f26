"""Device naming helpers (reference: spio/util/device_info.py:6-37)."""

import torch


def get_device_ordinal(device) -> int:
    """Ordinal of a torch device or device string; 0 when unspecified."""
    idx = torch.device(device).index
    return 0 if idx is None else idx


def get_formatted_device_name(device) -> str:
    """Device name usable in file names, e.g. amd_instinct_mi355x."""
    name = torch.cuda.get_device_name(torch.device(device))
    return name.replace(" ", "_").replace("(", "_").replace(")", "_").lower()


def get_formatted_arch(device) -> str:
    """GCN architecture of the device without feature suffixes, e.g. gfx950."""
    props = torch.cuda.get_device_properties(torch.device(device))
    return props.gcnArchName.split(":")[0]
