"""Device queries (reference ``gpu_utils.py:4-8``)."""
from typing import Optional

import torch


def get_gpu_sm_count(device: Optional[torch.device] = None):
    """Compute-unit count of ``device`` (the current device by default; 256 on MI355X)."""
    assert torch.cuda.device_count() > 0
    if device is None:
        device = torch.device("cuda", torch.cuda.current_device())
    return torch.cuda.get_device_properties(device).multi_processor_count
