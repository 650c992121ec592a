"""Small helpers (reference: ss_conv/utils/utils.py)."""
import torch


def Rs2dim(Rs):
    """Channel count of a list of (multiplicity, order) pairs: sum m * (2l + 1)."""
    return sum((2 * l + 1) * m for m, l in Rs)


def calculate_fan_in(channel_in, kernel_size):
    return channel_in * kernel_size.prod()


class torch_default_dtype:
    """Context manager that switches torch's default dtype."""

    def __init__(self, dtype):
        self.saved_dtype = None
        self.dtype = dtype

    def __enter__(self):
        self.saved_dtype = torch.get_default_dtype()
        torch.set_default_dtype(self.dtype)

    def __exit__(self, exc_type, exc_value, traceback):
        torch.set_default_dtype(self.saved_dtype)
