"""Argument checking of the public entry points (mirrors reference src/trigrad/util.py:1-16:
TypeError for a wrong device or dtype, ValueError for a wrong shape, same messages)."""


def create_check(default_device, default_dtype):
    """default_dtype: a torch dtype, or a function returning the dtype expected at the time of the call."""
    def check_tensor(tensor, name, shape=None, dtype=None, device=None):
        if not isinstance(shape, tuple):
            shape = (shape,)
        expected_device = default_device if device is None else device
        if tensor.device.type != expected_device:
            raise TypeError(f"{name} must be on {expected_device}, but got {tensor.device.type}")
        expected_dtype = (default_dtype() if callable(default_dtype) else default_dtype) if dtype is None else dtype
        if tensor.dtype != expected_dtype:
            raise TypeError(f"{name} must be of type {expected_dtype}, but got {tensor.dtype}")
        if shape is not None and tensor.shape != shape:
            raise ValueError(f"{name} must be of shape {shape}, but got {tensor.shape}")

    return check_tensor
