"""Backend string -> (tagCPUGPU, tag1D2D, tagHostDevice), as
pykeops/pykeops/common/get_options.py:14-140.  Every GPU backend is served: device-resident tensors travel as
device pointers (tagHostDevice = 1), host tensors and NumPy arrays as host pointers that the library stages
(tagHostDevice = 0).  "CPU" is rejected when the call is made: there is no CPU engine behind this front end."""

POSSIBLE_BACKENDS = [
    "auto", "CPU", "GPU", "GPU_1D", "GPU_1D_device", "GPU_1D_host", "GPU_2D", "GPU_2D_device", "GPU_2D_host",
]


def get_tag_backend(backend, variables):
    if backend not in POSSIBLE_BACKENDS:
        raise ValueError("Invalid backend. Should be one of ", POSSIBLE_BACKENDS)
    on_device = [bool(getattr(v, "is_cuda", False)) for v in variables]
    if any(on_device) and not all(on_device):
        raise ValueError("At least two input variables have different memory locations (Cpu/Gpu).")
    mem = 1 if all(on_device) and len(on_device) > 0 else 0
    parts = backend.split("_")
    dev = 1 if parts[0] in ("auto", "GPU") else 0
    grid = 1 if len(parts) > 1 and parts[1] == "2D" else 0
    if len(parts) == 3:
        mem = dict(host=0, device=1)[parts[2]]
    return dev, grid, mem
