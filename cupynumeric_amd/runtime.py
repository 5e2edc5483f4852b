"""Device plumbing: which GPU, which stream, raw device buffers.

PyTorch (ROCm) is used only as the owner of device memory and streams -- the part Legate's
runtime plays for the reference (`cupynumeric/runtime.py:428-445` creates thunks over Legate
stores; `src/cupynumeric/sort/sort.cu:1822` takes the task stream).  No torch operator takes
part in a sort.
"""
from __future__ import annotations

import os
from typing import TYPE_CHECKING

import numpy as np

if TYPE_CHECKING:
    import torch


class Runtime:
    """Process-wide state: device, settings."""

    def __init__(self) -> None:
        # read back the device status word after every sort (costs one stream sync)
        self.check_status = os.environ.get("CUPYNUMERIC_AMD_CHECK_STATUS", "1") != "0"
        self._torch = None

    @property
    def torch(self):
        if self._torch is None:
            import torch  # deferred: the first import can take a while on a fresh machine

            self._torch = torch
        return self._torch

    @property
    def num_gpus(self) -> int:
        return 1 if self.torch.cuda.is_available() else 0

    def require_device(self) -> "torch.device":
        torch = self.torch
        if not torch.cuda.is_available():
            raise RuntimeError(
                "cupynumeric_amd needs a HIP device: no GPU is visible to this process "
                "(there is no CPU fallback for the sort path)"
            )
        return torch.device("cuda", torch.cuda.current_device())

    def stream_handle(self) -> int:
        """hipStream_t of torch's current stream, as an integer."""
        return int(self.torch.cuda.current_stream().cuda_stream)

    def empty_bytes(self, nbytes: int) -> "torch.Tensor":
        """Uninitialised device buffer of `nbytes` bytes (at least one, so that it has an address)."""
        dev = self.require_device()
        return self.torch.empty(max(int(nbytes), 1), dtype=self.torch.uint8, device=dev)

    def zero_flag(self) -> "torch.Tensor":
        """A cleared 4-byte device word for kernels that report a condition (e.g. a bad index)."""
        dev = self.require_device()
        return self.torch.zeros(1, dtype=self.torch.int32, device=dev)

    def upload(self, host: np.ndarray) -> "torch.Tensor":
        """Copy a C-contiguous host array to a new device byte buffer."""
        dev = self.require_device()
        torch = self.torch
        flat = np.ascontiguousarray(host).reshape(-1).view(np.uint8)
        if flat.size == 0:
            return torch.empty(1, dtype=torch.uint8, device=dev)
        return torch.from_numpy(flat).to(dev)

    def download(self, buf: "torch.Tensor", shape: tuple[int, ...], dtype: np.dtype) -> np.ndarray:
        nbytes = int(np.prod(shape, dtype=np.int64)) * dtype.itemsize
        if nbytes == 0:
            return np.empty(shape, dtype=dtype)
        host = buf[:nbytes].cpu().numpy()
        return host.view(dtype).reshape(shape).copy()


runtime = Runtime()
