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

    # status words of global sorts not yet read back (lazy mode): this many fit before a flush
    STATUS_SLOTS = 256

    def __init__(self) -> None:
        # What happens to the device status word of a global sort (the per-row kernels cannot fail):
        #   "lazy"  (default) it is copied to a small device array, asynchronously, and read back when
        #           data next reaches the host; consecutive sorts do not synchronise
        #   "eager" read back after every global sort (one stream sync each); a sort that failed is
        #           repeated once with tiles handed out through one counter
        #   "off"   never read
        mode = os.environ.get("CUPYNUMERIC_AMD_CHECK_STATUS", "lazy").lower()
        self.check_mode = {"0": "off", "off": "off", "1": "eager", "eager": "eager"}.get(mode, "lazy")
        self._torch = None
        self._device_seen = False
        self._devices = {}
        self._status_slots = None
        self._status_kinds: list[str] = []
        self._status_used = 0

    def defer_status(self, temp: "torch.Tensor") -> None:
        """Lazy mode: keep the status word of the sort that just used `temp` (stream-ordered copy)."""
        self.defer_flag(temp[:4].view(self.torch.int32), "sort")

    def defer_flag(self, word: "torch.Tensor", kind: str) -> None:
        """Keep one 4-byte device word that a kernel raises on a condition the host has to report --
        "sort": the status word of a global sort, "index": an index out of bounds -- until data next
        reaches the host (`flush_status`).  The copy is ordered on the stream; nothing waits."""
        torch = self.torch
        if self._status_slots is None:
            self._status_slots = torch.zeros(self.STATUS_SLOTS, dtype=torch.int32, device=word.device)
            self._status_kinds = []
        if self._status_used == self.STATUS_SLOTS:
            self.flush_status()
        self._status_slots[self._status_used : self._status_used + 1].copy_(word)
        self._status_kinds.append(kind)
        self._status_used += 1

    def flush_status(self) -> None:
        """Read back the deferred words (synchronises); raises if a sort failed on the device or an
        index was out of bounds since the last host read."""
        used, self._status_used = self._status_used, 0
        if used == 0:
            return
        kinds, self._status_kinds = self._status_kinds, []
        words = self._status_slots[:used].cpu()
        if not bool(words.any()):
            return
        raised = {kinds[i] for i in range(used) if int(words[i]) != 0}
        if "sort" in raised:
            raise RuntimeError(
                "cpn_local_sort: a sort issued since the last host read failed on the device (a bounded wait "
                "inside a kernel ran out, cpn_status -7); its result and everything computed from it are "
                "invalid.  Repeat the work with CPN_SORT_TILE_ORDER=single or CUPYNUMERIC_AMD_CHECK_STATUS=eager"
            )
        raise IndexError(
            "index out of bounds in an indexed read (take / searchsorted sorter) issued since the last host read; "
            "its result and everything computed from it are invalid"
        )

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
        if not self._device_seen:  # (asked once: the answer does not change while the process lives, and the
            # question costs about 2 us, which a sort of a thousand keys notices)
            if not torch.cuda.is_available():
                raise RuntimeError(
                    "cupynumeric_amd needs a HIP device: no GPU is visible to this process "
                    "(there is no CPU fallback for the sort path)"
                )
            self._device_seen = True
        index = torch.cuda.current_device()
        dev = self._devices.get(index)
        if dev is None:
            dev = self._devices[index] = torch.device("cuda", index)
        return dev

    def stream_handle(self) -> int:
        """hipStream_t of torch's current stream, as an integer."""
        torch = self.torch
        raw = getattr(torch._C, "_cuda_getCurrentRawStream", None)
        if raw is not None:  # (the same handle as current_stream().cuda_stream without building a Stream object)
            return int(raw(torch.cuda.current_device()))
        return int(torch.cuda.current_stream().cuda_stream)

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
        self.flush_status()
        nbytes = int(np.prod(shape, dtype=np.int64)) * dtype.itemsize
        if nbytes == 0:
            return np.empty(shape, dtype=dtype)
        host = buf[:nbytes].cpu().numpy()
        return host.view(dtype).reshape(shape).copy()


runtime = Runtime()
