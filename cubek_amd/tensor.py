"""Borrowed tensor handles and the client object of the reference API.

``TensorHandleRef`` carries what the reference's ``TensorHandleRef`` carries —
device buffer, shape, strides (in elements), element size — and nothing else
(crates/cubek-quant/src/quantize.rs:234-239, src/layout/scales.rs:213-215).
``ComputeClient`` stands for ``ComputeClient<R>``: here it is just the HIP
stream launches are ordered on.  torch is used only to own device memory.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Tuple


@dataclass(frozen=True)
class TensorHandleRef:
    handle: int                 # device pointer
    shape: Tuple[int, ...]
    strides: Tuple[int, ...]    # in elements
    elem_size: int
    _c: list = field(default_factory=list, repr=False, compare=False)  # cached cq_tensor + its arrays

    def as_c(self):
        """The ``cq_tensor`` view of this handle (built once, reused by every launch)."""
        if not self._c:
            from . import _ffi

            self._c.extend(_ffi.make_tensor(self.handle, self.shape, self.strides, self.elem_size))
        return self._c[0]

    @staticmethod
    def from_torch(t) -> "TensorHandleRef":
        """Borrow a torch tensor living on the GPU (no copy, no ownership)."""
        if not t.is_cuda:
            raise ValueError("tensor handles must point at device memory")
        return TensorHandleRef(t.data_ptr(), tuple(t.shape), tuple(t.stride()), t.element_size())


@dataclass(frozen=True)
class ComputeClient:
    stream: int = 0  # hipStream_t as an integer; 0 = default stream

    @staticmethod
    def current() -> "ComputeClient":
        """Client bound to torch's current HIP stream."""
        import torch

        return ComputeClient(torch.cuda.current_stream().cuda_stream)
