"""Uniform handle on a non-blocking operation (pccl/request.py:6-80).

The reference wraps a torch.distributed Work or an mpi4py Request.  Work that
this package enqueues on a HIP stream is represented by `StreamRequest` (a
recorded event); `Request` accepts either kind and keeps the reference's
`wait(epilogue)` contract: block until done, then call `epilogue()` with no
argument (pccl/request.py:64-70).
"""
from __future__ import annotations

from typing import Any, Callable, Optional

import torch
import torch.distributed as dist


class StreamRequest:
    """Completion of everything enqueued so far on a HIP stream."""

    def __init__(self, stream: Optional["torch.cuda.Stream"] = None):
        self.stream = stream if stream is not None else torch.cuda.current_stream()
        self.event = torch.cuda.Event(enable_timing=False)
        self.event.record(self.stream)

    def Wait(self, status=None):
        self.event.synchronize()
        return True

    def Test(self) -> bool:
        return self.event.query()


class Request:
    """A unified request over torch.distributed and stream-ordered work."""

    def __init__(self, request: Any):
        if isinstance(request, dist.Work):
            self.backend = 'torch'
        elif isinstance(request, StreamRequest):
            self.backend = 'stream'
        else:
            raise ValueError(
                f"Unsupported request type: {type(request)}. "
                "Expected torch.distributed.Work or pccl.request.StreamRequest."
            )
        self.request = request

    def wait(self, epilogue: Optional[Callable[[], None]] = None) -> Optional[Any]:
        if self.backend == 'torch':
            self.request.wait()
        elif self.backend == 'stream':
            self.request.Wait()
        else:
            raise ValueError("Unsupported backend.")
        if epilogue is not None:
            if not callable(epilogue):
                raise TypeError("Epilogue must be a callable.")
            try:
                epilogue()
            except Exception as e:
                print(f"An error occurred in the epilogue: {e}")
                raise
        return None

    def __repr__(self) -> str:
        return f"<Request backend={self.backend} request={self.request}>"
