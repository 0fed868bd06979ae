"""EventOverlap: the stream-event wrapper handed back by every Buffer call.

Same contract as the reference's wrapper (deep_ep/utils.py:10-61): holds an
EventHandle recorded on a HIP stream; `current_stream_wait()` makes
`torch.cuda.current_stream()` wait for it; usable as a `with` block that
waits on exit.
"""
from typing import Any, Optional, Tuple

import torch

from .deep_ep_cpp import EventHandle


class EventOverlap:
    def __init__(self, event: Optional[EventHandle] = None,
                 extra_tensors: Optional[Tuple[torch.Tensor, ...]] = None) -> None:
        self.event = event
        # kept alive until the event is consumed: a stand-in for Tensor.record_stream
        # that stays valid under graph capture
        self.extra_tensors = extra_tensors

    def current_stream_wait(self) -> None:
        assert self.event is not None
        self.event.current_stream_wait()

    def __enter__(self) -> Any:
        return self

    def __exit__(self, exc_type: Any, exc_val: Any, exc_tb: Any) -> None:
        if self.event is not None:
            self.event.current_stream_wait()
