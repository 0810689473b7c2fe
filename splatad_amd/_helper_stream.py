"""The optional helper stream of `rasterization()` (switch `rendering.HELPER_STREAM`, off by default).

A call whose plan says so runs the work that only depends on the projection -- the colour
kernel, the packed rows, their opacities -- on a stream of its own beside the tile intersection;
everything else in `rendering.py` talks to the small interface both classes below share:
`with helper:` around work that may go beside, `refork()`, `join()`, and the `requests` /
`results` dicts through which the packed projection is asked to make things of its rows.
"""
import threading
from typing import Dict

import torch
from torch import Tensor

# one helper stream per (host thread, device): calls from different threads do not wait for one
# another's helper work, and a thread's streams go when the thread does
_THREAD = threading.local()


class HelperStream:
    """Runs the work of `with` blocks on a helper stream, beside what the caller's stream does
    between the creation of the object (the fork) and `join()`.

    The tile intersection ends with a segment sort whose few long workgroups leave most of the
    GPU idle; work that only depends on the projection -- the colours of the Gaussians -- is
    enqueued on a helper stream (default priority) to run meanwhile.  Create the object when
    the inputs of that work are enqueued on the caller's stream: the helper stream waits for
    that point only, not for what the caller's stream is given afterwards.  `join()` makes the
    caller's stream wait for the helper and tells the allocator that the tensors made there
    are used on the caller's stream from now on.  On a CPU device, or while a graph is being
    captured, the blocks simply run in place.
    """

    def __init__(self, device, requests=None):
        self.main = self.side = self.fork = self._ctx = self._waited = None
        # what the packed projection is asked to make on the helper stream, and what it made
        self.requests: Dict[str, object] = dict(requests or {})
        self.results: Dict[str, Tensor] = {}
        if device.type == "cuda" and not torch.cuda.is_current_stream_capturing():
            idx = device.index if device.index is not None else torch.cuda.current_device()
            streams = _THREAD.__dict__.setdefault("streams", {})
            if idx not in streams:
                streams[idx] = torch.cuda.Stream(device=idx)
            self.main = torch.cuda.current_stream(idx)
            self.side = streams[idx]
            self.fork = self.main.record_event()

    def __enter__(self):
        if self.side is not None:
            if self._waited is not self.fork:  # once per fork: the helper stream runs in order
                self.side.wait_event(self.fork)
                self._waited = self.fork
            self._ctx = torch.cuda.stream(self.side)
            self._ctx.__enter__()
        return self

    def __exit__(self, *exc):
        if self._ctx is not None:
            self._ctx.__exit__(*exc)
            self._ctx = None
        return False

    def refork(self):
        """Moves the fork to what the caller's stream holds now."""
        if self.side is not None:
            self.fork = self.main.record_event()

    def join(self, *tensors):
        if self.side is not None:
            self.main.wait_stream(self.side)
            for t in tensors:
                if t is not None:
                    t.record_stream(self.main)




class InPlace:
    """The same interface without a helper stream: the blocks run where they stand, on the
    caller's stream, and the packed projection serves its requests there."""

    side = None

    def __init__(self, requests=None):
        self.requests: Dict[str, object] = dict(requests or {})
        self.results: Dict[str, Tensor] = {}

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False

    def refork(self):
        pass

    def join(self, *tensors):
        pass
