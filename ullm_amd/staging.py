"""Host-to-device upload of small per-step arrays through pinned memory, without blocking the host.

A pageable copy waits on the stream for all work queued before it and holds the host meanwhile;
a pinned one is queued and returns.  Two pinned buffers are used in turn; a buffer is written
again only after the copy that last read it has finished."""
from __future__ import annotations

from typing import List, Optional

import numpy as np
import torch


class StagedUpload:
    def __init__(self, device: torch.device):
        self.device = device
        self._pin = device.type == "cuda"
        self._buffers: List[Optional[torch.Tensor]] = [None, None]
        self._done: List[Optional["torch.cuda.Event"]] = [None, None]
        self._turn = 0

    def stage(self, host: np.ndarray) -> torch.Tensor:
        """Put the int32 array ``host`` into the pinned buffer whose turn it is and return that view;
        nothing is queued yet.  The step that will be sent next can be staged (and staged again)
        while the device still runs the one before; small fix-ups may be written into the view."""
        i = self._turn
        if self._done[i] is not None:
            self._done[i].synchronize()
            self._done[i] = None
        if self._buffers[i] is None or self._buffers[i].numel() < host.size:
            self._buffers[i] = torch.empty(max(host.size, 4096), dtype=torch.int32, pin_memory=self._pin)
        stage = self._buffers[i][:host.size]
        stage.numpy()[:] = host
        return stage

    def send(self, stage: torch.Tensor, into: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Queue the copy of a staged view to the device (into ``into`` if given); returns the device tensor."""
        i = self._turn
        if self._buffers[i] is None or stage.data_ptr() != self._buffers[i].data_ptr():
            raise RuntimeError("only the view staged last can be sent")
        self._turn ^= 1
        if into is not None:
            into.copy_(stage, non_blocking=True)
            dev = into
        else:
            dev = stage.to(self.device, non_blocking=True)
        if self._pin:
            ev = torch.cuda.Event()
            ev.record()
            self._done[i] = ev
        elif dev.data_ptr() == stage.data_ptr():
            dev = dev.clone()
        return dev

    def __call__(self, host: np.ndarray, into: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Copy the int32 array ``host`` to the device (into ``into`` if given) and return the device tensor."""
        return self.send(self.stage(host), into)
