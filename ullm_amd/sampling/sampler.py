"""Chooses next tokens from a step's logits on the device (reference: ullm/layers/sampler.py).

One or two kernel launches per step for all rows; each row carries its own parameters and its own
(seed, position), so what a request draws does not depend on the rest of the batch."""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Sequence

import numpy as np
import torch

from ..kernels import ops
from ..staging import StagedUpload
from .params import SamplingParams


@dataclass
class SamplerInputs:
    """Per-row parameters on the device: rows of one int32 buffer (the float ones bit-cast)."""
    n: int
    packed: torch.Tensor      # int32 [7, n]: temperature, top_p, min_p (float bits), top_k, seed low, seed high, position
    cut_rows: bool = True     # some row has settings for which the kernels cut rows into parts (ops.sample)


class Sampler:
    def __init__(self, device: torch.device, cut_rows: bool = True):
        self.device = device
        self.cut_rows = cut_rows      # False: one block per row does all the work (ops.sample)
        self._upload = StagedUpload(device)

    def stage(self, params: Sequence[SamplingParams], seeds: Sequence[int], positions: Sequence[int]) -> torch.Tensor:
        """Pack the rows' parameters into pinned memory (host work only; may be done while the
        device runs the step before).  ``positions[i]`` = index the new token of row i will take in
        its request (the counter of the row's random stream)."""
        n = len(params)
        if not (len(seeds) == len(positions) == n):
            raise ValueError("one parameter set, seed and position per logits row is needed")
        flat = np.empty(7 * n + 1, dtype=np.int32)
        host = flat[:7 * n].reshape(7, n)
        host[0:3].view(np.float32)[:] = [[p.temperature for p in params], [p.top_p for p in params],
                                         [p.min_p for p in params]]
        host[3] = [p.top_k for p in params]
        s64 = np.array([s & 0xFFFFFFFFFFFFFFFF for s in seeds], dtype=np.uint64)
        host[4] = (s64 & np.uint64(0xFFFFFFFF)).astype(np.uint32).view(np.int32)
        host[5] = (s64 >> np.uint64(32)).astype(np.uint32).view(np.int32)
        host[6] = positions
        # one more word, for the host alone: whether any row has settings that the kernels serve by cutting rows
        # into parts (every setting but greedy and a top-k above ops.SAMPLE_PARTS_TOP_K); without one, that kernel
        # is not launched
        flat[-1] = int(any(p.temperature != 0 and p.top_k <= ops.SAMPLE_PARTS_TOP_K for p in params))
        return self._upload.stage(flat)

    def send(self, staged: torch.Tensor) -> SamplerInputs:
        """Queue the upload of staged parameters.  Called before the model step is launched, the copy
        does not wait for the step, and sampling can follow it without the host in between."""
        n = staged.numel() // 7
        return SamplerInputs(n, self._upload.send(staged)[:7 * n].view(7, n), bool(int(staged[-1])))

    def prepare(self, params: Sequence[SamplingParams], seeds: Sequence[int], positions: Sequence[int]) -> SamplerInputs:
        return self.send(self.stage(params, seeds, positions))

    def launch(self, logits: torch.Tensor, prepared: SamplerInputs, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Queue the sampling kernel; returns the n token ids as an int32 device tensor (reading it
        waits for the step), the first n entries of ``out`` if that is given."""
        if prepared.n != logits.shape[0]:
            raise ValueError("one parameter set, seed and position per logits row is needed")
        f = prepared.packed[0:3].view(torch.float32)
        i = prepared.packed
        return ops.sample(logits, f[0], i[3], f[1], f[2], i[4], i[5], i[6], out=out,
                          parts=self.cut_rows and prepared.cut_rows)[:prepared.n]

    def sample(self, logits: torch.Tensor, params: Optional[Sequence[SamplingParams]] = None,
               seeds: Optional[Sequence[int]] = None, positions: Optional[Sequence[int]] = None,
               prepared: Optional[SamplerInputs] = None) -> List[int]:
        """``logits`` float32 [n, V]; the rows' parameters either as lists or as the result of
        :meth:`prepare`.  Returns n token ids."""
        if prepared is None:
            prepared = self.prepare(params, seeds, positions)
        return self.launch(logits, prepared).tolist()
