"""Chooses next tokens from a step's logits on the device (reference: ullm/layers/sampler.py).

One kernel launch per step for all rows; each row carries its own parameters and its own
(seed, position), so what a request draws does not depend on the rest of the batch."""
from __future__ import annotations

from typing import List, Sequence

import numpy as np
import torch

from ..kernels import ops
from .params import SamplingParams


class Sampler:
    def __init__(self, device: torch.device):
        self.device = device

    def sample(self, logits: torch.Tensor, params: Sequence[SamplingParams], seeds: Sequence[int],
               positions: Sequence[int]) -> List[int]:
        """``logits`` float32 [n, V]; ``positions[i]`` = index the new token of row i will take in its
        request (the counter of the row's random stream).  Returns n token ids."""
        n = logits.shape[0]
        if not (len(params) == len(seeds) == len(positions) == n):
            raise ValueError("one parameter set, seed and position per logits row is needed")
        f = np.empty((3, n), dtype=np.float32)
        i = np.empty((4, n), dtype=np.int32)
        for r, (p, s, pos) in enumerate(zip(params, seeds, positions)):
            f[0, r], f[1, r], f[2, r] = p.temperature, p.top_p, p.min_p
            s &= (1 << 64) - 1
            i[0, r] = p.top_k
            i[1, r] = np.uint32(s & 0xFFFFFFFF).astype(np.int32)
            i[2, r] = np.uint32(s >> 32).astype(np.int32)
            i[3, r] = pos
        fd = torch.from_numpy(f).to(self.device)
        idev = torch.from_numpy(i).to(self.device)
        out = ops.sample(logits, fd[0], idev[0], fd[1], fd[2], idev[1], idev[2], idev[3])
        return out.tolist()
