"""Token choice on the device from float32 logits.  Each wanted row carries four
words: the uniform its request drew (float bits), temperature (float bits),
top_k, top_p (float bits) (csrc/host/scheduler.cpp fills them).

Greedy rows take the largest logit, lowest index on ties.  Other rows follow the
reference's order of operations (src/sampler/mod.rs:84-154): logits / temperature,
keep the top_k largest, softmax, keep the smallest set of most likely tokens whose
mass reaches top_p and renormalise, then walk the cumulative sum in index order
until it exceeds the uniform.  Only the token ids travel to the host."""
from __future__ import annotations

import torch

from ..kernels import kernels


class Sampler:
    def __init__(self, device):
        self.device = torch.device(device)
        self._out = torch.zeros(1024, dtype=torch.int32, device=self.device)
        self._scratch = torch.zeros(1024 * 64, dtype=torch.int32, device=self.device)   # 256 bytes per row

    def sample(self, logits: torch.Tensor, sampling_words: torch.Tensor, all_greedy: bool) -> torch.Tensor:
        """int32 [rows] on the device."""
        n = logits.shape[0]
        if self._out.numel() < n:
            self._out = torch.zeros(2 * n, dtype=torch.int32, device=self.device)
            self._scratch = torch.zeros(2 * n * 64, dtype=torch.int32, device=self.device)
        out = self._out[:n]
        if all_greedy:
            kernels().argmax_rows(logits, out, self._scratch)
        else:
            kernels().sample_rows(logits, sampling_words, out)
        return out
