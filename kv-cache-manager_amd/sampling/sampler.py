"""Token choice for the rows a step sampled from: greedy (the reference's rule, lowest index on
ties, src/cuda/kernels.cu:90-119) or temperature sampling by Gumbel-max with a counter-based
draw keyed by (sampler seed, request id, index of the generated token).  The draw of a request's
k-th token is the same however the request was batched, cut into portions or preempted."""
from typing import Sequence

import numpy as np
import torch


class Sampler:
    def __init__(self, ops, device, max_rows: int):
        self.ops, self.device, self.max_rows = ops, device, max_rows
        self.out = torch.zeros(max_rows, dtype=torch.int32, device=device)
        self.temperature = torch.zeros(max_rows, dtype=torch.float32, device=device)
        self.seeds = torch.zeros(max_rows, dtype=torch.int64, device=device)
        self.request_ids = torch.zeros(max_rows, dtype=torch.int64, device=device)
        self.token_index = torch.zeros(max_rows, dtype=torch.int32, device=device)
        self._host = torch.zeros(max_rows, dtype=torch.int32, pin_memory=True)

    def sample(self, logits: torch.Tensor, temperatures: Sequence[float], seeds: Sequence[int],
               request_ids: Sequence[int], token_index: Sequence[int]) -> np.ndarray:
        """logits [R, V] float32 on the device -> R token ids on the host."""
        R = logits.shape[0]
        if R > self.max_rows:
            raise RuntimeError(f"sampler: {R} rows exceed the limit of {self.max_rows}")
        out = self.out[:R]
        if not any(t > 0 for t in temperatures):
            self.ops.sample(logits, out)
        else:
            self.temperature[:R].copy_(torch.tensor(list(temperatures), dtype=torch.float32))
            # seeds are 64-bit patterns; keep the bits when they exceed the signed range
            s = np.asarray([x & ((1 << 64) - 1) for x in seeds], dtype=np.uint64).view(np.int64)
            self.seeds[:R].copy_(torch.from_numpy(s.copy()))
            self.request_ids[:R].copy_(torch.tensor(list(request_ids), dtype=torch.int64))
            self.token_index[:R].copy_(torch.tensor(list(token_index), dtype=torch.int32))
            self.ops.sample(logits, out, self.temperature[:R], self.seeds[:R], self.request_ids[:R],
                            self.token_index[:R])
        return self.download(R)

    def sample_on_device(self, logits: torch.Tensor, params) -> np.ndarray:
        """As ``sample`` with the parameters already on the device: (temperature, seeds, request
        ids, token index) as the step's metadata buffer carries them."""
        R = logits.shape[0]
        if R > self.max_rows:
            raise RuntimeError(f"sampler: {R} rows exceed the limit of {self.max_rows}")
        t, seeds, ids, idx = params
        self.ops.sample(logits, self.out[:R], t[:R], seeds[:R], ids[:R], idx[:R])
        return self.download(R)

    def download(self, R: int) -> np.ndarray:
        self._host[:R].copy_(self.out[:R])          # synchronous: the ids are needed on the host now
        return self._host[:R].numpy().copy()
