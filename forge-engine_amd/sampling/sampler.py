"""Token selection over float32 logits rows.

Greedy batches take the argmax kernel.  Otherwise one kernel takes every row
with its own parameters and filters in the order of the reference
(src/forge_engine/sampling.py:83-140): temperature, top-k, top-p, min-p, each
as a threshold on the logit, then draws by inverse CDF with a counter-based
generator, so the n-th token of a request depends only on (seed, n) and the
logits, not on what else was in the batch or on how often the request was
preempted.  NaN, +inf or a row without a finite entry raise, as in
sampling.py:62-70; the check runs inside the kernels and comes back with the
tokens in one transfer.
"""

from __future__ import annotations

import torch
from torch import Tensor

from ..kernels import ops
from .params import SamplingParams


def _raise_on_status(status: list[int]) -> None:
    for flags in status:
        if flags & 8:
            raise RuntimeError("the sampling kernel was given too few launches for a row's filters")
        if flags & 1:
            raise ValueError("logits must not contain NaN")
        if flags & 2:
            raise ValueError("logits must not contain positive infinity")
        if flags & 4:
            raise ValueError("each logits row must contain a finite value")


class Sampler:
    def __init__(self, device: torch.device) -> None:
        self.device = device
        # the rows' parameters go to the device from pinned memory without the host waiting for the
        # stream (a copy from pageable memory waits for everything queued before it, the step
        # included); two buffers in turn, each free again once its last copy has run
        self._staging: list[tuple[Tensor, torch.cuda.Event] | None] = [None, None]
        self._turn = 0

    def _to_device(self, packed: Tensor) -> Tensor:
        if self.device.type != "cuda":
            return packed.to(self.device)
        self._turn ^= 1
        slot = self._staging[self._turn]
        if slot is None or slot[0].shape[0] < packed.shape[0]:
            rows = max(64, 2 * packed.shape[0])
            slot = (torch.empty((rows, packed.shape[1]), dtype=packed.dtype, pin_memory=True), torch.cuda.Event())
            self._staging[self._turn] = slot
        else:
            slot[1].synchronize()
        host = slot[0][:packed.shape[0]]
        host.copy_(packed)
        on_device = host.to(self.device, non_blocking=True)
        slot[1].record(torch.cuda.current_stream(self.device))
        return on_device

    def sample_greedy_on_device(self, logits: Tensor) -> Tensor:
        """Arg-max of every row, left on the device: int32 [2, rows], the tokens and the rows'
        status words.  Nothing is read back; ``read`` does that, whenever the host wants them
        (a step later, if the tokens are fed to the next step on the device)."""
        rows = logits.shape[0]
        both = torch.empty((2, rows), dtype=torch.int32, device=self.device)
        ops.argmax_rows(logits, both[0], both[1])
        return both

    @staticmethod
    def read(both: Tensor) -> list[int]:
        """The tokens of ``sample_greedy_on_device``, on the host; raises as ``sample`` does."""
        host = both.cpu()
        _raise_on_status(host[1].tolist())
        return host[0].tolist()

    def sample_on_device(self, logits: Tensor, params: list[SamplingParams], seeds: list[int],
                         draw_index: list[int]) -> Tensor:
        """One token per row, left on the device: int32 [2, rows], the tokens and the rows' status
        words, for ``read``.  ``seeds[r]`` and ``draw_index[r]`` (how many tokens the request has
        drawn so far) key the generator of row r."""
        rows = logits.shape[0]
        if not (len(params) == len(seeds) == len(draw_index) == rows):
            raise ValueError("one parameter set, seed and draw index per logits row is needed")
        both = torch.empty((2, rows), dtype=torch.int32, device=self.device)   # one transfer brings both back
        if rows == 0:
            return both
        if all(p.greedy for p in params):
            ops.argmax_rows(logits, both[0], both[1])
        else:
            # all rows in one call, each with its own parameters (greedy rows among them), fed by one
            # transfer: filters and draw run in the kernel, on the logits where they lie
            packed = ops.pack_sample_params([
                (0.0 if p.greedy else p.temperature, p.top_k, p.top_p, p.min_p, seeds[r], draw_index[r])
                for r, p in enumerate(params)])
            ops.sample_filtered_rows(logits.float(), self._to_device(packed), both[0], both[1],
                                     any_top_k=any(p.top_k is not None for p in params if not p.greedy),
                                     any_top_p=any(p.top_p < 1.0 for p in params if not p.greedy))
        return both

    def sample(self, logits: Tensor, params: list[SamplingParams], seeds: list[int],
               draw_index: list[int]) -> list[int]:
        """One token per row, on the host (``sample_on_device``, read at once)."""
        if logits.shape[0] == 0:
            return []
        return self.read(self.sample_on_device(logits, params, seeds, draw_index))
