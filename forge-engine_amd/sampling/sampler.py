"""Token selection over float32 logits rows.

Greedy rows take the argmax kernel.  Other rows are filtered in the order of
the reference (src/forge_engine/sampling.py:83-140): temperature, top-k, top-p,
min-p; the draw itself is the inverse-CDF kernel with a counter-based
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

NEG_INF = float("-inf")


def filter_logits(logits: Tensor, params: SamplingParams) -> Tensor:
    """Rows after temperature, top-k, top-p and min-p; removed entries are -inf."""
    if params.greedy:
        raise ValueError("greedy sampling does not filter logits")
    x = logits.float()
    x = (x - x.amax(dim=-1, keepdim=True)) / params.temperature
    if params.top_k is not None and params.top_k < x.shape[-1]:
        values, indices = torch.topk(x, params.top_k, dim=-1)
        x = torch.full_like(x, NEG_INF).scatter_(-1, indices, values)
    if params.top_p < 1.0:
        ordered, order = torch.sort(x, dim=-1, descending=True)
        mass = torch.softmax(ordered, dim=-1, dtype=torch.float32).cumsum(dim=-1)
        # a token goes if the mass of the tokens before it already exceeds top_p;
        # the first token always stays
        before = torch.zeros_like(mass)
        before[..., 1:] = mass[..., :-1]
        ordered = ordered.masked_fill(before > params.top_p, NEG_INF)
        x = torch.full_like(x, NEG_INF).scatter_(-1, order, ordered)
    if params.min_p > 0.0:
        probs = torch.softmax(x, dim=-1, dtype=torch.float32)
        x = x.masked_fill(probs < probs.amax(dim=-1, keepdim=True) * params.min_p, NEG_INF)
    return x


def _raise_on_status(status: list[int]) -> None:
    for flags in status:
        if flags & 1:
            raise ValueError("logits must not contain NaN")
        if flags & 2:
            raise ValueError("logits must not contain positive infinity")
        if flags & 4:
            raise ValueError("each logits row must contain a finite value")


class Sampler:
    def __init__(self, device: torch.device) -> None:
        self.device = device

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

    def sample(self, logits: Tensor, params: list[SamplingParams], seeds: list[int],
               draw_index: list[int]) -> list[int]:
        """One token per row.  ``seeds[r]`` and ``draw_index[r]`` (how many tokens
        the request has drawn so far) key the generator of row r."""
        rows = logits.shape[0]
        if rows == 0:
            return []
        if not (len(params) == len(seeds) == len(draw_index) == rows):
            raise ValueError("one parameter set, seed and draw index per logits row is needed")
        both = torch.empty((2, rows), dtype=torch.int32, device=self.device)   # one transfer brings both back
        tokens, status = both[0], both[1]
        greedy = [r for r in range(rows) if params[r].greedy]
        drawn = [r for r in range(rows) if not params[r].greedy]
        if not drawn:
            ops.argmax_rows(logits, tokens, status)
        else:
            self._mixed(logits, params, seeds, draw_index, greedy, drawn, tokens, status)
        host = both.cpu()
        _raise_on_status(host[1].tolist())
        return host[0].tolist()

    def _mixed(self, logits, params, seeds, draw_index, greedy, drawn, tokens, status) -> None:
        if greedy:
            index = torch.tensor(greedy, device=self.device)
            t = torch.empty(len(greedy), dtype=torch.int32, device=self.device)
            s = torch.empty(len(greedy), dtype=torch.int32, device=self.device)
            ops.argmax_rows(logits.index_select(0, index).contiguous(), t, s)
            tokens[index] = t
            status[index] = s
        groups: dict[tuple, list[int]] = {}
        for r in drawn:
            p = params[r]
            groups.setdefault((p.temperature, p.top_k, p.top_p, p.min_p), []).append(r)
        for key, members in groups.items():
            p = params[members[0]]
            index = torch.tensor(members, device=self.device)
            rows = logits.index_select(0, index).contiguous()
            filtered = p.top_k is not None or p.top_p < 1.0 or p.min_p > 0.0
            if filtered:
                check_t = torch.empty(len(members), dtype=torch.int32, device=self.device)
                check_s = torch.empty(len(members), dtype=torch.int32, device=self.device)
                ops.argmax_rows(rows, check_t, check_s)     # the guards see the logits before any filter
                rows = filter_logits(rows, p).contiguous()  # temperature already applied
                temperature = 1.0
            else:
                temperature = p.temperature
            t = torch.empty(len(members), dtype=torch.int32, device=self.device)
            s = torch.empty(len(members), dtype=torch.int32, device=self.device)
            ops.sample_rows(
                rows, torch.full((len(members),), temperature, dtype=torch.float32, device=self.device),
                torch.tensor([_as_int64(seeds[r]) for r in members], dtype=torch.int64, device=self.device),
                torch.tensor([draw_index[r] for r in members], dtype=torch.int64, device=self.device), t, s)
            tokens[index] = t
            status[index] = check_s if filtered else s


def _as_int64(seed: int) -> int:
    """Seeds are 64-bit keys; values above 2^63 wrap into the signed range."""
    seed &= (1 << 64) - 1
    return seed - (1 << 64) if seed >= (1 << 63) else seed
