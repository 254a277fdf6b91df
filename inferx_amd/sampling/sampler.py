"""Choosing the next token of each sampling row, on the device.

Order (reference: src/engine/host_sampling.cc:21-111): penalties and masks on
the logits, then greedy (temperature <= 0: first maximum, lowest index on
ties) or temperature softmax with top-k / min-p / top-p cut-offs and one
uniform draw.  The draw of a request's n-th sampled token depends only on
(seed, n), so a preempted request that is recomputed draws the same numbers.
"""
from __future__ import annotations

from collections import Counter
from typing import List, Sequence, Tuple

import numpy as np
import torch

from .. import ops
from .params import SamplingParams

# (params, number of tokens sampled so far for this request, its generated tokens so far)
Row = Tuple[SamplingParams, int, Sequence[int]]


class Sampler:
    def __init__(self, rt):
        self.rt = rt
        # after `sample`: per row None, or (log-probability of the chosen token, [(token, log-probability), ...])
        self.last_logprobs = None
        # The sampling rows' settings and random streams live on the device: temperature, top-p, top-k, min-p, the
        # stream's key and the number of its next draw, which the kernel itself moves on.  While the same requests
        # sample step after step (a batch that decodes) nothing is brought to the device again; the host keeps what
        # it expects to be there (`_resident`) and uploads afresh when the rows change: a request admitted, ended or
        # recomputed after a preemption, whose n-th draw still depends on (seed, n) alone.
        self._resident = None   # ([(params, draws expected next)], device block) of the last launch
        self.uploads = 0        # how often the block went to the device (tests)

    def _dev(self, values, dtype) -> torch.Tensor:
        return torch.tensor(list(values), dtype=dtype).to(self.rt.device)

    def sample(self, logits: torch.Tensor, rows: List[Row]) -> List[int]:
        """logits float32 [R, V] on the device (changed in place when penalties apply)."""
        return self.launch(logits, rows).result()

    def launch(self, logits: torch.Tensor, rows: List[Row]) -> "PendingSample":
        """Queue the kernels that choose the rows' tokens; `result()` of what is returned waits for them and brings
        the tokens to the host.  The caller can do other host work in between."""
        R = logits.shape[0]
        if R != len(rows):
            raise ValueError(f"{R} logits rows for {len(rows)} sampling rows")
        if R == 0:
            return PendingSample(self, None, rows, None)
        out = self.rt.empty((R,), torch.int32)
        masks = [list(p.stop_tokens) if len(gen) < p.min_tokens else [] for p, _, gen in rows]
        if any(p.needs_penalties for p, _, _ in rows) or any(masks):
            hist_begin, hist_ids, hist_counts, mask_begin, mask_ids = [0], [], [], [0], []
            for (p, _, gen), m in zip(rows, masks):
                if p.needs_penalties:
                    for tok, cnt in sorted(Counter(gen).items()):
                        hist_ids.append(tok)
                        hist_counts.append(cnt)
                hist_begin.append(len(hist_ids))
                mask_ids.extend(m)
                mask_begin.append(len(mask_ids))
            ops.apply_penalties(
                logits, self._dev(hist_begin, torch.int32), self._dev(hist_ids or [0], torch.int32),
                self._dev(hist_counts or [0], torch.int32),
                self._dev([p.presence_penalty for p, _, _ in rows], torch.float32),
                self._dev([p.frequency_penalty for p, _, _ in rows], torch.float32),
                self._dev([p.repetition_penalty for p, _, _ in rows], torch.float32),
                self._dev(mask_begin, torch.int32), self._dev(mask_ids or [0], torch.int32))
        if all(p.temperature <= 0 for p, _, _ in rows):
            ops.argmax(logits, out)
        else:
            expected = [(p, n) for p, n, _ in rows]
            resident = self._resident
            if resident is not None and len(resident[0]) == R and \
                    all(a is p and b == n for (a, b), (p, n) in zip(resident[0], expected)):
                dev = resident[1]  # the same rows as last time, each at its next draw: all of it is there already
            else:
                # all per-row settings in one upload: four 32-bit columns, then two 64-bit ones
                host = np.empty(8 * R, dtype=np.int32)
                host[0:R].view(np.float32)[:] = [p.temperature for p, _, _ in rows]
                host[R:2 * R].view(np.float32)[:] = [p.top_p for p, _, _ in rows]
                host[2 * R:3 * R] = [p.top_k for p, _, _ in rows]
                host[3 * R:4 * R].view(np.float32)[:] = [p.min_p for p, _, _ in rows]
                host[4 * R:6 * R].view(np.uint64)[:] = [p.seed % (1 << 64) for p, _, _ in rows]
                host[6 * R:8 * R].view(np.uint64)[:] = [n for _, n, _ in rows]
                dev = torch.from_numpy(host).to(self.rt.device)
                self.uploads += 1
            ops.sample(logits, out, dev[0:R].view(torch.float32), dev[R:2 * R].view(torch.float32), dev[2 * R:3 * R],
                       dev[3 * R:4 * R].view(torch.float32), dev[4 * R:6 * R].view(torch.int64),
                       dev[6 * R:8 * R].view(torch.int64), advance=True)
            self._resident = ([(p, n + 1) for p, n in expected], dev)
        lp = None
        if any(p.want_logprobs or p.top_logprobs for p, _, _ in rows):
            n_top = max(p.top_logprobs for p, _, _ in rows)
            chosen_lp = self.rt.empty((R,), torch.float32)
            top_ids = self.rt.empty((R, n_top), torch.int32)
            top_lp = self.rt.empty((R, n_top), torch.float32)
            ops.logprobs(logits, out, chosen_lp, top_ids, top_lp)
            lp = (chosen_lp, top_ids, top_lp)
        return PendingSample(self, out, rows, lp)


class PendingSample:
    """Tokens that the device is choosing."""

    def __init__(self, sampler: Sampler, out, rows: List[Row], logprob_tensors):
        self._sampler, self._out, self._rows, self._lp = sampler, out, rows, logprob_tensors

    def result(self) -> List[int]:
        """Waits for the device; also sets the sampler's `last_logprobs`."""
        self._sampler.last_logprobs = None
        if self._out is None:
            return []
        tokens = self._out.tolist()
        if self._lp is not None:
            chosen_lp, top_ids, top_lp = self._lp
            lp, ids, tlp = chosen_lp.tolist(), top_ids.tolist(), top_lp.tolist()
            self._sampler.last_logprobs = [
                (lp[r], list(zip(ids[r][:p.top_logprobs], tlp[r][:p.top_logprobs])))
                if (p.want_logprobs or p.top_logprobs) else None for r, (p, _, _) in enumerate(self._rows)]
        return tokens
