"""Helpers for the GPU tests: traces in the four ways of running a request, a
replay through the framework's runner, and the comparison with the plain
implementation."""
import random
from typing import Dict, List, Sequence, Tuple

import torch

import plain_model

# relative to the largest |logit| of the expected rows; fixed before the first run
FP32_TOL = 2e-5
BF16_TOL = 2e-2

Step = dict  # {"entries": [(id, tokens, want)], "end": [ids]}


def whole(prompts: Dict[str, List[int]]) -> List[Step]:
    return [{"entries": [(rid, toks, list(range(len(toks))))], "end": [rid]} for rid, toks in prompts.items()]


def tail_decoded(prompts: Dict[str, List[int]], tail: int = 32) -> List[Step]:
    steps = []
    for rid, toks in prompts.items():
        head = max(1, len(toks) - tail)
        steps.append({"entries": [(rid, toks[:head], list(range(head)))], "end": []})
        for i in range(head, len(toks)):
            steps.append({"entries": [(rid, toks[i:i + 1], [0])], "end": [rid] if i == len(toks) - 1 else []})
        if head == len(toks):
            steps[-1]["end"] = [rid]
    return steps


def chunked(prompts: Dict[str, List[int]], sizes: Sequence[int] = (7, 2, 13, 3, 2, 16, 5, 31, 2, 64)) -> List[Step]:
    steps = []
    for rid, toks in prompts.items():
        at, i = 0, 0
        while at < len(toks):
            n = min(sizes[i % len(sizes)], len(toks) - at)
            if len(toks) - at - n == 1:  # never leave a single token: portions go down to two
                n += 1
            steps.append({"entries": [(rid, toks[at:at + n], list(range(n)))],
                          "end": [rid] if at + n == len(toks) else []})
            at += n
            i += 1
    return steps


def mixed(prompts: Dict[str, List[int]], seed: int, max_live: int = 4, max_tokens: int = 10 ** 9,
          round_to: int = 64) -> List[Step]:
    """Up to `max_live` requests at a time; each step gives some of them a portion
    of their prompt, others a single token, and leaves some out.  A request is
    admitted only if the live requests' lengths, each rounded up to `round_to`,
    stay within `max_tokens`."""
    rng = random.Random(seed)
    waiting = list(prompts.items())
    live: Dict[str, int] = {}  # id -> tokens fed so far
    steps: List[Step] = []
    held = lambda n: -(-n // round_to) * round_to
    while waiting or live:
        while waiting and len(live) < max_live and \
                sum(held(len(prompts[r])) for r in live) + held(len(waiting[0][1])) <= max_tokens:
            live[waiting.pop(0)[0]] = 0
        entries, end = [], []
        for rid in list(live):
            toks, at = prompts[rid], live[rid]
            if len(live) > 1 and rng.random() < 0.2:
                continue  # left out of this step
            left = len(toks) - at
            mode = rng.random()
            n = 1 if (mode < 0.4 and at > 0) else min(left, rng.choice([2, 3, 5, 8, 17, 33]))
            entries.append((rid, toks[at:at + n], list(range(n))))
            live[rid] = at + n
            if at + n == len(toks):
                end.append(rid)
                del live[rid]
        if entries:
            steps.append({"entries": entries, "end": end})
    return steps


def replay(runner, steps: List[Step], page_owners: dict = None) -> Dict[Tuple[str, int], torch.Tensor]:
    """Run the steps; logits by (request, position) on the CPU.  `page_owners`, if given, collects for every
    physical page (group, page) the requests that held it during some step."""
    got: Dict[Tuple[str, int], torch.Tensor] = {}
    for step in steps:
        for rid, _, _ in step["entries"]:
            if rid not in runner.cache:
                runner.add_request(rid)
        before = {rid: runner.cache.cached(rid) for rid, _, _ in step["entries"]}
        logits = runner.run_entries(step["entries"]).cpu()
        row = 0
        for rid, toks, want in step["entries"]:
            for w in want:
                key = (rid, before[rid] + w)
                assert key not in got, f"{key} produced twice"
                got[key] = logits[row]
                row += 1
        assert row == logits.shape[0]
        if page_owners is not None:
            for rid, _, _ in step["entries"]:
                for g in range(len(runner.cache.groups)):
                    for page in runner.cache.block_row(rid, g):
                        if page >= 0:
                            page_owners.setdefault((g, int(page)), set()).add(rid)
        for rid in step["end"]:
            runner.end_request(rid)
        runner.cache.check()
    return got


def expected_logits(cfg: dict, weights, prompts: Dict[str, List[int]]) -> Dict[str, torch.Tensor]:
    return {rid: plain_model.forward(cfg, weights, toks) for rid, toks in prompts.items()}


NEAR_TIE = 5e-3  # relative gap between the last chosen expert's probability and the first one's left out


def near_ties(cfg: dict, weights, prompts: Dict[str, List[int]]):
    """Places where the plain implementation's routing hangs on a gap below NEAR_TIE in some sparse layer.
    bfloat16 activations put an error of about 6e-4 on a router score here, so there a bfloat16 run may choose the other
    expert, which changes that token's feed-forward output by far more than rounding; such places are left out
    of bfloat16 comparisons (never of float32 ones).  The tolerance of all other places stays what it is."""
    out = set()
    for rid, toks in prompts.items():
        margins: List[torch.Tensor] = []
        plain_model.forward(cfg, weights, toks, margins=margins)
        if margins:
            worst = torch.stack(margins).min(0).values
            out |= {(rid, int(p)) for p in torch.nonzero(worst < NEAR_TIE).flatten()}
    return out


def compare(got, expected: Dict[str, torch.Tensor], tol: float, what: str = "", skip=()) -> float:
    """Largest |difference| relative to the largest |expected logit|; names the first bad place.
    Places in `skip` (near ties of the routing, bfloat16 only) must be present and finite, no more."""
    worst = 0.0
    scale = max(float(e.abs().max()) for e in expected.values())
    n = 0
    for rid, exp in expected.items():
        for pos in range(exp.shape[0]):
            assert (rid, pos) in got, f"{what}: no logits for request {rid} position {pos}"
            n += 1
            row = got[(rid, pos)].double()
            assert torch.isfinite(row).all(), f"{what}: non-finite logits at request {rid} position {pos}"
            err = float((row - exp[pos]).abs().max()) / scale
            if (rid, pos) in skip:
                continue
            if err > tol:
                raise AssertionError(
                    f"{what}: request {rid} position {pos} is the first wrong place: error {err:.3e} of the largest "
                    f"logit, tolerance {tol:.1e}")
            worst = max(worst, err)
    assert n == len(got), f"{what}: {len(got)} rows produced, {n} expected"
    return worst
