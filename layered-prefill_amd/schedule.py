"""Batch shapes of layered prefill: which (prefill, decode) token mix each MoE
layer call sees, iteration by iteration.

A host-only restatement of the reference's ``layered_prefill_schedule`` and
``get_num_stages`` (nanovllm/engine/scheduler.py:181-328, bookkeeping of
``postprocess`` at :337-370) together with the stage -> layer split of its model
runner (nanovllm/engine/model_runner.py:251-256: ``np.array_split`` of the layer
indices).  No KV-cache block manager (memory is taken to be sufficient, so
nothing is preempted), no tokens, no model: only counts.

One engine iteration runs every decoding sequence (one token each) through all
layers.  A group of prompts is admitted when no group is in flight, up to
``max_num_batched_tokens`` prompt tokens; the group is then carried for
``num_stages`` consecutive iterations and in iteration ``stage`` its tokens go
through the ``stage``-th slice of the layers only.  So a layer call sees
``decode + prefill`` tokens when the layer lies in the current slice and
``decode`` tokens otherwise: each expert's weights are streamed once per prompt
group instead of once per chunk.
"""
from __future__ import annotations

import csv
import os
import random
from collections import Counter, deque
from dataclasses import dataclass, field
from typing import Deque, Dict, Iterable, List, Optional, Sequence, Tuple

TRACE_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "traces")
SHAREGPT_SAMPLE = os.path.join(TRACE_DIR, "sharegpt_8k_lengths_first2048.csv")

# get_num_stages (nanovllm/engine/scheduler.py:181-224): configured stage count ->
# (upper bound of the group's prompt tokens, stages used) pairs, last entry open-ended
_STAGE_TABLE: Dict[int, Tuple[Tuple[Optional[int], int], ...]] = {
    4: ((512, 1), (1024, 2), (None, 4)),
    12: ((512, 1), (1024, 2), (2048, 4), (4096, 6), (None, 12)),
    16: ((512, 1), (1024, 2), (2048, 4), (4096, 8), (None, 16)),
    24: ((512, 1), (1024, 2), (2048, 4), (4096, 8), (None, 24)),
}


def get_num_stages(configured_stages: int, num_batched_tokens: int) -> int:
    """Stages a prompt group of ``num_batched_tokens`` tokens is spread over."""
    if configured_stages not in _STAGE_TABLE:
        raise ValueError(f"Unsupported number of stages: {configured_stages}")
    for bound, stages in _STAGE_TABLE[configured_stages]:
        if bound is None or num_batched_tokens <= bound:
            return stages
    raise AssertionError("unreachable")


def stage_layers(num_layers: int, num_stages: int, stage: int) -> range:
    """Layers the prompt group runs through in iteration ``stage`` of its
    ``num_stages``: ``np.array_split(np.arange(num_layers), num_stages)[stage]``
    (the first ``num_layers % num_stages`` slices get one layer more)."""
    base, extra = divmod(num_layers, num_stages)
    lo = stage * base + min(stage, extra)
    return range(lo, lo + base + (1 if stage < extra else 0))


@dataclass
class Request:
    prompt_len: int
    output_len: int       # tokens to generate (the reference's max_tokens with ignore_eos)
    arrival_iter: int = 0  # first iteration that may admit it


@dataclass
class _Seq:
    req: Request
    processed: int = 0        # prompt tokens already through all layers
    to_process: int = 0       # prompt tokens of the group in flight
    generated: int = 0


@dataclass
class IterationShape:
    index: int
    decode_tokens: int
    prefill_tokens: int           # prompt tokens of the group in flight (0: none)
    stage: int                    # -1 without a group
    num_stages: int               # -1 without a group
    prefill_layers: range = field(default_factory=lambda: range(0))

    def layer_tokens(self, layer: int) -> int:
        """Tokens the MoE call of ``layer`` sees in this iteration."""
        return self.decode_tokens + (self.prefill_tokens if layer in self.prefill_layers else 0)


def simulate(requests: Sequence[Request], num_layers: int, configured_stages: int = 16,
             max_num_seqs: int = 512, max_num_batched_tokens: int = 16384,
             max_iterations: int = 1_000_000) -> List[IterationShape]:
    """Runs the schedule until every request has finished.  Defaults are the
    reference's (nanovllm/config.py:11-12)."""
    pending = deque(sorted(requests, key=lambda r: r.arrival_iter))
    waiting: Deque[_Seq] = deque()
    prefilling: Deque[_Seq] = deque()     # prompts cut by the token budget, to be continued
    decoding: Deque[_Seq] = deque()
    group: List[_Seq] = []
    stage, num_stages = -1, -1
    out: List[IterationShape] = []
    it = 0
    while pending or waiting or prefilling or decoding or group:
        if it >= max_iterations:
            raise RuntimeError("schedule did not finish")
        while pending and pending[0].arrival_iter <= it:
            waiting.append(_Seq(pending.popleft()))
        # decodes first: every running sequence, up to the sequence cap (scheduler.py:235-249)
        decode_now = list(decoding)[:max_num_seqs]
        num_seqs = len(decode_now)
        if not group:
            # admit a new group: cut prompts first, then new ones (scheduler.py:259-304)
            batched = 0
            for queue in (prefilling, waiting):
                while queue and num_seqs < max_num_seqs and batched < max_num_batched_tokens:
                    seq = queue.popleft()
                    seq.to_process = min(seq.req.prompt_len - seq.processed, max_num_batched_tokens - batched)
                    batched += seq.to_process
                    num_seqs += 1
                    group.append(seq)
            if group:
                num_stages = get_num_stages(configured_stages, batched)
                stage = -1
        if group:
            stage += 1
            shape = IterationShape(it, len(decode_now), sum(s.to_process for s in group), stage, num_stages,
                                   stage_layers(num_layers, num_stages, stage))
        else:
            if not decode_now:     # idle until the next arrival
                it = pending[0].arrival_iter if pending else it + 1
                continue
            shape = IterationShape(it, len(decode_now), 0, -1, -1)
        out.append(shape)
        # bookkeeping after the step (scheduler.py:337-370)
        if group and stage == num_stages - 1:
            for seq in group:
                seq.processed += seq.to_process
                seq.to_process = 0
                if seq.processed >= seq.req.prompt_len:
                    seq.generated = 1          # the last stage samples the first token
                    if seq.generated < seq.req.output_len:
                        decoding.append(seq)
                else:
                    prefilling.append(seq)
            group, stage, num_stages = [], -1, -1
        for seq in decode_now:
            seq.generated += 1
            if seq.generated >= seq.req.output_len:
                decoding.remove(seq)
        it += 1
    return out


def moe_call_sizes(shapes: Iterable[IterationShape], num_layers: int) -> Counter:
    """How often a MoE layer call of each token count occurs over the run."""
    sizes: Counter = Counter()
    for s in shapes:
        with_prefill = len(s.prefill_layers)
        if s.decode_tokens + s.prefill_tokens > 0 and with_prefill:
            sizes[s.decode_tokens + s.prefill_tokens] += with_prefill
        if s.decode_tokens > 0:
            sizes[s.decode_tokens] += num_layers - with_prefill
    return sizes


def load_length_trace(path: str = SHAREGPT_SAMPLE) -> List[Tuple[int, int]]:
    """(prompt tokens, output tokens) pairs of a length trace in the reference's
    CSV layout (benchmarks/preprocessed_traces/*.csv: the first two columns)."""
    pairs = []
    with open(path, newline="") as f:
        for row in csv.reader(line for line in f if not line.startswith("#")):
            if row and row[0].isdigit():
                pairs.append((int(row[0]), int(row[1])))
    return pairs


def poisson_requests(lengths: Sequence[Tuple[int, int]], n: int, per_iteration: float,
                     seed: int = 0) -> List[Request]:
    """``n`` requests drawn in trace order with exponential gaps of mean
    ``1 / per_iteration`` iterations (``per_iteration <= 0``: all present at the start)."""
    rng = random.Random(seed)
    t = 0.0
    reqs = []
    for i in range(n):
        p, d = lengths[i % len(lengths)]
        reqs.append(Request(p, max(d, 1), int(t)))
        if per_iteration > 0:
            t += rng.expovariate(per_iteration)
    return reqs
