"""Host-only layered-prefill shape generator against the reference's scheduler
(nanovllm/engine/scheduler.py:181-328,337-370; model_runner.py:251-256): the stage
table read off the reference, a schedule worked by hand, and invariants."""
import importlib
import itertools
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sched = importlib.import_module("layered-prefill_amd.schedule")


def test_stage_table_matches_the_reference_thresholds():
    # scheduler.py:183-222, every branch
    want = {
        16: [(1, 1), (512, 1), (513, 2), (1024, 2), (1025, 4), (2048, 4), (2049, 8), (4096, 8), (4097, 16), (10 ** 6, 16)],
        4: [(512, 1), (513, 2), (1024, 2), (1025, 4), (10 ** 6, 4)],
        12: [(512, 1), (1024, 2), (2048, 4), (2049, 6), (4096, 6), (4097, 12)],
        24: [(512, 1), (1024, 2), (2048, 4), (4096, 8), (4097, 24)],
    }
    for cfg, cases in want.items():
        for tokens, stages in cases:
            assert sched.get_num_stages(cfg, tokens) == stages, (cfg, tokens)
    with pytest.raises(ValueError, match="Unsupported number of stages"):
        sched.get_num_stages(8, 100)


def test_stage_layers_are_numpy_array_split():
    for layers, stages in itertools.product((1, 8, 24, 36, 48, 61), (1, 2, 4, 6, 8, 12, 16, 24)):
        if stages > layers:
            continue
        parts = np.array_split(np.arange(layers), stages)
        for s in range(stages):
            assert list(sched.stage_layers(layers, stages, s)) == parts[s].tolist()


def test_hand_worked_schedule():
    # two prompts arrive together: 600 + 300 = 900 tokens -> 2 stages of a 4-stage setup,
    # 8 layers -> layers 0-3 then 4-7.  The last stage samples the first token of both;
    # A (3 tokens) decodes twice more, B (2 tokens) once more.
    reqs = [sched.Request(600, 3), sched.Request(300, 2)]
    shapes = sched.simulate(reqs, num_layers=8, configured_stages=4, max_num_batched_tokens=1024)
    got = [(s.decode_tokens, s.prefill_tokens, s.stage, s.num_stages, list(s.prefill_layers)) for s in shapes]
    assert got == [
        (0, 900, 0, 2, [0, 1, 2, 3]),
        (0, 900, 1, 2, [4, 5, 6, 7]),
        (2, 0, -1, -1, []),
        (1, 0, -1, -1, []),
    ]
    assert shapes[0].layer_tokens(2) == 900 and shapes[0].layer_tokens(5) == 0
    assert sched.moe_call_sizes(shapes, 8) == {900: 8, 2: 8, 1: 8}


def test_token_budget_cuts_a_prompt_and_continues_it():
    # budget 1024: the 1500-token prompt runs as 1024 (4 stages... of a 16-stage setup: 2) then 476 (1 stage)
    shapes = sched.simulate([sched.Request(1500, 1)], num_layers=4, configured_stages=16,
                            max_num_batched_tokens=1024)
    assert [(s.prefill_tokens, s.stage, s.num_stages) for s in shapes] == [(1024, 0, 2), (1024, 1, 2), (476, 0, 1)]


def test_decodes_ride_along_and_late_arrivals_wait_for_the_group():
    # a long-running decode is present in every iteration; a request arriving while a
    # group is in flight is admitted only after the group's last stage
    reqs = [sched.Request(100, 50, 0), sched.Request(5000, 2, 1), sched.Request(200, 2, 3)]
    shapes = sched.simulate(reqs, num_layers=16, configured_stages=16, max_num_batched_tokens=8192)
    assert (shapes[0].prefill_tokens, shapes[0].num_stages) == (100, 1)
    big = [s for s in shapes if s.prefill_tokens == 5000]
    assert [s.stage for s in big] == list(range(16)) and all(s.decode_tokens == 1 for s in big)
    assert [s.index for s in big] == list(range(1, 17))
    nxt = shapes[17]
    assert (nxt.prefill_tokens, nxt.num_stages, nxt.decode_tokens) == (200, 1, 2)


def test_invariants_on_the_sharegpt_sample():
    lengths = sched.load_length_trace()
    assert len(lengths) == 2048 and lengths[0] == (74, 918) and lengths[3] == (2497, 918)
    reqs = sched.poisson_requests(lengths, 200, per_iteration=0.05, seed=1)
    L, cap_seqs, cap_tok = 48, 64, 8192
    shapes = sched.simulate(reqs, num_layers=L, configured_stages=16, max_num_seqs=cap_seqs,
                            max_num_batched_tokens=cap_tok)
    # every prompt token passes every layer exactly once
    per_layer = np.zeros(L, dtype=np.int64)
    for s in shapes:
        for l in s.prefill_layers:
            per_layer[l] += s.prefill_tokens
    assert (per_layer == sum(r.prompt_len for r in reqs)).all()
    # decode tokens: each request generates output_len tokens, the first at the end of its prefill
    assert sum(s.decode_tokens for s in shapes) == sum(r.output_len - 1 for r in reqs)
    # a group runs its stages in consecutive iterations, in order, with constant size
    runs = [list(g) for k, g in itertools.groupby(shapes, key=lambda s: s.num_stages > 0) if k]
    for run in runs:
        i = 0
        while i < len(run):
            n = run[i].num_stages
            grp = run[i:i + n]
            assert [s.stage for s in grp] == list(range(n))
            assert len({s.prefill_tokens for s in grp}) == 1
            assert grp[0].prefill_tokens <= cap_tok and n == sched.get_num_stages(16, grp[0].prefill_tokens)
            i += n
    assert all(s.decode_tokens <= cap_seqs for s in shapes)
    sizes = sched.moe_call_sizes(shapes, L)
    assert sum(sizes.values()) <= L * len(shapes) and min(sizes) >= 1
