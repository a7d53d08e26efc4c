#!/usr/bin/env python3
"""Writes the golden fixtures of this directory from the CPU oracle.

The reference ships no tests, fixtures or golden vectors for the MoE path, so
these vectors pin THIS build's oracle against silent change: they are produced
by oracle/moe_oracle.{c,py} (itself pinned by tests/test_oracle.py against the
worked examples in the reference's comments, closed forms and brute force) on
the seeded workloads of layered-prefill_amd/workloads.py.

    python tests/golden/make_golden.py

  tiny_fp32.npz      config 1 in full: routing, alignment (block 16) and the
                     fp32 layer output
  routing_hashes.json sha256 of topk_ids / topk_weights / alignment outputs of
                     configs 2 and 3 plus a few sampled rows
"""
import hashlib
import importlib
import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)


def sha(t: torch.Tensor) -> str:
    return hashlib.sha256(t.contiguous().numpy().tobytes()).hexdigest()


def main() -> None:
    moe = importlib.import_module("layered-prefill_amd")
    oracle = importlib.import_module("oracle.moe_oracle")
    wl = moe.workloads

    shape, x, logits, w13, w2 = wl.make_config("tiny_fp32")
    tw, ids, tei = oracle.fused_topk(x, logits, shape.top_k, True)
    s, e, n = oracle.moe_align_block_size(ids, 16, shape.experts)
    out = oracle.fused_experts_ref(x, w13, w2, tw, ids)
    np.savez_compressed(os.path.join(HERE, "tiny_fp32.npz"), topk_weights=tw.numpy(),
                        topk_ids=ids.numpy(), token_expert_indices=tei.numpy(),
                        sorted_token_ids=s.numpy(), expert_ids=e.numpy(),
                        num_tokens_post_pad=n.numpy(), out=out.numpy())

    hashes = {}
    for name, bm in (("decode_256", 32), ("layered_8192p_256d", 256)):
        shape, tokens, seed, dtype = wl.CONFIGS[name]
        x, logits = wl.make_inputs(shape, tokens, seed, dtype)
        tw, ids, tei = oracle.fused_topk(x, logits, shape.top_k, True)
        s, e, n = oracle.moe_align_block_size(ids, bm, shape.experts)
        hashes[name] = {
            "block_size": bm, "topk_ids": sha(ids), "topk_weights": sha(tw),
            "token_expert_indices": sha(tei), "sorted_token_ids": sha(s), "expert_ids": sha(e),
            "num_tokens_post_pad": int(n.item()),
            "active_experts": int(torch.unique(ids).numel()),
            "sample_rows": {str(r): {"ids": ids[r].tolist(), "weights_bits": tw[r].view(torch.int32).tolist()}
                            for r in (0, tokens // 2, tokens - 1)},
        }
    with open(os.path.join(HERE, "routing_hashes.json"), "w") as f:
        json.dump(hashes, f, indent=1, sort_keys=True)


if __name__ == "__main__":
    main()
