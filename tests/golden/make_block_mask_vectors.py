"""Writes tests/golden/block_mask_vectors.json.

The vectors come from torch.nn.attention.flex_attention.create_block_mask run on
the CPU -- the PyTorch original of the algorithm the reference re-implements in
flaxattention/core/blockmask.py:253-455 -- so they are independent of this
repository's oracle and of its HIP builder.  Nothing from the reference tree is
imported or executed.  Run from the repository root:

    python tests/golden/make_block_mask_vectors.py
"""
import json
import os

import torch
from torch.nn.attention.flex_attention import create_block_mask

CASES = {
    "causal_B1_H4_256": dict(B=1, H=4, Q=256, KV=256),
    "causal_B1_H1_2048": dict(B=1, H=1, Q=2048, KV=2048),
    "window1024_sink_lt4_8192": dict(B=1, H=1, Q=8192, KV=8192),
    "sink_le4_window300_2048": dict(B=1, H=1, Q=2048, KV=2048),
    "sliding_window_10_1024": dict(B=1, H=1, Q=1024, KV=1024),
    "causal_rect_384x640": dict(B=1, H=1, Q=384, KV=640),
}


def mask_for(name):
    if name.startswith("causal"):
        return lambda b, h, q, kv: q >= kv
    if name.startswith("window1024_sink_lt4"):
        return lambda b, h, q, kv: ((kv < 4) | (q - kv <= 1024)) & (q >= kv)
    if name.startswith("sink_le4_window300"):
        return lambda b, h, q, kv: ((kv <= 4) | (q - kv <= 300)) & (q >= kv)
    if name.startswith("sliding_window_10"):
        return lambda b, h, q, kv: (q - kv <= 10) & (q >= kv)
    raise KeyError(name)


def main():
    out = {}
    for name, c in CASES.items():
        bm = create_block_mask(mask_for(name), c["B"], c["H"], c["Q"], c["KV"], device="cpu", BLOCK_SIZE=128)
        entry = dict(c)
        entry["BLOCK_SIZE"] = 128
        for f in ("kv_num_blocks", "kv_indices", "full_kv_num_blocks", "full_kv_indices",
                  "q_num_blocks", "q_indices", "full_q_num_blocks", "full_q_indices"):
            t = getattr(bm, f)
            # one (b, h) slice is enough: these masks do not depend on b or h
            entry[f] = t[0, 0].to(torch.int32).tolist()
        out[name] = entry
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "block_mask_vectors.json")
    with open(path, "w") as fh:
        json.dump(out, fh, separators=(",", ":"))
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
