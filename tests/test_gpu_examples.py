"""The one numeric claim of the example scripts (reference: examples/example.py:86): `flax_attention` with a block
mask and `flax_attention_pallas` with the bare mask_mod agree to two decimals for an ALiBi score_mod under a causal
sliding window of 10, fp16 [8,8,2048,64]; and the example itself runs to the end."""
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import flaxattention_amd as fa
from flaxattention_amd.masks import causal_mask, generate_sliding_window
from flaxattention_amd.mods import generate_alibi_bias
from oracle import o_alibi, o_sliding_window, ref_attention, rel_l2

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_both_front_ends_agree_to_two_decimals(dev):
    B, H, L, D = 8, 8, 2048, 64

    def normal(seed, length):
        g = torch.Generator().manual_seed(seed)
        return torch.randn(B, H, length, D, generator=g).to(torch.float16)
    key, query, value = normal(0, L), normal(1, L), normal(2, L)
    merged = fa.and_masks(causal_mask, generate_sliding_window(10))
    bm = fa.create_block_mask(merged, B, H, L, L, device=dev)
    alibi = generate_alibi_bias(H)
    qd, kd, vd = query.to(dev), key.to(dev), value.to(dev)
    out = fa.flax_attention(qd, kd, vd, score_mod=alibi, block_mask=bm)
    out_p = fa.flax_attention_pallas(qd, kd, vd, score_mod=alibi, mask_mod=merged)
    np.testing.assert_almost_equal(out.float().cpu().numpy(), out_p.float().cpu().numpy(), decimal=2)
    # and both are the dense path's result (one batch element against the oracle)
    want = ref_attention(query[:1], key[:1], value[:1], o_alibi(H), o_sliding_window(10))
    assert rel_l2(out[:1].cpu(), want) <= 1e-3 and rel_l2(out_p[:1].cpu(), want) <= 1e-3


def test_example_script_runs(dev):
    r = subprocess.run([sys.executable, os.path.join(ROOT, "examples", "example.py")], capture_output=True, text=True,
                       timeout=110)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    assert "agree to two decimals" in r.stdout
