"""HIP block-mask builder vs the CPU oracle: bit-exact integer outputs."""
import numpy as np
import pytest
import torch

import flaxattention_amd as fa
from flaxattention_amd.masks import causal_mask, generate_attention_sink, generate_sliding_window, offset_causal_mask
from flaxattention_amd.core.common import MaskMod, INT_MIN
from oracle import (o_attention_sink, o_causal_mask, o_full_masked, o_noop_mask, o_offset_causal, o_sink_window_lt,
                    o_sliding_window, ref_create_block_mask)

pytestmark = pytest.mark.gpu

FIELDS = ["kv_num_blocks", "kv_indices", "full_kv_num_blocks", "full_kv_indices",
          "q_num_blocks", "q_indices", "full_q_num_blocks", "full_q_indices"]


def check(bm, ref):
    for f in FIELDS:
        got = getattr(bm, f).cpu().numpy()
        assert got.dtype == np.int32
        assert got.shape == ref[f].shape, (f, got.shape, ref[f].shape)
        assert np.array_equal(got, ref[f]), f
    assert bm.BLOCK_SIZE == ref["BLOCK_SIZE"]
    assert bm.used_block_size == ref["used_block_size"]


def sink_lt(window, sink):
    # benchmark-config spelling: kv_idx < sink always visible
    return generate_attention_sink(window, sink - 1)


CASES = [
    ("causal_c1", causal_mask, o_causal_mask, 1, 4, 256, 256, 128),
    ("causal_c3", causal_mask, o_causal_mask, 2, 3, 2048, 2048, 128),
    ("causal_bs64", causal_mask, o_causal_mask, 1, 2, 512, 512, 64),
    ("causal_ragged", causal_mask, o_causal_mask, 1, 1, 300, 500, 128),
    ("causal_rect_blocks", causal_mask, o_causal_mask, 1, 2, 384, 512, (128, 64)),
    ("window", generate_sliding_window(10), o_sliding_window(10), 1, 1, 1024, 1024, 128),
    ("sink_ref", generate_attention_sink(300, 4), o_attention_sink(300, 4), 1, 2, 2048, 2048, 128),
    ("sink_c4", sink_lt(1024, 4), o_sink_window_lt(1024, 4), 1, 1, 8192, 8192, 128),
    ("noop", fa.noop_mask, o_noop_mask, 1, 1, 256, 384, 128),
    ("short_q", causal_mask, o_causal_mask, 4, 8, 64, 64, 128),
    ("decode_q1", offset_causal_mask(16383), o_offset_causal(16383), 1, 1, 1, 16384, 128),
    ("decode_q16", offset_causal_mask(16384 - 16), o_offset_causal(16384 - 16), 1, 1, 16, 16384, 128),
    ("decode_q64", offset_causal_mask(16384 - 64), o_offset_causal(16384 - 64), 2, 2, 64, 16384, 128),
]


@pytest.mark.parametrize("name,mask,omask,B,H,Q,KV,bs", CASES, ids=[c[0] for c in CASES])
def test_builder_matches_oracle(name, mask, omask, B, H, Q, KV, bs, dev):
    print(f"case {name} B{B} H{H} Q{Q} KV{KV} bs{bs}", flush=True)
    bm = fa.create_block_mask(mask, B, H, Q, KV, BLOCK_SIZE=bs, device=dev)
    ref = ref_create_block_mask(omask, B, H, Q, KV, BLOCK_SIZE=bs)
    check(bm, ref)


def test_fully_masked(dev):
    def fullmask(b, h, q_idx, kv_idx):
        return False
    bm = fa.create_block_mask(fullmask, 4, 8, 64, 64, device=dev)
    ref = ref_create_block_mask(o_full_masked, 4, 8, 64, 64)
    check(bm, ref)
    assert bm.sparsity() == 100.0


def test_python_callable_recognised_as_band(dev):
    def my_causal(b, h, q_idx, kv_idx):
        return q_idx >= kv_idx
    bm = fa.create_block_mask(my_causal, 1, 1, 512, 512, device=dev)
    assert bm.spec.bits is None and (bm.spec.lo, bm.spec.sink) == (0, -1)
    check(bm, ref_create_block_mask(o_causal_mask, 1, 1, 512, 512))


def test_python_callable_bitmap(dev):
    # depends on b and h, not a band: goes through the packed bitmap
    def weird(b, h, q_idx, kv_idx):
        return ((q_idx * 7 + kv_idx * 3 + h) % 11 < 6) & (kv_idx <= q_idx + 200 * b)
    bm = fa.create_block_mask(weird, 2, 3, 384, 640, device=dev)
    assert bm.spec.bits is not None
    check(bm, ref_create_block_mask(weird, 2, 3, 384, 640))

    def doc_mask(b, h, q_idx, kv_idx):  # document mask: block-diagonal, many full/empty tiles
        return (q_idx // 256) == (kv_idx // 256)
    bm = fa.create_block_mask(doc_mask, 1, 1, 1024, 1024, device=dev)
    check(bm, ref_create_block_mask(doc_mask, 1, 1, 1024, 1024))


def test_score_mod_as_mask(dev):
    # blockmask.py:307-315: a five-argument mod masks where it returns -inf
    def smod(score, b, h, q_idx, kv_idx):
        return torch.where(q_idx >= kv_idx, score, torch.full_like(score, -float("inf")))
    bm = fa.create_block_mask(smod, 1, 2, 256, 256, device=dev)
    check(bm, ref_create_block_mask(o_causal_mask, 1, 2, 256, 256))


def test_create_mask_matches_oracle(dev):
    """The public dense-mask helper (flaxattention/core/blockmask.py:277-322): a tagged mask, an untagged callable that
    looks at batch and head, a five-argument score_mod (masked where it returns -inf), and B = H = None."""
    from oracle import ref_create_mask

    def doc(b, h, q_idx, kv_idx):
        return ((q_idx // 40) == (kv_idx // 40)) & ((h + b) % 2 == 0)

    def as_score(score, b, h, q_idx, kv_idx):
        return torch.where(q_idx >= kv_idx, score, float("-inf"))
    for got_fn, want_fn, B, H in ((causal_mask, o_causal_mask, 2, 3), (doc, doc, 2, 3), (as_score, as_score, 1, 2),
                                  (generate_sliding_window(10), o_sliding_window(10), None, None)):
        got = fa.create_mask(got_fn, B, H, 100, 130, device=dev)
        want = ref_create_mask(want_fn, B, H, 100, 130)
        assert got.dtype == torch.bool and tuple(got.shape) == want.shape
        assert np.array_equal(got.cpu().numpy(), want)
    with pytest.raises(AssertionError):   # neither four nor five positional arguments (flaxattention/core/common.py:33)
        fa.create_mask(lambda a, b: a, 1, 1, 8, 8, device=dev)


def test_sparsity_and_repr(dev):
    bm = fa.create_block_mask(causal_mask, 1, 1, 2048, 2048, device=dev)
    assert abs(bm.sparsity() - 100 * (1 - 136 / 256)) < 1e-9
    assert "BlockMask(" in repr(bm) and "causal_mask" in repr(bm)
    assert bm.shape == (1, 1, 2048, 2048)
    t = bm.as_tuple()
    assert len(t) == 11 and t[8] == 128 and t[9] == 128 and t[10] is causal_mask


def test_from_kv_blocks_transposes(dev):
    bm = fa.create_block_mask(generate_sliding_window(200), 1, 2, 1024, 1024, device=dev)
    bm2 = fa.BlockMask.from_kv_blocks(bm.kv_num_blocks, bm.kv_indices, bm.full_kv_num_blocks, bm.full_kv_indices,
                                      mask_mod=bm.mask_mod)
    for f in ["q_num_blocks", "q_indices", "full_q_num_blocks", "full_q_indices"]:
        assert torch.equal(getattr(bm, f), getattr(bm2, f)), f


@pytest.mark.parametrize("seed", range(12))
def test_band_closed_form_matches_brute_force(dev, seed):
    """Band masks are classified per tile from a closed-form row count; the oracle evaluates every
    (q, kv) pair.  Random band parameters, including unbounded sides, sinks and offsets."""
    import random
    from flaxattention_amd.core.common import INT_MAX
    rnd = random.Random(50 + seed)
    Q, KV = rnd.choice([(256, 384), (300, 200), (512, 512), (64, 1000)])
    lo = rnd.choice([INT_MIN, 0, -17, 5, 130])
    hi = rnd.choice([INT_MAX, 10, 128, 333, max(lo, 0) + 40])
    sink = rnd.choice([-1, 0, 3, 127, 200])
    off = rnd.choice([0, 0, KV - Q, 13])
    bs = rnd.choice([128, 64, (128, 64)])
    print(f"band lo={lo} hi={hi} sink={sink} off={off} Q{Q} KV{KV} bs{bs}", flush=True)
    mask = MaskMod(lo, hi, sink, off, name="band")

    def omask(b, h, q_idx, kv_idx):
        d = q_idx + off - kv_idx
        return (d >= lo) & ((d <= hi) | (kv_idx <= sink))
    bm = fa.create_block_mask(mask, 1, 2, Q, KV, BLOCK_SIZE=bs, device=dev)
    check(bm, ref_create_block_mask(omask, 1, 2, Q, KV, BLOCK_SIZE=bs))


def test_head_and_batch_dependent_callable_at_config4_size(dev):
    """An untagged callable that depends on the batch and the head index, at [4,16,8192,8192]: the dense mask would be
    4.3 GB of booleans; it is evaluated in slabs and packed straight into bitmap words, so that building the block
    mask stays below 1 GiB of device memory, and the lists are the oracle's bit for bit."""
    import flaxattention_amd as fa
    B, H, L = 4, 16, 8192

    def mask(b, h, q_idx, kv_idx):
        return (q_idx >= kv_idx) & (((q_idx - kv_idx) <= 256 * (h + 1) + 64 * b) | (kv_idx < 4))
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats(dev)
    base = torch.cuda.memory_allocated(dev)
    bm = fa.create_block_mask(mask, B, H, L, L, device=dev)
    torch.cuda.synchronize()
    peak = torch.cuda.max_memory_allocated(dev) - base
    print(f"  peak device memory while building: {peak / 2 ** 20:.0f} MiB", flush=True)
    assert peak < 2 ** 30
    assert bm.spec.bits is not None and tuple(bm.spec.bits.shape) == (B, H, L, L // 32)
    for b0, h0 in ((0, 0), (3, 15), (2, 5)):
        ref = ref_create_block_mask(lambda b, h, q, kv: mask(b + b0, h + h0, q, kv), 1, 1, L, L)
        for f in ("kv_num_blocks", "kv_indices", "full_kv_num_blocks", "full_kv_indices", "q_num_blocks", "q_indices",
                  "full_q_num_blocks", "full_q_indices"):
            assert (getattr(bm, f)[b0, h0].cpu().numpy() == ref[f][0, 0]).all(), (f, b0, h0)
