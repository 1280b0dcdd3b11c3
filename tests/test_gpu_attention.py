"""HIP attention kernels vs the CPU oracle (same seeded inputs on both sides).

Tolerances (stated by the build goal): fp32 max-abs and relative-L2 1e-4;
fp16/bf16 max-abs 2e-2 and relative-L2 1e-3.  The faithful ("strict") kernels
and the fused MFMA kernels in their default numerics (fp16: "fast", bf16:
"parity") are held to those numbers against the strict oracle.  Only the
explicitly requested kernel_options={"numerics": "fast"} on bf16 inputs --
one-pass softmax with the unnormalised P rounded to bf16, which sits at the
bf16 quantisation floor of about 3e-3 -- is held to 6e-3, with max-abs scaled
by the largest reference entry (one bf16 ulp at |x| >= 4 is 3.1e-2).
"""
import math

import pytest
import torch

import flaxattention_amd as fa
from flaxattention_amd.masks import causal_mask, generate_attention_sink, generate_sliding_window, offset_causal_mask
from flaxattention_amd.mods import (checkerboard, generate_alibi_bias, generate_checkerboard, generate_rel_bias,
                                    generate_tanh_softcap)
from oracle import (max_abs, o_alibi, o_alibi_config, o_attention_sink, o_causal_mask, o_checkerboard,
                    o_checkerboard_kv, o_full_masked, o_offset_causal, o_rel_bias, o_sink_window_lt,
                    o_sliding_window, o_tanh_softcap, ref_attention, ref_attention_bwd, rel_l2, seeded_qkv)

pytestmark = pytest.mark.gpu

TOL = {torch.float32: (1e-4, 1e-4), torch.float16: (2e-2, 1e-3), torch.bfloat16: (2e-2, 1e-3)}


def tol_for(dtype, fast_bf16):
    ma, rl = TOL[dtype]
    if fast_bf16 and dtype == torch.bfloat16:
        rl = 6e-3
    return ma, rl


def ulp_at(x, dtype):
    """Spacing of `dtype` at magnitude x."""
    if dtype == torch.float32 or x <= 0.0:
        return 0.0
    bits = 7 if dtype == torch.bfloat16 else 10
    return 2.0 ** (math.floor(math.log2(x)) - bits)


def close(got, want, dtype, what, fast_bf16=False, scale_maxabs=False):
    """fast_bf16: the result comes from the explicitly requested fast numerics on bf16 inputs."""
    ma, rl = tol_for(dtype, fast_bf16)
    got = got.detach().cpu()
    a, r = max_abs(got, want), rel_l2(got, want)
    if scale_maxabs or (fast_bf16 and dtype == torch.bfloat16):
        # gradients grow with the sequence length: where the largest reference entry is so large that ONE unit in
        # the last place of the dtype exceeds the absolute bound (bf16: 3.1e-2 from |x| = 4, fp16: from |x| = 32),
        # two correctly rounded results may differ by that much, and the bound is that unit instead
        # (the fast bf16 numerics, whose P and dS carry 8 bits, get two such units)
        ma = max(ma, (2.0 if fast_bf16 else 1.0) * ulp_at(want.abs().max().item(), dtype))
    print(f"  {what}: max-abs {a:.3e} rel-L2 {r:.3e} (tol {ma:.1e} / {rl:.1e})", flush=True)
    assert a <= ma, f"{what}: max-abs {a} > {ma}"
    assert r <= rl, f"{what}: rel-L2 {r} > {rl}"


def run(dev, dtype, B, Hq, Hkv, Lq, Lkv, D, score=None, oscore=None, mask=None, omask=None, Dv=None,
        opts=None, grad=True, strict=True, use_block_mask=True, scale=None, pallas=False, scale_maxabs=False):
    q, k, v = seeded_qkv(B, Hq, Hkv, Lq, Lkv, D, dtype, Dv)
    g = torch.Generator().manual_seed(3)
    d_o = torch.randn((B, Hq, Lq, Dv or D), generator=g).to(dtype)
    opts = dict(opts or {})
    fused = (not strict) and opts.get("numerics") == "fast" and dtype == torch.bfloat16   # widened bounds: fast bf16 only
    if strict:
        opts["strict"] = True
    qd, kd, vd = (t.to(dev).requires_grad_(grad) for t in (q, k, v))
    gqa = Hq != Hkv
    if pallas:
        out = fa.flax_attention_pallas(qd, kd, vd, score_mod=score, mask_mod=mask, enable_gqa=gqa,
                                       sm_scale=scale, kernel_options=opts)
        lse = None
    else:
        bm = None
        if mask is not None and use_block_mask:
            bm = fa.create_block_mask(mask, B, Hq, Lq, Lkv, device=dev)
        out, lse = fa.flax_attention(qd, kd, vd, score_mod=score, block_mask=bm, enable_gqa=gqa, return_lse=True,
                                     scale=scale, kernel_options=opts)
    want, want_lse = ref_attention(q, k, v, oscore, omask, scale=scale, strict=True, return_lse=True)
    close(out, want, dtype, "O", fused)
    if lse is not None:
        lse_c = lse.detach().cpu()
        dead = torch.isneginf(want_lse)
        assert torch.equal(torch.isneginf(lse_c), dead)
        assert max_abs(lse_c[~dead], want_lse[~dead]) <= (1e-4 if dtype == torch.float32 else 2e-2)
    if grad:
        out.backward(d_o.to(dev))
        wq, wk, wv = ref_attention_bwd(q, k, v, d_o, oscore, omask, scale=scale, strict=True)
        close(qd.grad, wq, dtype, "dQ", fused, scale_maxabs)
        close(kd.grad, wk, dtype, "dK", fused, scale_maxabs)
        close(vd.grad, wv, dtype, "dV", fused, scale_maxabs)
    return out


# ---- the reference's own test cases (tests/attention_test.py), shapes B4 H8 L64 D32 fp32 ----
def test_ref_equivalence(dev):                      # attention_test.py:23-63
    run(dev, torch.float32, 4, 8, 8, 64, 64, 32)


def test_ref_fully_masked(dev):                     # attention_test.py:65-96
    def fullmask(b, h, q_idx, kv_idx):
        return False
    out = run(dev, torch.float32, 4, 8, 8, 64, 64, 32, mask=fullmask, omask=o_full_masked)
    assert torch.count_nonzero(out).item() == 0


def test_ref_pallas_fully_masked(dev):              # attention_test.py:98-129
    def fullmask(b, h, q_idx, kv_idx):
        return False
    out = run(dev, torch.float32, 4, 8, 8, 64, 64, 32, mask=fullmask, omask=o_full_masked, pallas=True)
    assert torch.count_nonzero(out).item() == 0


def test_ref_pallas_equivalence(dev):               # attention_test.py:131-171
    run(dev, torch.float32, 4, 8, 8, 64, 64, 32, pallas=True)


def test_ref_decoding_alibi(dev):                   # attention_test.py:173-232
    run(dev, torch.float32, 4, 8, 8, 1, 64, 32, score=generate_alibi_bias(8), oscore=o_alibi(8))


def test_ref_pallas_decoding_alibi(dev):            # attention_test.py:234-293
    run(dev, torch.float32, 4, 8, 8, 1, 64, 32, score=generate_alibi_bias(8), oscore=o_alibi(8), pallas=True)


def test_ref_gqa(dev):                              # attention_test.py:295-324 (values checked too)
    out = run(dev, torch.float32, 4, 8, 2, 64, 64, 32)
    assert out.shape == (4, 8, 64, 32)


def test_ref_score_mod(dev):                        # attention_test.py:326-352
    run(dev, torch.float32, 4, 8, 8, 64, 64, 32, score=generate_alibi_bias(8), oscore=o_alibi(8))


# ---- benchmark configuration 1: fp32 [1,4,256,64], causal at 128x128, forward ----
def test_config1_fp32_causal(dev):
    run(dev, torch.float32, 1, 4, 4, 256, 256, 64, mask=causal_mask, omask=o_causal_mask)


# ---- float32 on the matrix cores: what float32 inputs run on unless kernel_options["strict"] is set ----
def family(dev, dtype, B, Hq, Hkv, Lq, Lkv, D, mask=None, backward=False, opts=None):
    q = torch.zeros((B, Hq, Lq, D), dtype=dtype, device=dev)
    k = torch.zeros((B, Hkv, Lkv, D), dtype=dtype, device=dev)
    bm = fa.create_block_mask(mask, B, Hq, Lq, Lkv, device=dev) if mask is not None else None
    return fa.kernel_family(q, k, k, block_mask=bm, kernel_options=opts, backward=backward)


def test_kernel_family_query(dev):
    for bwd in (False, True):
        assert family(dev, torch.float32, 1, 4, 4, 256, 256, 64, causal_mask, bwd) == "mfma_f32"
        assert family(dev, torch.float32, 1, 4, 4, 256, 256, 32, causal_mask, bwd) == "mfma_f32"   # zero-padded to 64
        assert family(dev, torch.float32, 1, 4, 4, 256, 256, 64, causal_mask, bwd, {"strict": True}) == "generic"
        assert family(dev, torch.float32, 1, 4, 4, 256, 256, 256, None, bwd) == "generic"
        assert family(dev, torch.float16, 1, 4, 4, 256, 256, 64, causal_mask, bwd) == "mfma_16bit"
        assert family(dev, torch.bfloat16, 1, 4, 2, 100, 300, 128, None, bwd) == "mfma_16bit"
        assert family(dev, torch.bfloat16, 1, 4, 4, 256, 256, 64, None, bwd, {"backend": "generic"}) == "generic"
        assert family(dev, torch.bfloat16, 1, 4, 4, 256, 256, 256, causal_mask, bwd) == "mfma_16bit"
        assert family(dev, torch.float16, 1, 4, 2, 100, 300, 160, None, bwd) == "mfma_16bit"          # zero-padded to 192
        assert family(dev, torch.float16, 1, 4, 4, 256, 256, 320, None, bwd) == "generic"
    # a score_mod outside the functor families is linearised into dense tables, which the matrix-core kernels read
    q = torch.zeros((1, 2, 64, 64), dtype=torch.float16, device=dev)
    assert fa.kernel_family(q, q, q, score_mod=lambda s, b, h, qi, ki: s * s) == "mfma_16bit"


SCORES_F32 = [
    ("identity", None, None),
    ("checker_diff", checkerboard, o_checkerboard),
    ("checker_kv", generate_checkerboard(2.0, 0.5, "kv"), o_checkerboard_kv),
    ("alibi_cfg", generate_alibi_bias(4, sign=-1.0), o_alibi_config(4)),
    ("softcap", generate_tanh_softcap(5.0), o_tanh_softcap(5.0)),
    ("relbias", generate_rel_bias(0.03), o_rel_bias(0.03)),
]


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("name,score,oscore", SCORES_F32, ids=[s[0] for s in SCORES_F32])
def test_fp32_mfma_scores(dev, D, name, score, oscore):
    print(f"case fp32 mfma {name} D{D}", flush=True)
    run(dev, torch.float32, 2, 4, 4, 192, 256, D, score=score, oscore=oscore, mask=causal_mask, omask=o_causal_mask,
        strict=False)


MASKS_F32 = [
    ("window", generate_sliding_window(40), o_sliding_window(40)),
    ("sink", generate_attention_sink(50, 4), o_attention_sink(50, 4)),
    ("sink_lt", generate_attention_sink(50, 3), o_sink_window_lt(50, 4)),
    ("offset", offset_causal_mask(64), o_offset_causal(64)),
]


@pytest.mark.parametrize("name,mask,omask", MASKS_F32, ids=[m[0] for m in MASKS_F32])
def test_fp32_mfma_masks(dev, name, mask, omask):
    print(f"case fp32 mfma mask {name}", flush=True)
    run(dev, torch.float32, 1, 2, 2, 300, 450, 64, mask=mask, omask=omask, strict=False)


def test_fp32_mfma_config1(dev):
    """Benchmark configuration 1 on the path float32 takes by default."""
    run(dev, torch.float32, 1, 4, 4, 256, 256, 64, mask=causal_mask, omask=o_causal_mask, strict=False)


def test_fp32_mfma_bitmap_mask_and_dead_rows(dev):
    def weird(b, h, q_idx, kv_idx):
        return ((q_idx * 7 + kv_idx * 3 + h) % 11 < 6) & (q_idx % 5 != 0)
    run(dev, torch.float32, 2, 3, 3, 100, 150, 32, mask=weird, omask=weird, strict=False)


def test_fp32_mfma_gqa_ragged_no_lists(dev):
    run(dev, torch.float32, 2, 8, 2, 77, 203, 64, Dv=32, mask=causal_mask, omask=o_causal_mask,
        score=generate_alibi_bias(8, -1.0), oscore=o_alibi_config(8), strict=False, opts={"tile_lists": False})
    run(dev, torch.float32, 1, 4, 1, 130, 140, 128, scale=0.05, strict=False)


def test_fp32_mfma_arbitrary_score_mod(dev):
    """A score_mod outside the functor families (linearised into dense tables) on float32 inputs."""
    def squash(score, b, h, q_idx, kv_idx):
        return score * score * 0.1 + score
    run(dev, torch.float32, 1, 2, 2, 96, 160, 64, score=squash, oscore=squash, mask=causal_mask, omask=o_causal_mask,
        strict=False)


# ---- 16-bit head sizes above 128 (192 and 256, others zero-padded to them) on the matrix cores ----
WIDE = [
    ("identity", None, None, causal_mask, o_causal_mask),
    ("checker_kv", generate_checkerboard(2.0, 0.5, "kv"), o_checkerboard_kv, None, None),
    ("alibi_cfg", generate_alibi_bias(4, sign=-1.0), o_alibi_config(4), causal_mask, o_causal_mask),
    ("softcap_sink", generate_tanh_softcap(5.0), o_tanh_softcap(5.0), generate_attention_sink(50, 4), o_attention_sink(50, 4)),
]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
@pytest.mark.parametrize("D", [192, 256])
@pytest.mark.parametrize("name,score,oscore,mask,omask", WIDE, ids=[w[0] for w in WIDE])
def test_wide_heads_default_numerics(dev, dtype, D, name, score, oscore, mask, omask):
    """fp16 in its default ("fast") and bf16 in its default ("parity") numerics at the stated tolerance."""
    print(f"case wide {name} {dtype} D{D}", flush=True)
    run(dev, dtype, 2, 4, 4, 192, 256, D, score=score, oscore=oscore, mask=mask, omask=omask, strict=False)


def test_wide_heads_other_modes(dev):
    run(dev, torch.float16, 1, 2, 2, 160, 200, 256, mask=causal_mask, omask=o_causal_mask, strict=False,
        opts={"numerics": "parity"})
    run(dev, torch.bfloat16, 1, 2, 2, 160, 200, 256, mask=causal_mask, omask=o_causal_mask, strict=False,
        opts={"numerics": "fast"})


def test_wide_heads_gqa_ragged_padded_bitmap(dev):
    def weird(b, h, q_idx, kv_idx):
        return ((q_idx * 7 + kv_idx * 3 + h) % 11 < 6) & (q_idx % 5 != 0)
    run(dev, torch.bfloat16, 2, 8, 2, 77, 203, 160, mask=causal_mask, omask=o_causal_mask,
        score=generate_alibi_bias(8, -1.0), oscore=o_alibi_config(8), strict=False, opts={"tile_lists": False})
    run(dev, torch.float16, 2, 3, 3, 100, 150, 224, Dv=200, mask=weird, omask=weird, strict=False)


SPLIT_CASES = [
    # name, dtype, D, B, Hq, Hkv, Lq, kernel_options
    ("f32-64", torch.float32, 64, 1, 2, 2, 5, None),
    ("f32-128-gqa-two-tiles", torch.float32, 128, 1, 4, 2, 130, None),
    ("bf16-192-parity", torch.bfloat16, 192, 2, 2, 2, 3, None),
    ("f16-192-fast", torch.float16, 192, 1, 3, 3, 33, None),
    ("f16-256-forward-kernel", torch.float16, 256, 1, 2, 2, 40, {"decode": False}),
    ("bf16-256-fast-no-lists", torch.bfloat16, 256, 1, 2, 1, 17, {"numerics": "fast", "tile_lists": False, "decode": False}),
    # the tuned 16-bit kernels (D 64 / 128)
    ("f16-64", torch.float16, 64, 1, 2, 2, 100, None),
    ("f16-64-short-no-lists", torch.float16, 64, 2, 2, 2, 7, {"decode": False, "tile_lists": False}),
    ("bf16-128-parity-gqa", torch.bfloat16, 128, 1, 4, 2, 150, None),
    ("bf16-64-fast", torch.bfloat16, 64, 1, 3, 3, 129, {"numerics": "fast"}),
    ("f16-128-parity", torch.float16, 128, 1, 2, 2, 33, {"numerics": "parity", "decode": False}),
]


@pytest.mark.parametrize("name,dtype,D,B,Hq,Hkv,Lq,opts", SPLIT_CASES, ids=[c[0] for c in SPLIT_CASES])
def test_forward_split_over_keys(dev, name, dtype, D, B, Hq, Hkv, Lq, opts):
    """Few query rows against many keys: the matrix-core forward is split over the keys and merged (one-pass and both
    passes of the parity numerics), ALiBi + offset-causal with a ragged key length; in a second call the first rows
    see no key at all (lse -inf, O = 0)."""
    from flaxattention_amd import _lib
    from flaxattention_amd.core.attention import _make_plan
    print(f"case split forward {name}", flush=True)
    Lkv, off = 2100, 2100 - Lq - 2   # row i sees keys <= i + off: the window ends two keys before the end
    mask, omask = offset_causal_mask(off), o_offset_causal(off)
    run(dev, dtype, B, Hq, Hkv, Lq, Lkv, D, score=generate_alibi_bias(Hq, -1.0), oscore=o_alibi_config(Hq),
        mask=mask, omask=omask, strict=False, opts=opts)
    dead_off = -2                     # rows 0 and 1 see nothing
    run(dev, dtype, B, Hq, Hkv, Lq, Lkv, D, mask=offset_causal_mask(dead_off), omask=o_offset_causal(dead_off),
        strict=False, opts=opts, grad=False)
    # the library does ask for room for the partial results of such a call
    q, k, v = (t.to(dev) for t in seeded_qkv(B, Hq, Hkv, Lq, Lkv, D, dtype))
    plan = _make_plan(q, k, v, None, None, None, 1.0, opts)
    o = torch.empty_like(q)
    nbytes = _lib.lib().flexattn_fwd_workspace_bytes(plan.params(q, k, v, o))
    assert nbytes >= 2 * B * Hq * Lq * (D + 2) * 4


def test_forward_split_unrounded_equals_unsplit(dev):
    """The "unrounded" numerics over split key ranges against the same call without a workspace (one pass over all
    keys), through the C ABI; a causal bitmap-free band mask with tile lists."""
    from flaxattention_amd import _lib
    from flaxattention_amd.core.attention import _make_plan
    L = _lib.lib()
    B, H, Lq, Lkv, D = 1, 2, 90, 3000, 128
    q, k, v = (t.to(dev) for t in seeded_qkv(B, H, H, Lq, Lkv, D, torch.bfloat16))
    bm = fa.create_block_mask(offset_causal_mask(Lkv - Lq), B, H, Lq, Lkv, device=dev)
    plan = _make_plan(q, k, v, generate_alibi_bias(H, -1.0), bm, None, D ** -0.5, {"numerics": "unrounded", "decode": False})
    outs = []
    stream = torch.cuda.current_stream().cuda_stream
    for with_ws in (False, True):
        o = torch.empty_like(q)
        lse = torch.empty((B, H, Lq), dtype=torch.float32, device=dev)
        p = plan.params(q, k, v, o)
        n = L.flexattn_fwd_workspace_bytes(p)
        assert n > 0
        ws = torch.empty(n, dtype=torch.uint8, device=dev) if with_ws else None
        rc = L.flexattn_fwd(p, q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr(),
                            ws.data_ptr() if with_ws else None, stream)
        assert rc == 0, L.flexattn_last_error()
        torch.cuda.synchronize()
        outs.append((o.float().cpu(), lse.cpu()))
    assert max_abs(outs[0][0], outs[1][0]) <= 4e-3 and rel_l2(outs[1][0], outs[0][0]) <= 1e-3
    assert max_abs(outs[0][1], outs[1][1]) <= 1e-4


# ---- faithful kernels, 16-bit, every functor ----
SCORES = [
    ("identity", None, None),
    ("checker_diff", checkerboard, o_checkerboard),
    ("checker_kv", generate_checkerboard(2.0, 0.5, "kv"), o_checkerboard_kv),
    ("alibi_ref", generate_alibi_bias(4), o_alibi(4)),
    ("alibi_cfg", generate_alibi_bias(4, sign=-1.0), o_alibi_config(4)),
    ("softcap", generate_tanh_softcap(5.0), o_tanh_softcap(5.0)),
    ("relbias", generate_rel_bias(0.03), o_rel_bias(0.03)),
]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
@pytest.mark.parametrize("name,score,oscore", SCORES, ids=[s[0] for s in SCORES])
def test_strict_scores(dev, dtype, name, score, oscore):
    print(f"case strict {name} {dtype}", flush=True)
    big = name == "alibi_ref"  # (q-kv)*slope grows the gradients well past 1
    run(dev, dtype, 2, 4, 4, 192, 256, 64, score=score, oscore=oscore, mask=causal_mask, omask=o_causal_mask,
        scale_maxabs=big)


MASKS = [
    ("window", generate_sliding_window(40), o_sliding_window(40)),
    ("sink", generate_attention_sink(50, 4), o_attention_sink(50, 4)),
    ("sink_lt", generate_attention_sink(50, 3), o_sink_window_lt(50, 4)),
    ("offset", offset_causal_mask(64), o_offset_causal(64)),
]


@pytest.mark.parametrize("name,mask,omask", MASKS, ids=[m[0] for m in MASKS])
def test_strict_masks(dev, name, mask, omask):
    print(f"case strict mask {name}", flush=True)
    run(dev, torch.bfloat16, 1, 2, 2, 192, 256, 32, mask=mask, omask=omask)


def test_strict_bitmap_mask_and_dead_rows(dev):
    def weird(b, h, q_idx, kv_idx):
        return ((q_idx * 7 + kv_idx * 3 + h) % 11 < 6) & (q_idx % 5 != 0)
    run(dev, torch.float32, 2, 3, 3, 100, 150, 32, mask=weird, omask=weird)


def test_strict_gqa_dv_ragged(dev):
    run(dev, torch.float16, 2, 8, 2, 77, 203, 64, Dv=32, mask=causal_mask, omask=o_causal_mask,
        score=generate_alibi_bias(8, -1.0), oscore=o_alibi_config(8))


def test_strict_scale_and_d128(dev):
    run(dev, torch.bfloat16, 1, 2, 1, 130, 140, 128, scale=0.05, score=generate_tanh_softcap(50.0),
        oscore=o_tanh_softcap(50.0))


def test_mask_without_block_mask_pallas(dev):
    run(dev, torch.float32, 1, 2, 2, 96, 96, 32, mask=fa.and_masks(causal_mask, generate_sliding_window(10)),
        omask=o_sliding_window(10), score=generate_alibi_bias(2), oscore=o_alibi(2), pallas=True)


def test_untagged_mask_lowering_follows_captured_tensor(dev):
    """flax_attention_pallas(mask_mod=callable): the dense lowering of the callable is reused from call to call
    and redone when the tensor it captures is updated in place or the closure variable is rebound."""
    q, k, v = seeded_qkv(1, 2, 2, 96, 96, 64, torch.float16)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    doc_cpu = torch.arange(96) // 24
    doc = doc_cpu.to(dev)

    def doc_mask(b, h, q_idx, kv_idx):
        d = doc if q_idx.is_cuda else doc_cpu
        return d[q_idx.long()] == d[kv_idx.long()]
    for step in range(3):
        if step == 1:
            doc.copy_(torch.arange(96, device=dev) // 40)
            doc_cpu = torch.arange(96) // 40
        if step == 2:
            doc_cpu = torch.arange(96) // 7
            doc = doc_cpu.to(dev)
        out = fa.flax_attention_pallas(qd, kd, vd, mask_mod=doc_mask)
        again = fa.flax_attention_pallas(qd, kd, vd, mask_mod=doc_mask)
        want = ref_attention(q, k, v, None, doc_mask, strict=True)
        assert rel_l2(out.cpu(), want) <= 1e-3 and torch.equal(out, again), f"step {step}"


def test_bhln_false_layout(dev):
    q, k, v = seeded_qkv(2, 4, 4, 64, 80, 32, torch.float32)
    want = ref_attention(q, k, v, None, o_causal_mask)
    qd, kd, vd = (t.transpose(1, 2).contiguous().to(dev) for t in (q, k, v))   # [B,L,H,D]
    out = fa.flax_attention_pallas(qd, kd, vd, mask_mod=causal_mask, bhln=False)
    assert out.shape == (2, 64, 4, 32)
    close(out.transpose(1, 2), want, torch.float32, "O bhln=False")


@pytest.mark.parametrize("dtype,D", [(torch.float32, 64), (torch.bfloat16, 256), (torch.float16, 128)],
                         ids=["f32_64", "bf16_256", "f16_128"])
def test_bhln_false_layout_read_in_place(dev, dtype, D):
    """[B,L,H,D] tensors reach every matrix-core kernel family through their strides, forward and backward."""
    q, k, v = seeded_qkv(2, 4, 4, 96, 160, D, dtype)
    d_o = torch.randn((2, 4, 96, D), generator=torch.Generator().manual_seed(3)).to(dtype)
    want = ref_attention(q, k, v, None, o_causal_mask)
    wq, wk, wv = ref_attention_bwd(q, k, v, d_o, None, o_causal_mask, strict=True)
    qd, kd, vd = (t.transpose(1, 2).contiguous().to(dev).requires_grad_(True) for t in (q, k, v))   # [B,L,H,D]
    out = fa.flax_attention_pallas(qd, kd, vd, mask_mod=causal_mask, bhln=False)
    assert out.shape == (2, 96, 4, D)
    close(out.transpose(1, 2), want, dtype, "O bhln=False")
    out.backward(d_o.transpose(1, 2).contiguous().to(dev))
    close(qd.grad.transpose(1, 2), wq, dtype, "dQ bhln=False")
    close(kd.grad.transpose(1, 2), wk, dtype, "dK bhln=False")
    close(vd.grad.transpose(1, 2), wv, dtype, "dV bhln=False")


@pytest.mark.parametrize("dtype,D", [(torch.float16, 64), (torch.bfloat16, 64), (torch.float32, 64), (torch.bfloat16, 192)],
                         ids=["f16_fast", "bf16_parity", "f32", "bf16_wide_parity"])
def test_train_step_replays_from_a_captured_graph(dev, dtype, D):
    """Forward and backward record into a HIP graph (no entry point synchronises, allocates outside the caller's
    allocator or records a memset): every replay, with eager steps between the replays, gives the eager step's bits."""
    print(f"case graph capture of a training step {dtype} D{D}", flush=True)
    B, H, L = 2, 4, 384
    g0 = torch.Generator(device="cpu").manual_seed(0)
    mk = lambda: torch.randn(B, H, L, D, generator=g0, dtype=torch.float32).to(dtype).to(dev)
    q, k, v = (mk().requires_grad_(True) for _ in range(3))
    d_o = mk()
    bm = fa.create_block_mask(causal_mask, 1, 1, L, L, device=dev)

    def step():
        out = fa.flax_attention(q, k, v, score_mod=generate_alibi_bias(H, -1.0), block_mask=bm)
        return (out,) + torch.autograd.grad(out, (q, k, v), d_o)
    side = torch.cuda.Stream()   # default priority; warm-up off the default stream as graph capture asks
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static = step()
    for i in range(3):
        with torch.no_grad():
            for t in (q, k, v):
                t.copy_(mk())
        graph.replay()
        eager = step()
        torch.cuda.synchronize()
        for name, a, b in zip(("O", "dQ", "dK", "dV"), static, eager):
            assert torch.equal(a, b), f"replay {i}: {name} differs from the eager step"


def test_untagged_score_mod_is_recognised(dev):
    def my_alibi(score, b, h, q_idx, kv_idx):
        return score + (q_idx - kv_idx) * torch.exp2(-((h + 1) * 8.0 / 8))
    run(dev, torch.float32, 1, 8, 8, 64, 64, 32, score=my_alibi, oscore=o_alibi(8))

    # the same bias with its slopes in a captured device tensor, for a single query row: the probe must stay
    # inside the real index ranges and run on the device, and still find the ALiBi family (fused kernels)
    from flaxattention_amd.core.common import resolve_score_mod
    from flaxattention_amd import _lib
    slopes = torch.exp2(-(torch.arange(8, device=dev) + 1.0))
    per_row = torch.zeros(1, device=dev)      # one entry per query row: q_idx 1.. would be out of range

    def slopes_alibi(score, b, h, q_idx, kv_idx):
        return score + (q_idx - kv_idx) * slopes[h.long()] + per_row[q_idx.long()]
    assert resolve_score_mod(slopes_alibi, 8, (2, 8, 1, 700), dev).kind == _lib.SCORE_ALIBI
    run(dev, torch.float16, 2, 8, 8, 1, 700, 64, score=slopes_alibi, oscore=o_alibi(8), strict=False, grad=False)

    def unknown(score, b, h, q_idx, kv_idx):
        return score * score
    # outside every family and not affine in the score: served by linearisation at the call's scores
    q, k, v = seeded_qkv(1, 2, 2, 16, 16, 32, torch.float32)
    out = fa.flax_attention(q.to(dev), k.to(dev), v.to(dev), score_mod=unknown)
    assert rel_l2(out.cpu(), ref_attention(q, k, v, unknown, None)) <= 1e-4


def test_errors(dev):
    q, k, v = (t.to(dev) for t in seeded_qkv(1, 4, 2, 16, 16, 32, torch.float32))
    with pytest.raises(ValueError):
        fa.flax_attention(q, k, v)                      # head mismatch without GQA
    with pytest.raises(ValueError):
        fa.flax_attention(q, k.half(), v)               # dtype mismatch
    with pytest.raises(NotImplementedError):
        fa.flax_attention(q[0], k[0], v[0])             # not 4-D
    with pytest.raises(ValueError):
        fa.flax_attention(q, k[..., :16], v, enable_gqa=True)   # E mismatch
    with pytest.raises(fa.FlexAttnError):
        fa.flax_attention(q.cpu(), k.cpu(), v.cpu(), enable_gqa=True)   # no CPU fallback
    with pytest.raises(RuntimeError):
        fa.and_masks(causal_mask, 3)


# ---- fused MFMA kernels (default path for fp16 / bf16, D in {64, 128}) ----
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("name,score,oscore", SCORES, ids=[s[0] for s in SCORES])
def test_fused_scores(dev, dtype, D, name, score, oscore):
    print(f"case fused {name} {dtype} D{D}", flush=True)
    big = name == "alibi_ref"
    run(dev, dtype, 2, 4, 4, 256, 320, D, score=score, oscore=oscore, mask=causal_mask, omask=o_causal_mask,
        strict=False, scale_maxabs=big)


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("name,score,oscore", SCORES, ids=[s[0] for s in SCORES])
def test_fused_fast_numerics_bf16(dev, D, name, score, oscore):
    """The explicitly requested fast numerics on bf16 inputs: the one case held to the widened bound."""
    print(f"case fused fast bf16 {name} D{D}", flush=True)
    run(dev, torch.bfloat16, 2, 4, 4, 256, 320, D, score=score, oscore=oscore, mask=causal_mask, omask=o_causal_mask,
        strict=False, opts={"numerics": "fast"})


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("name,score,oscore", SCORES, ids=[s[0] for s in SCORES])
def test_fused_parity_numerics_f16(dev, D, name, score, oscore):
    """The parity numerics on fp16 inputs (not their default): an order of magnitude inside the stated bound."""
    print(f"case fused parity f16 {name} D{D}", flush=True)
    big = name == "alibi_ref"
    run(dev, torch.float16, 2, 4, 4, 256, 320, D, score=score, oscore=oscore, mask=causal_mask, omask=o_causal_mask,
        strict=False, opts={"numerics": "parity"}, scale_maxabs=big)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("name,score,oscore", SCORES, ids=[s[0] for s in SCORES])
def test_fused_unrounded_numerics(dev, dtype, D, name, score, oscore):
    """kernel_options={"numerics": "unrounded"}: no internal round trip (S unrounded, P and dS carried as high and low
    parts, delta from an unrounded row sweep).  Held to the stated tolerance against the oracle WITHOUT the dense
    path's round trips (strict=False), the variant an XLA build that optimises them away would compute."""
    print(f"case fused unrounded {name} {dtype} D{D}", flush=True)
    B, Hq, Hkv, Lq, Lkv = 2, 4, 2, 256, 320
    q, k, v = seeded_qkv(B, Hq, Hkv, Lq, Lkv, D, dtype)
    d_o = torch.randn((B, Hq, Lq, D), generator=torch.Generator().manual_seed(3)).to(dtype)
    qd, kd, vd = (t.to(dev).requires_grad_(True) for t in (q, k, v))
    bm = fa.create_block_mask(causal_mask, B, Hq, Lq, Lkv, device=dev)
    out, lse = fa.flax_attention(qd, kd, vd, score_mod=score, block_mask=bm, enable_gqa=True, return_lse=True,
                                 kernel_options={"numerics": "unrounded"})
    out.backward(d_o.to(dev))
    want, want_lse = ref_attention(q, k, v, oscore, o_causal_mask, strict=False, return_lse=True)
    wq, wk, wv = ref_attention_bwd(q, k, v, d_o, oscore, o_causal_mask, strict=False)
    big = name == "alibi_ref"
    close(out, want, dtype, "O")
    assert max_abs(lse.detach().cpu(), want_lse) <= 2e-2
    close(qd.grad, wq, dtype, "dQ", scale_maxabs=big)
    close(kd.grad, wk, dtype, "dK", scale_maxabs=big)
    close(vd.grad, wv, dtype, "dV", scale_maxabs=big)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
@pytest.mark.parametrize("D", [192, 256])
def test_unrounded_numerics_at_wide_heads(dev, dtype, D):
    """192- and 256-wide heads in the "unrounded" numerics: the forward runs on the list-driven matrix-core kernel (P in
    high and low parts), the backward on the vector-ALU kernels; both against the oracle without round trips."""
    name, score, oscore = SCORES[4]
    assert name == "alibi_cfg"
    test_fused_unrounded_numerics(dev, dtype, D, name, score, oscore)
    q, k, v = (t.to(dev) for t in seeded_qkv(2, 4, 2, 256, 320, D, dtype))
    assert fa.kernel_family(q, k, v, kernel_options={"numerics": "unrounded"}) == "mfma_16bit"
    assert fa.kernel_family(q, k, v, kernel_options={"numerics": "unrounded"}, backward=True) == "generic"


def test_parity_numerics_dense_no_lists(dev):
    """Parity numerics without a mask (no tile lists, every tile visited) and with a ragged key length."""
    for dtype in (torch.bfloat16, torch.float16):
        run(dev, dtype, 1, 2, 2, 512, 512, 64, score=generate_checkerboard(2.0, 0.5, "kv"), oscore=o_checkerboard_kv,
            strict=False, opts={"numerics": "parity"})
        run(dev, dtype, 1, 2, 1, 200, 333, 128, score=generate_tanh_softcap(5.0), oscore=o_tanh_softcap(5.0),
            strict=False, opts={"numerics": "parity"})


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
def test_fused_forward_exponent_reference_guard(dev, dtype):
    """The one-pass forward keeps the reference value of a row's exponents where the first visible block put it and
    only moves it when a block's exponentials leave the safe range.  Both directions, on a dense problem (the
    pipelined D = 64 kernel) and under a causal mask (the list-driven kernel): (a) scores that climb by far more than
    2^15 along the keys -- every block has to move the reference up; (b) rows whose every score lies hundreds of
    binades below zero -- the first block has to move it down, or the whole row would underflow to an empty sum."""
    opts = {"numerics": "fast"}
    fast_bf16 = dtype == torch.bfloat16
    B, H, L, D = 1, 2, 512, 64
    q, k, v = seeded_qkv(B, H, H, L, L, D, dtype)
    for mask, omask in ((None, None), (causal_mask, o_causal_mask)):
        bm = None if mask is None else fa.create_block_mask(mask, B, H, L, L, device=dev)
        # (a) a relative-position bias of +0.75 per key: +24 in the exponent (+35 binades) from one 32-key block to the next
        out, lse = fa.flax_attention(q.to(dev), k.to(dev), v.to(dev), score_mod=generate_rel_bias(0.75), block_mask=bm,
                                     return_lse=True, kernel_options=opts)
        want, want_lse = ref_attention(q, k, v, o_rel_bias(0.75), omask, return_lse=True)
        close(out, want, dtype, f"O, climbing scores, mask {mask is not None}", fast_bf16)
        assert max_abs(lse.cpu(), want_lse) <= 2e-2 * max(1.0, want_lse.abs().max().item() / 64)
        # (b) keys opposed to the queries: every scaled score of a row near -|q|^2 * 6 / 8, i.e. about -50 +- noise ...
        u = torch.randn(B, H, 1, D, generator=torch.Generator().manual_seed(9))
        q2 = (6.0 * u + 0.3 * q.float()).to(dtype)
        k2 = (-6.0 * u + 0.3 * k.float()).to(dtype)
        # ... times a score_mod factor of 8: about -400 in every entry (-580 binades), a spread of tens inside a row
        big = generate_checkerboard(8.0, 8.0, "kv")
        obig = lambda s, b, h, qi, ki: s * 8.0   # noqa: E731
        out, lse = fa.flax_attention(q2.to(dev), k2.to(dev), v.to(dev), score_mod=big, block_mask=bm, return_lse=True,
                                     kernel_options=opts)
        want, want_lse = ref_attention(q2, k2, v, obig, omask, return_lse=True)
        assert float(want_lse.max()) < -100.0   # the case is what it claims to be
        close(out, want, dtype, f"O, scores far below zero, mask {mask is not None}", fast_bf16)
        assert torch.isfinite(lse).all() and max_abs(lse.cpu(), want_lse) <= 2e-2 * max(1.0, want_lse.abs().max().item() / 64)


ARBITRARY = [
    ("square", lambda s, b, h, q, kv: 0.1 * s * s + s),
    ("sin", lambda s, b, h, q, kv: 3.0 * torch.sin(s) + 0.01 * (kv - q)),
    ("leaky_by_head", lambda s, b, h, q, kv: torch.where(s > 0, s, 0.25 * (h + 1) * s)),
    ("batch_dependent", lambda s, b, h, q, kv: s * torch.sigmoid(s) * (1.0 + 0.5 * b)),
]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32], ids=["f16", "bf16", "f32"])
@pytest.mark.parametrize("name,fn", ARBITRARY, ids=[a[0] for a in ARBITRARY])
def test_arbitrary_score_mod_is_linearised(dev, dtype, name, fn):
    """A score_mod that is neither one of the functor families nor affine in the score (the reference applies any
    scalar callable, attention.py:59-63): evaluated, with its derivative, at the scores of the call and handed to the
    kernels as dense tables.  Forward, lse and all three gradients against the oracle, which applies the same callable
    densely and differentiates it with autograd; batch of 3 in chunks, GQA, ragged lengths, causal mask."""
    import flaxattention_amd.core.attention as att
    print(f"case arbitrary score_mod {name} {dtype}", flush=True)
    old = att._LINEARISE_BYTES
    att._LINEARISE_BYTES = 5 * 4 * 200 * 333 * 4 * 2   # two batch elements per chunk: the batch of 3 takes two chunks
    try:
        run(dev, dtype, 3, 4, 2, 200, 333, 64, score=fn, oscore=fn, mask=causal_mask, omask=o_causal_mask,
            strict=False, scale_maxabs=True)
        run(dev, dtype, 3, 2, 2, 130, 130, 128 if dtype != torch.float32 else 32, score=fn, oscore=fn, strict=False,
            pallas=True, scale_maxabs=True)
    finally:
        att._LINEARISE_BYTES = old


def test_linearised_score_mod_in_head_group_slabs(dev):
    """When the dense temporaries of ONE batch element exceed the budget, the linearised path walks groups of query
    heads that share a KV head; the callable and a head-dependent mask must still see absolute batch and head indices."""
    import flaxattention_amd.core.attention as att
    print("case linearised score_mod, head-group slabs", flush=True)
    fn = lambda s, b, h, q, kv: torch.where(s > 0, s, 0.25 * (h + 1) * s) * (1.0 + 0.5 * b)   # noqa: E731
    by_head = lambda b, h, q, kv: (q >= kv) | ((h % 2 == 1) & (kv < 8))                            # noqa: E731
    old = att._LINEARISE_BYTES
    att._LINEARISE_BYTES = 5 * 2 * 200 * 333 * 4   # two heads = one group of the 4 query / 2 KV heads
    try:
        assert att._linearise_chunks(2, 4, 2, 200, 333) == [(0, 1, 0, 2), (0, 1, 2, 4), (1, 2, 0, 2), (1, 2, 2, 4)]
        run(dev, torch.float16, 2, 4, 2, 200, 333, 64, score=fn, oscore=fn, mask=by_head, omask=by_head, strict=False,
            scale_maxabs=True)
    finally:
        att._LINEARISE_BYTES = old


PIECEWISE = [
    ("cap_past_sinks", lambda s, b, h, q, kv: torch.where(kv > 100, torch.tanh(s), s)),
    ("square_for_late_batches", lambda s, b, h, q, kv: torch.where(b >= 2, 0.2 * s * s, s)),
    ("sine_for_late_rows", lambda s, b, h, q, kv: torch.where(q >= 64, 3 * torch.sin(s), 2 * s)),
]


@pytest.mark.parametrize("name,fn", PIECEWISE, ids=[a[0] for a in PIECEWISE])
def test_score_mod_affine_only_near_the_origin(dev, name, fn):
    """Affine in the score for the first keys / rows / batch entries and something else beyond them: the dense-table
    lowering must refuse it (it once trusted a corner of the index range) and the call must come out as the reference
    computes it, which applies the callable to every element (attention.py:59-63)."""
    from flaxattention_amd.core.common import ScoreModNotLowered, resolve_score_mod
    print(f"case piecewise score_mod {name}", flush=True)
    with pytest.raises(ScoreModNotLowered):
        resolve_score_mod(fn, 2, (3, 2, 200, 333), dev)
    run(dev, torch.float16, 3, 2, 2, 200, 333, 64, score=fn, oscore=fn, mask=causal_mask, omask=o_causal_mask,
        strict=False, scale_maxabs=True)


def test_repeated_calls_reuse_the_plan_and_stay_correct(dev):
    """A training loop calls the front end with the same functors, block mask, shapes and options: the plan (lowered
    functors, tile lists, parameter block) is made once and found again.  A different block mask, other shapes, other
    options or another layout of the same shapes must not be served the remembered one."""
    import flaxattention_amd.core.attention as att
    made = []
    orig = att._make_plan

    def counting(*a, **k):
        made.append(1)
        return orig(*a, **k)
    att._make_plan = counting
    try:
        q, k, v = (t.to(dev) for t in seeded_qkv(2, 4, 4, 256, 256, 64, torch.float16))
        score = generate_alibi_bias(4, -1.0)
        bm = fa.create_block_mask(causal_mask, 1, 1, 256, 256, device=dev)
        want = ref_attention(q.cpu(), k.cpu(), v.cpu(), o_alibi_config(4), o_causal_mask)
        a = fa.flax_attention(q, k, v, score_mod=score, block_mask=bm)
        n = len(made)
        b = fa.flax_attention(q, k, v, score_mod=score, block_mask=bm)
        assert len(made) == n and torch.equal(a, b)
        close(a, want, torch.float16, "O, remembered plan")
        # [B,L,H,D] storage of the same logical shapes: same plan, another parameter block (strides)
        qt, kt, vt = (t.transpose(1, 2).contiguous().transpose(1, 2) for t in (q, k, v))
        c = fa.flax_attention(qt, kt, vt, score_mod=score, block_mask=bm)
        assert len(made) == n and torch.equal(a, c)
        # another mask object, other options, other shapes: planned anew, and right
        window = fa.create_block_mask(generate_sliding_window(40), 1, 1, 256, 256, device=dev)
        d = fa.flax_attention(q, k, v, score_mod=score, block_mask=window)
        assert len(made) == n + 1
        close(d, ref_attention(q.cpu(), k.cpu(), v.cpu(), o_alibi_config(4), o_sliding_window(40)), torch.float16, "O, other mask")
        e = fa.flax_attention(q, k, v, score_mod=score, block_mask=bm, kernel_options={"numerics": "parity"})
        assert len(made) == n + 2
        close(e, want, torch.float16, "O, other options")
        f = fa.flax_attention(q[:, :, :128], k, v, score_mod=score, block_mask=bm)
        assert len(made) == n + 3
        close(f, want[:, :, :128], torch.float16, "O, fewer rows")
        # gradients through a remembered plan, twice in a row
        for _ in range(2):
            qq, kk, vv = (t.clone().requires_grad_(True) for t in (q, k, v))
            fa.flax_attention(qq, kk, vv, score_mod=score, block_mask=bm).sum().backward()
            wq, wk, wv = ref_attention_bwd(q.cpu(), k.cpu(), v.cpu(), torch.ones_like(want), o_alibi_config(4), o_causal_mask)
            close(qq.grad, wq, torch.float16, "dQ, remembered plan", scale_maxabs=True)
            close(kk.grad, wk, torch.float16, "dK, remembered plan", scale_maxabs=True)
            close(vv.grad, wv, torch.float16, "dV, remembered plan", scale_maxabs=True)
        assert len(made) == n + 3
    finally:
        att._make_plan = orig


def test_lse_is_differentiable(dev):
    """The log-sum-exp output carries a gradient, as in the reference's dense path (attention.py:97-106): a loss of
    sum(O * dO) + sum(lse * w) against torch autograd through a dense fp64 evaluation."""
    for dtype, opts in ((torch.float16, {}), (torch.bfloat16, {}), (torch.float32, {})):
        B, H, L, D = 2, 2, 192, 64
        q, k, v = seeded_qkv(B, H, H, L, L, D, dtype)
        g = torch.Generator().manual_seed(5)
        d_o = torch.randn((B, H, L, D), generator=g).to(dtype)
        w = torch.randn((B, H, L), generator=g)
        qd, kd, vd = (t.to(dev).requires_grad_(True) for t in (q, k, v))
        bm = fa.create_block_mask(causal_mask, B, H, L, L, device=dev)
        out, lse = fa.flax_attention(qd, kd, vd, block_mask=bm, return_lse=True, kernel_options=opts)
        ((out.float() * d_o.to(dev).float()).sum() + (lse * w.to(dev)).sum()).backward()
        q64, k64, v64 = (t.double().requires_grad_(True) for t in (q, k, v))
        s = (q64 @ k64.transpose(-1, -2)) / math.sqrt(D)
        s = s.masked_fill(~torch.tril(torch.ones(L, L, dtype=torch.bool)), float("-inf"))
        o64 = torch.softmax(s, -1) @ v64
        ((o64 * d_o.double()).sum() + (torch.logsumexp(s, -1) * w.double()).sum()).backward()
        tol = 1e-4 if dtype == torch.float32 else 4e-3   # against the fp64 truth, not the rounding oracle
        for name, a, b in (("dQ", qd.grad, q64.grad), ("dK", kd.grad, k64.grad), ("dV", vd.grad, v64.grad)):
            r = rel_l2(a.detach().cpu(), b)
            print(f"  lse-gradient {dtype} {name}: rel-L2 {r:.2e}", flush=True)
            assert r <= tol, (dtype, name, r)
        # and the lse term alone is not silently dropped: its share of dQ is of the same order as the output's
        qd.grad = None
        out, lse = fa.flax_attention(qd, kd, vd, block_mask=bm, return_lse=True, kernel_options=opts)
        (lse * w.to(dev)).sum().backward()
        assert qd.grad.float().abs().max().item() > 1e-3


def test_block_mask_built_for_other_batch_and_heads(dev):
    """A BlockMask built for B=2, H=2 used with a batch of 4 and 4 heads: the reference only reads its mask_mod, so it
    works for any extents; the tile lists are rebuilt instead of being read past their end."""
    B, H, L, D = 4, 4, 384, 64
    def per_head(b, h, q_idx, kv_idx):
        return (q_idx >= kv_idx) & ((q_idx - kv_idx) <= 64 * (h + 1))
    q, k, v = (t.to(dev) for t in seeded_qkv(B, H, H, L, L, D, torch.float16))
    small = fa.create_block_mask(per_head, 2, 2, L, L, device=dev)
    whole = fa.create_block_mask(per_head, B, H, L, L, device=dev)
    a = fa.flax_attention(q, k, v, block_mask=small)
    b = fa.flax_attention(q, k, v, block_mask=whole)
    assert torch.equal(a, b)
    want = ref_attention(q.cpu(), k.cpu(), v.cpu(), None, per_head)
    close(a, want, torch.float16, "O")


@pytest.mark.parametrize("name,mask,omask", MASKS, ids=[m[0] for m in MASKS])
def test_fused_masks(dev, name, mask, omask):
    print(f"case fused mask {name}", flush=True)
    run(dev, torch.float16, 1, 2, 2, 384, 448, 64, mask=mask, omask=omask, strict=False)


def test_fused_no_mask_checkerboard_config2_small(dev):
    # benchmark configuration 2 at reduced batch: fp16, checkerboard, no mask
    run(dev, torch.float16, 1, 2, 2, 2048, 2048, 64, score=checkerboard, oscore=o_checkerboard, strict=False)


def test_fused_ragged_gqa(dev):
    run(dev, torch.float16, 2, 8, 2, 77, 203, 64, mask=causal_mask, omask=o_causal_mask,
        score=generate_alibi_bias(8, -1.0), oscore=o_alibi_config(8), strict=False)
    run(dev, torch.bfloat16, 1, 4, 1, 300, 131, 128, strict=False)


def test_fused_bitmap_mask_dead_rows(dev):
    def weird(b, h, q_idx, kv_idx):
        return ((q_idx * 7 + kv_idx * 3 + h) % 11 < 6) & (q_idx % 5 != 0)
    run(dev, torch.float16, 2, 3, 3, 200, 260, 64, mask=weird, omask=weird, strict=False)

    def doc_mask(b, h, q_idx, kv_idx):
        return (q_idx // 192) == (kv_idx // 192)
    run(dev, torch.float16, 1, 2, 2, 768, 768, 64, mask=doc_mask, omask=doc_mask, strict=False)


def test_fused_other_head_sizes_by_zero_padding(dev):
    """D = 32, 96 and Dv < D reach the fused kernels through zero-padded feature columns."""
    run(dev, torch.float16, 2, 4, 2, 130, 200, 32, mask=causal_mask, omask=o_causal_mask, strict=False, scale_maxabs=True)
    run(dev, torch.bfloat16, 1, 4, 4, 100, 100, 96, score=generate_alibi_bias(4), oscore=o_alibi(4), strict=False, scale_maxabs=True)
    run(dev, torch.float16, 1, 2, 2, 64, 300, 64, Dv=32, strict=False, scale_maxabs=True)
    run(dev, torch.float16, 1, 2, 2, 64, 300, 80, Dv=48, strict=False, pallas=True, scale_maxabs=True)
    # the generic kernels still take the sizes as they are
    run(dev, torch.float16, 1, 2, 2, 40, 70, 32, strict=False, opts={"pad_head_dim": False}, scale_maxabs=True)


def test_fused_fully_masked(dev):
    def fullmask(b, h, q_idx, kv_idx):
        return False
    out = run(dev, torch.float16, 1, 2, 2, 128, 128, 64, mask=fullmask, omask=o_full_masked, strict=False)
    assert torch.count_nonzero(out).item() == 0


def test_fused_round_s_off_matches_excess_precision_oracle(dev):
    q, k, v = seeded_qkv(1, 2, 2, 512, 512, 64, torch.float16)
    want = ref_attention(q, k, v, o_checkerboard, None, strict=False)
    out = fa.flax_attention(q.to(dev), k.to(dev), v.to(dev), score_mod=checkerboard, kernel_options={"round_s": False})
    close(out, want, torch.float16, "O (no S rounding vs non-strict oracle)")


def test_fused_decode_shapes_through_prefill_kernel(dev):
    for ql in (1, 16, 64):
        run(dev, torch.float16, 2, 4, 4, ql, 1024, 64, score=generate_alibi_bias(4, -1.0), oscore=o_alibi_config(4),
            mask=offset_causal_mask(1024 - ql), omask=o_offset_causal(1024 - ql), strict=False, grad=False)


# ---- seeded sweep over shapes x functors for the fused kernels (forward, dQ, dK, dV, lse) ----
def _sweep_case(seed):
    import random
    rnd = random.Random(1000 + seed)
    dtype = rnd.choice([torch.float16, torch.float16, torch.bfloat16])
    D = rnd.choice([64, 64, 128])
    Hkv = rnd.choice([1, 2, 3])
    G = rnd.choice([1, 1, 2, 4])
    B = rnd.choice([1, 2])
    Lq = rnd.choice([1, 17, 64, 129, 256, 300, 511, 640])
    Lkv = rnd.choice([33, 64, 200, 257, 512, 600, 777])
    name, score, oscore = rnd.choice([s for s in SCORES if s[0] != "alibi_ref"])
    if name.startswith("alibi"):   # the slope table depends on the head count
        score, oscore = (generate_alibi_bias(Hkv * G, sign=-1.0), o_alibi_config(Hkv * G))
    w = rnd.choice([16, 40, 130])
    masks = [(None, None), (causal_mask, o_causal_mask), (generate_sliding_window(w), o_sliding_window(w)),
             (generate_attention_sink(w, 4), o_attention_sink(w, 4)),
             (offset_causal_mask(max(Lkv - Lq, 0)), o_offset_causal(max(Lkv - Lq, 0)))]
    mask, omask = rnd.choice(masks)
    return dict(dtype=dtype, B=B, Hq=Hkv * G, Hkv=Hkv, Lq=Lq, Lkv=Lkv, D=D, score=score, oscore=oscore, mask=mask,
                omask=omask, use_block_mask=rnd.random() < 0.7, pallas=False, name=name)


@pytest.mark.parametrize("seed", range(24))
def test_fused_seeded_sweep(dev, seed):
    c = _sweep_case(seed)
    print(f"sweep {seed}: {c['dtype']} B{c['B']} Hq{c['Hq']} Hkv{c['Hkv']} Lq{c['Lq']} Lkv{c['Lkv']} D{c['D']} "
          f"score {c['name']} mask {getattr(c['mask'], '__name__', c['mask'])} block_mask {c['use_block_mask']}", flush=True)
    if c["mask"] is not None and not c["use_block_mask"]:
        # a bare mask_mod goes through flax_attention_pallas (flax_attention takes block masks only)
        run(dev, c["dtype"], c["B"], c["Hq"], c["Hkv"], c["Lq"], c["Lkv"], c["D"], score=c["score"], oscore=c["oscore"],
            mask=c["mask"], omask=c["omask"], strict=False, pallas=True, scale_maxabs=True)
    else:
        run(dev, c["dtype"], c["B"], c["Hq"], c["Hkv"], c["Lq"], c["Lkv"], c["D"], score=c["score"], oscore=c["oscore"],
            mask=c["mask"], omask=c["omask"], strict=False, scale_maxabs=True)


@pytest.mark.parametrize("seed", range(100, 116))
def test_simple_kernels_seeded_sweep(dev, seed):
    """The same sweep over the shapes of the simple matrix-core kernels: float32 (D 32 .. 128) and 16-bit head sizes
    above 128 (160 is zero-padded to 192)."""
    import random
    c = _sweep_case(seed)
    rnd = random.Random(seed)
    if rnd.random() < 0.5:
        c["dtype"], c["D"] = torch.float32, rnd.choice([32, 64, 96, 128])
    else:
        c["D"] = rnd.choice([160, 192, 256])
    print(f"sweep {seed}: {c['dtype']} B{c['B']} Hq{c['Hq']} Hkv{c['Hkv']} Lq{c['Lq']} Lkv{c['Lkv']} D{c['D']} "
          f"score {c['name']} mask {getattr(c['mask'], '__name__', c['mask'])} block_mask {c['use_block_mask']}", flush=True)
    pallas = c["mask"] is not None and not c["use_block_mask"]
    run(dev, c["dtype"], c["B"], c["Hq"], c["Hkv"], c["Lq"], c["Lkv"], c["D"], score=c["score"], oscore=c["oscore"],
        mask=c["mask"], omask=c["omask"], strict=False, pallas=pallas, scale_maxabs=True)


@pytest.mark.parametrize("dtype,D", [(torch.float32, 64), (torch.float32, 128), (torch.bfloat16, 192), (torch.float16, 256),
                                     (torch.float16, 64), (torch.bfloat16, 128)],
                         ids=["f32_64", "f32_128", "bf16_192", "f16_256", "f16_64", "bf16_128"])
def test_tiny_and_odd_shapes_on_every_family(dev, dtype, D):
    """Sequence lengths far below a tile, one key, one row, odd head counts: every matrix-core kernel family."""
    for B, Hq, Hkv, Lq, Lkv, mask, omask in ((1, 1, 1, 1, 1, None, None), (3, 5, 5, 5, 7, causal_mask, o_causal_mask),
                                             (1, 6, 3, 33, 31, None, None), (2, 7, 1, 2, 129, causal_mask, o_causal_mask)):
        print(f"case tiny {dtype} D{D} B{B} Hq{Hq} Hkv{Hkv} Lq{Lq} Lkv{Lkv}", flush=True)
        run(dev, dtype, B, Hq, Hkv, Lq, Lkv, D, mask=mask, omask=omask, strict=False, scale_maxabs=True)


# ---- score_mods that add a captured bias: a dense additive table read by the fused kernels ----
def test_fused_additive_bias_table(dev):
    g = torch.Generator().manual_seed(11)
    rel = torch.randn(6, 63, generator=g)            # per-head relative-position bias (T5 style)
    full = torch.randn(2, 1, 150, 333, generator=g)  # a bias given per (batch, query, key), shared by the heads
    rel_dev, full_dev = rel.to(dev), full.to(dev)

    def rel_bias(score, b, h, q_idx, kv_idx):
        t = rel_dev if score.is_cuda else rel
        return score + t[h.long(), (kv_idx - q_idx).clamp(-31, 31).long() + 31]

    def full_bias(score, b, h, q_idx, kv_idx):
        t = full_dev if score.is_cuda else full
        return score + t[b.long(), 0, q_idx.long(), kv_idx.long()]
    from flaxattention_amd.core.common import resolve_score_mod
    from flaxattention_amd import _lib
    spec = resolve_score_mod(rel_bias, 6, (2, 6, 200, 200), dev)
    assert spec.kind == _lib.SCORE_AFFINE and spec.mul is None
    assert spec.add.shape == (1, 6, 399) and spec.diag_zero == 199      # depends on kv - q only: kept per diagonal
    for dtype, D in ((torch.float16, 64), (torch.bfloat16, 128)):
        print(f"case additive table rel_bias {dtype} D{D}", flush=True)
        run(dev, dtype, 2, 6, 6, 200, 200, D, score=rel_bias, oscore=rel_bias, mask=causal_mask, omask=o_causal_mask,
            strict=False, scale_maxabs=True)
        run(dev, dtype, 2, 6, 2, 130, 257, D, score=rel_bias, oscore=rel_bias, strict=False, scale_maxabs=True)   # GQA, ragged
    # the table is a snapshot of the captured tensor: an in-place update (a learned bias after an optimizer step)
    # must be seen by the next call
    q, k, v = seeded_qkv(1, 6, 6, 64, 64, 64, torch.float16)
    before = fa.flax_attention(q.to(dev), k.to(dev), v.to(dev), score_mod=rel_bias)
    rel_dev.mul_(-3.0)
    rel.mul_(-3.0)
    after = fa.flax_attention(q.to(dev), k.to(dev), v.to(dev), score_mod=rel_bias)
    want = ref_attention(q, k, v, rel_bias, None, strict=True)
    assert rel_l2(after.cpu(), want) <= 1e-3 and rel_l2(before.cpu(), want) > 1e-1
    print("case additive table full_bias", flush=True)
    run(dev, torch.float16, 2, 4, 4, 150, 333, 64, score=full_bias, oscore=full_bias, mask=generate_sliding_window(40),
        omask=o_sliding_window(40), strict=False, scale_maxabs=True)
    run(dev, torch.float16, 2, 4, 4, 150, 333, 64, score=full_bias, oscore=full_bias, strict=False, pallas=True, scale_maxabs=True)


# ---- score_mods outside the functor families: lowered to dense affine tables, generic kernels ----
def test_affine_score_mod_tables(dev):
    table = torch.randn(4, 31, generator=torch.Generator().manual_seed(7))
    table_dev = table.to(dev)

    def rel_table(score, b, h, q_idx, kv_idx):   # learned relative-position bias (a captured buffer)
        t = table_dev if score.is_cuda else table
        return score + t[h.long(), (q_idx - kv_idx).clamp(-15, 15).long() + 15]

    def block_scale(score, b, h, q_idx, kv_idx):  # position-dependent scaling plus a per-batch shift
        return torch.where(q_idx // 32 == kv_idx // 32, score, score * 0.5) + 0.25 * b

    for fn in (rel_table, block_scale):
        for dtype in (torch.float32, torch.float16):
            print(f"case affine {fn.__name__} {dtype}", flush=True)
            run(dev, dtype, 2, 4, 2, 70, 150, 64, score=fn, oscore=fn, mask=causal_mask, omask=o_causal_mask,
                strict=(dtype == torch.float16), opts=None if dtype == torch.float16 else {}, scale_maxabs=True)

    # math_attention hands captured buffers to the mods as trailing arguments (attention.py:22-23)
    def bias_from(score, b, h, q_idx, kv_idx, tab):
        return score + tab[h.long(), (q_idx - kv_idx).clamp(-15, 15).long() + 15]

    def doc_mask(b, h, q_idx, kv_idx, doc):
        return doc[q_idx.long()] == doc[kv_idx.long()]
    doc = torch.arange(96) // 20
    q, k, v = seeded_qkv(1, 4, 4, 96, 96, 64, torch.float32)
    out, lse2 = fa.math_attention(q.to(dev), k.to(dev), v.to(dev), bias_from, (doc_mask,), 0.125, {},
                                  score_mod_other_buffers=(table_dev,), mask_mod_other_buffers=(doc.to(dev),))
    want, want_lse = ref_attention(q, k, v, lambda s, b, h, qi, ki: bias_from(s, b, h, qi, ki, table),
                                   lambda b, h, qi, ki: doc_mask(b, h, qi, ki, doc), scale=0.125, strict=True, return_lse=True)
    assert max_abs(out.cpu(), want) <= 1e-4 and max_abs(lse2.cpu() * 0.6931471805599453, want_lse) <= 1e-4

    def quadratic(score, b, h, q_idx, kv_idx):
        return score * score
    # not affine in the score: no score-independent functor exists, the front-end linearises it per call
    from flaxattention_amd.core.common import ScoreModNotLowered, resolve_score_mod
    with pytest.raises(ScoreModNotLowered):
        resolve_score_mod(quadratic, 2, (1, 2, 16, 16), dev)
    q, k, v = seeded_qkv(1, 2, 2, 16, 16, 64, torch.float16)
    out = fa.flax_attention(q.to(dev), k.to(dev), v.to(dev), score_mod=quadratic)
    assert rel_l2(out.cpu(), ref_attention(q, k, v, quadratic, None)) <= 1e-3


@pytest.mark.parametrize("shape", [(2, 2, 0, 64, 64), (2, 2, 16, 0, 64), (0, 2, 16, 64, 64), (1, 2, 300, 0, 128)])
def test_empty_inputs(dev, shape):
    """No query rows / batches give empty outputs; no keys make every row a fully masked row: output 0,
    log-sum-exp -inf, zero gradients (attention.py:97-104; tests/attention_test.py:65-129 for the masked form)."""
    B, H, Lq, Lkv, D = shape
    print(f"case empty inputs {shape}", flush=True)
    mk = lambda *s: torch.randn(*s, device=dev, dtype=torch.float16, requires_grad=True)
    q, k, v = mk(B, H, Lq, D), mk(B, H, Lkv, D), mk(B, H, Lkv, D)
    out, lse = fa.flax_attention(q, k, v, return_lse=True)
    assert out.shape == (B, H, Lq, D) and lse.shape == (B, H, Lq) and out.dtype == q.dtype
    if Lkv == 0:
        assert out.abs().sum().item() == 0 and bool(torch.isneginf(lse).all())
    out.sum().backward()
    for t in (q, k, v):
        assert t.grad.shape == t.shape and t.grad.abs().sum().item() == 0
    out_p = fa.flax_attention_pallas(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), mask_mod=causal_mask, bhln=False)
    assert out_p.shape == (B, Lq, H, D) and out_p.abs().sum().item() == 0
    with pytest.raises(ValueError):   # the validators still run first
        fa.flax_attention(q, k.float(), v)


def test_bitmap_mask_with_and_without_query_packed_copy(dev):
    """A bitmap mask carries a second copy packed along the query axis for the dK/dV kernel (one word per 32 x 32
    block instead of one per entry).  A caller of the C ABI may leave it out: the gradients are the same bits."""
    from flaxattention_amd.core.common import resolve_mask_mod
    print("case bitmap with / without query-packed copy", flush=True)
    B, H, Lq, Lkv, D = 2, 2, 200, 330, 64
    g = torch.Generator(device="cpu").manual_seed(5)
    keep = (torch.rand(B, 1, Lq, Lkv, generator=g) < 0.5)
    keep[..., 0] = True
    keep_dev = keep.to(dev)

    def mask(b, h, q_idx, kv_idx):
        t = keep_dev if q_idx.is_cuda else keep
        return t[b.long(), 0, q_idx.long(), kv_idx.long()]
    spec = resolve_mask_mod(mask, B, H, Lq, Lkv, dev)
    assert spec.bits is not None and spec.bits_t is not None
    assert spec.bits_t.shape[-2] == spec.bits.shape[-1] * 32 and spec.bits_t.shape[-1] * 32 == spec.bits.shape[-2]
    mk = lambda *s: torch.randn(*s, generator=g, dtype=torch.float32).to(torch.float16).to(dev)
    q, k, v, d_o = mk(B, H, Lq, D), mk(B, H, Lkv, D), mk(B, H, Lkv, D), mk(B, H, Lq, D)
    grads = []
    for with_copy in (True, False):
        m = spec if with_copy else type(spec)(name="no_copy", bits=spec.bits, fn=spec.fn)
        qd, kd, vd = (t.clone().requires_grad_(True) for t in (q, k, v))
        out = fa.flax_attention_pallas(qd, kd, vd, mask_mod=m)
        out.backward(d_o)
        grads.append((out.detach(), qd.grad, kd.grad, vd.grad))
    for a, b_ in zip(*grads):
        assert torch.equal(a, b_)
    # and against the oracle
    want = ref_attention(q.cpu(), k.cpu(), v.cpu(), None, mask, strict=True)
    assert rel_l2(grads[0][0].cpu(), want) <= 1e-3
    wq, wk, wv = ref_attention_bwd(q.cpu(), k.cpu(), v.cpu(), d_o.cpu(), None, mask, strict=True)
    for got, w in zip(grads[0][1:], (wq, wk, wv)):
        assert rel_l2(got.cpu(), w) <= 1e-3


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("kind", ["causal", "window", "bitmap", "none"])
def test_masks_without_tile_lists(dev, D, kind):
    """The C ABI allows a call without tile lists: every tile is visited and the mask evaluated in each.  Forward
    and backward must then give what they give with lists (and the oracle's result)."""
    print(f"case no tile lists D{D} {kind}", flush=True)
    B, H, Lq, Lkv = 2, 2, 200, 330
    g = torch.Generator(device="cpu").manual_seed(11)
    if kind == "causal":
        mask, omask = offset_causal_mask(Lkv - Lq), o_offset_causal(Lkv - Lq)
    elif kind == "window":
        mask, omask = generate_sliding_window(40), o_sliding_window(40)
    elif kind == "none":
        mask = omask = None
    else:
        keep = torch.rand(1, 1, Lq, Lkv, generator=g) < 0.5
        keep[..., 0] = True
        keep_dev = keep.to(dev)

        def mask(b, h, q_idx, kv_idx):
            t = keep_dev if q_idx.is_cuda else keep
            return t[0, 0, q_idx.long(), kv_idx.long()]
        omask = mask
    mk = lambda *s: torch.randn(*s, generator=g, dtype=torch.float32).to(torch.float16)
    q, k, v, d_o = mk(B, H, Lq, D), mk(B, H, Lkv, D), mk(B, H, Lkv, D), mk(B, H, Lq, D)
    res = []
    for lists in (True, False):
        qd, kd, vd = (t.to(dev).requires_grad_(True) for t in (q, k, v))
        out = fa.flax_attention_pallas(qd, kd, vd, mask_mod=mask, kernel_options={"tile_lists": lists})
        out.backward(d_o.to(dev))
        res.append((out.detach().cpu(), qd.grad.cpu(), kd.grad.cpu(), vd.grad.cpu()))
    want = ref_attention(q, k, v, None, omask, strict=True)
    wq, wk, wv = ref_attention_bwd(q, k, v, d_o, None, omask, strict=True)
    for name, a, b_, w in zip(("O", "dQ", "dK", "dV"), res[0], res[1], (want, wq, wk, wv)):
        print(f"  {name}: lists vs none {max_abs(a, b_):.3e}; none vs oracle rel-L2 {rel_l2(b_, w):.3e}", flush=True)
        assert rel_l2(b_, w) <= 1e-3 and max_abs(b_, w) <= 2e-2 * max(1.0, w.abs().max().item())
        assert max_abs(a, b_) <= 4e-3 * max(1.0, w.abs().max().item())


def test_views_that_start_inside_a_row(dev):
    """Inputs sliced along the feature axis (not 16-byte aligned, row stride not a multiple of 8 elements for one of
    them) are copied once by the front-end instead of being refused by the fused kernels."""
    print("case misaligned views", flush=True)
    g = torch.Generator(device="cpu").manual_seed(2)
    big = torch.randn(3, 2, 2, 150, 72, generator=g).to(torch.float16).to(dev)
    q, k, v = big[0, ..., 4:68], big[1, ..., 4:68], big[2, ..., 8:72]
    assert q.data_ptr() % 16 != 0 and q.stride(-1) == 1
    out = fa.flax_attention(q, k, v)
    want = fa.flax_attention(q.contiguous(), k.contiguous(), v.contiguous())
    assert torch.equal(out, want)
    odd = torch.randn(2, 2, 150, 68, generator=g).to(torch.float16).to(dev)[..., :64]   # row stride 68
    out = fa.flax_attention(odd, k, v)
    assert torch.equal(out, fa.flax_attention(odd.contiguous(), k.contiguous(), v.contiguous()))


@pytest.mark.parametrize("D", [64, 128])
def test_softcap_saturates_cleanly(dev, D):
    """Scores far beyond the cap (|s| / cap in the hundreds): tanh is exactly +-1 there, its derivative 0, and nothing
    turns into NaN in the fused kernels (their tanh goes through exp2 and a reciprocal without a clamp)."""
    print(f"case soft-cap saturation D{D}", flush=True)
    B, H, L = 1, 2, 192
    g = torch.Generator(device="cpu").manual_seed(4)
    mk = lambda *s: (6.0 * torch.randn(*s, generator=g, dtype=torch.float32)).to(torch.float16)
    q, k, v, d_o = mk(B, H, L, D), mk(B, H, L, D), mk(B, H, L, D) / 6, mk(B, H, L, D) / 6
    qd, kd, vd = (t.to(dev).requires_grad_(True) for t in (q, k, v))
    out = fa.flax_attention(qd, kd, vd, score_mod=generate_tanh_softcap(2.0))
    out.backward(d_o.to(dev))
    for t in (out, qd.grad, kd.grad, vd.grad):
        assert bool(torch.isfinite(t).all())
    want = ref_attention(q, k, v, o_tanh_softcap(2.0), None, strict=True)
    wq, wk, wv = ref_attention_bwd(q, k, v, d_o, o_tanh_softcap(2.0), None, strict=True)
    assert rel_l2(out.detach().cpu(), want) <= 1e-3
    for got, w in ((qd.grad, wq), (kd.grad, wk), (vd.grad, wv)):
        assert rel_l2(got.cpu(), w) <= 2e-3 and max_abs(got.cpu(), w) <= 2e-2 * max(1.0, w.abs().max().item())


def test_document_mask_equals_per_document_attention(dev):
    """A document mask written as a plain callable over a captured tensor of document ids: the result must be what
    ordinary attention gives on every document by itself (here torch's math-path SDPA in fp32 on the same device, an
    implementation that shares nothing with the kernels or the oracle)."""
    print("case document mask vs per-document attention", flush=True)
    B, H, L, D = 2, 4, 1000, 64
    lengths = [137, 400, 63, 400]
    doc = torch.repeat_interleave(torch.arange(len(lengths)), torch.tensor(lengths)).to(dev)

    def same_document(b, h, q_idx, kv_idx):
        d = doc if q_idx.is_cuda else doc.cpu()
        return d[q_idx.long()] == d[kv_idx.long()]
    g = torch.Generator(device="cpu").manual_seed(9)
    mk = lambda: torch.randn(B, H, L, D, generator=g, dtype=torch.float32).to(torch.float16).to(dev).requires_grad_(True)
    q, k, v = mk(), mk(), mk()
    d_o = torch.randn(B, H, L, D, generator=g, dtype=torch.float32).to(torch.float16).to(dev)
    bm = fa.create_block_mask(same_document, 1, 1, L, L, device=dev)
    out = fa.flax_attention(q, k, v, block_mask=bm)
    out.backward(d_o)
    qf, kf, vf = (t.detach().float().requires_grad_(True) for t in (q, k, v))
    pieces, at = [], 0
    from torch.nn.attention import SDPBackend, sdpa_kernel
    with sdpa_kernel(SDPBackend.MATH):
        for n in lengths:
            s = slice(at, at + n)
            pieces.append(torch.nn.functional.scaled_dot_product_attention(qf[:, :, s], kf[:, :, s], vf[:, :, s]))
            at += n
    want = torch.cat(pieces, dim=2)
    want.backward(d_o.float())
    assert rel_l2(out.detach().float().cpu(), want.detach().cpu()) <= 1e-3
    for got, ref in ((q.grad, qf.grad), (k.grad, kf.grad), (v.grad, vf.grad)):
        assert rel_l2(got.float().cpu(), ref.cpu()) <= 2e-3
