"""Pins the CPU oracle (oracle/flex_oracle.py) without the reference package:
golden vectors from PyTorch's own block-mask builder, hand-derived closed forms,
torch SDPA / flex_attention (the comparator the reference's tests use,
tests/attention_test.py:52-63), fp64 brute force, autograd and finite
differences.  Runs on the CPU."""
import json
import math
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import (max_abs, o_alibi, o_alibi_config, o_attention_sink, o_causal_mask, o_checkerboard,
                    o_checkerboard_kv, o_full_masked, o_offset_causal, o_rel_bias, o_sink_window_lt,
                    o_sliding_window, o_tanh_softcap, ref_attention, ref_attention_bwd, ref_create_block_mask,
                    ref_create_mask, rel_l2, seeded_qkv, truth_attention)

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "block_mask_vectors.json")))
GOLD_MASKS = {
    "causal_B1_H4_256": o_causal_mask, "causal_B1_H1_2048": o_causal_mask,
    "window1024_sink_lt4_8192": o_sink_window_lt(1024, 4), "sink_le4_window300_2048": o_attention_sink(300, 4),
    "sliding_window_10_1024": o_sliding_window(10), "causal_rect_384x640": o_causal_mask,
}
FIELDS = ["kv_num_blocks", "kv_indices", "full_kv_num_blocks", "full_kv_indices",
          "q_num_blocks", "q_indices", "full_q_num_blocks", "full_q_indices"]


@pytest.mark.parametrize("name", sorted(GOLD))
def test_block_mask_oracle_vs_torch_golden(name):
    g = GOLD[name]
    ref = ref_create_block_mask(GOLD_MASKS[name], g["B"], g["H"], g["Q"], g["KV"], g["BLOCK_SIZE"])
    for f in FIELDS:
        want = np.asarray(g[f], dtype=np.int32)
        for b in range(g["B"]):
            for h in range(g["H"]):
                assert np.array_equal(ref[f][b, h], want), (name, f)


def test_block_mask_hand_derived():
    # causal at 128: row i has one partial block [i] and i full blocks [0..i-1]
    r = ref_create_block_mask(o_causal_mask, 1, 4, 256, 256)
    assert r["kv_num_blocks"].tolist() == [[[1, 1]] * 4]
    assert r["kv_indices"][0, 0].tolist() == [[0, 1], [1, 0]]
    assert r["full_kv_num_blocks"][0, 0].tolist() == [0, 1]
    assert r["full_kv_indices"][0, 0].tolist() == [[0, 1], [0, 1]]
    assert r["q_num_blocks"][0, 0].tolist() == [1, 1] and r["q_indices"][0, 0].tolist() == [[0, 1], [1, 0]]
    # what the reference itself yields for the transposed lists (blockmask.py:46-47 drops the scatter)
    assert r["refq_num_blocks"][0, 0].tolist() == [0, 0] and r["refq_indices"][0, 0].tolist() == [[0, 1], [0, 1]]
    r = ref_create_block_mask(o_causal_mask, 1, 1, 2048, 2048)
    assert int(r["kv_num_blocks"].sum()) == 16 and int(r["full_kv_num_blocks"].sum()) == 120
    r = ref_create_block_mask(o_sink_window_lt(1024, 4), 1, 1, 8192, 8192)
    assert int(r["kv_num_blocks"].sum()) == 175 and int(r["full_kv_num_blocks"].sum()) == 420
    assert r["kv_indices"][0, 0, 9, :8].tolist() == [0, 1, 9, 2, 3, 4, 5, 6]
    assert r["full_kv_indices"][0, 0, 9, :7].tolist() == [2, 3, 4, 5, 6, 7, 8]
    # decode shapes: Q_LEN < 128 makes one query block of Q_LEN rows (blockmask.py:440-441)
    for ql, partial in ((1, 0), (16, 1), (64, 1)):
        r = ref_create_block_mask(o_offset_causal(16384 - ql), 1, 1, ql, 16384)
        assert r["used_block_size"] == (ql, 128)
        assert int(r["kv_num_blocks"].sum()) == partial and int(r["full_kv_num_blocks"].sum()) == 128 - partial
    # lengths are rounded up and the mask is evaluated on the padded range (blockmask.py:442-444)
    r = ref_create_block_mask(o_causal_mask, 1, 1, 300, 500)
    assert r["kv_indices"].shape == (1, 1, 3, 4)
    assert r["BLOCK_SIZE"] == (128, 128)


def test_score_mod_as_mask_source():
    def smod(score, b, h, q_idx, kv_idx):
        return torch.where(q_idx >= kv_idx, score, torch.full_like(score, -math.inf))
    assert np.array_equal(ref_create_mask(smod, 1, 2, 64, 64), ref_create_mask(o_causal_mask, 1, 2, 64, 64))


# ---- forward ----
def test_forward_vs_sdpa_and_flex():
    from torch.nn.attention.flex_attention import flex_attention
    q, k, v = seeded_qkv(4, 8, 8, 64, 64, 32, torch.float32)     # the reference's test shape
    assert max_abs(ref_attention(q, k, v), F.scaled_dot_product_attention(q, k, v)) < 2e-6
    assert max_abs(ref_attention(q, k, v, mask_mod=o_causal_mask),
                   F.scaled_dot_product_attention(q, k, v, is_causal=True)) < 2e-6
    i = torch.arange(64)
    for name, omod, bias in (
        ("alibi_ref", o_alibi(8), (i[:, None] - i[None, :]).float() * torch.exp2(-(torch.arange(8) + 1.0))[:, None, None]),
        ("alibi_cfg", o_alibi_config(8), (i[None, :] - i[:, None]).float() * torch.exp2(-(torch.arange(8) + 1.0))[:, None, None]),
        ("rel", o_rel_bias(0.05), (i[None, :] - i[:, None]).float() * 0.05),
    ):
        want = F.scaled_dot_product_attention(q, k, v, attn_mask=bias.expand(4, 8, 64, 64))
        assert max_abs(ref_attention(q, k, v, omod), want) < 5e-6, name
    win = (i[:, None] - i[None, :] <= 10) & (i[:, None] >= i[None, :])
    assert max_abs(ref_attention(q, k, v, mask_mod=o_sliding_window(10)),
                   F.scaled_dot_product_attention(q, k, v, attn_mask=win)) < 2e-6

    def t_checker(s, b, h, qi, ki):
        s = torch.where((ki - qi) % 2 == 0, s * 0.5, s)
        return torch.where((ki - qi) % 2 == 1, s * 2.0, s)
    assert max_abs(ref_attention(q, k, v, o_checkerboard), flex_attention(q, k, v, score_mod=t_checker)) < 5e-6
    assert max_abs(ref_attention(q, k, v, o_tanh_softcap(3.0)),
                   flex_attention(q, k, v, score_mod=lambda s, b, h, qi, ki: 3.0 * torch.tanh(s / 3.0))) < 5e-6
    # Lq = 1 decode with ALiBi (tests/attention_test.py:173-232)
    q1 = q[:, :, :1]
    assert max_abs(ref_attention(q1, k, v, o_alibi(8)),
                   flex_attention(q1, k, v, score_mod=lambda s, b, h, qi, ki: s + (qi - ki) * torch.exp2(-((h + 1) * 8.0 / 8)))) < 5e-6


def test_forward_bruteforce_fp64_tiny():
    q, k, v = seeded_qkv(1, 2, 2, 5, 7, 4, torch.float64)
    got = ref_attention(q, k, v, o_checkerboard_kv, o_offset_causal(2), scale=0.3)
    for h in range(2):
        for i in range(5):
            num, den = torch.zeros(4, dtype=torch.float64), 0.0
            for j in range(7):
                if i + 2 >= j:
                    s = float(q[0, h, i] @ k[0, h, j]) * 0.3
                    s = s * (0.5 if j % 2 == 1 else 2.0)
                    num += math.exp(s) * v[0, h, j]
                    den += math.exp(s)
            assert max_abs(got[0, h, i], num / den) < 1e-12


def test_lse_and_invariants():
    q, k, v = seeded_qkv(2, 4, 4, 48, 80, 16, torch.float32)
    O, lse = ref_attention(q, k, v, o_alibi(4), o_causal_mask, return_lse=True)
    S = q @ k.transpose(-1, -2) / 4.0
    i, j = torch.arange(48)[:, None], torch.arange(80)[None, :]
    X = S + (i - j).float() * torch.exp2(-(torch.arange(4) + 1.0) * 2.0)[:, None, None]
    X = X.masked_fill(i < j, -math.inf)
    assert max_abs(lse, torch.logsumexp(X, -1)) < 1e-5
    assert max_abs(O, torch.exp(X - lse[..., None]) @ v) < 1e-5          # O == sum_j exp(X - lse) V_j
    assert max_abs(ref_attention(q, k, torch.ones_like(v), o_alibi(4), o_causal_mask), torch.ones_like(O)) < 1e-6
    # fully masked rows: output 0, lse -inf (tests/attention_test.py:65-129)
    O, lse = ref_attention(q, k, v, None, o_full_masked, return_lse=True)
    assert torch.count_nonzero(O) == 0 and torch.isneginf(lse).all()
    # GQA == explicit repeat along the head axis (attention.py:80-82)
    qg, kg, vg = seeded_qkv(2, 8, 2, 16, 24, 8, torch.float32)
    assert max_abs(ref_attention(qg, kg, vg), ref_attention(qg, kg.repeat_interleave(4, 1), vg.repeat_interleave(4, 1))) == 0
    # decode rows equal the last rows of the prefill problem under the offset-causal mask
    full = ref_attention(q[:, :, :48], k[:, :, :48], v[:, :, :48], None, o_causal_mask)
    last = ref_attention(q[:, :, 40:48], k[:, :, :48], v[:, :, :48], None, o_offset_causal(40))
    assert max_abs(full[:, :, 40:], last) < 1e-6


def test_strict_rounding_points():
    q, k, v = seeded_qkv(1, 2, 2, 64, 64, 32, torch.float16)
    a, b = ref_attention(q, k, v, o_checkerboard, strict=True), ref_attention(q, k, v, o_checkerboard, strict=False)
    t = truth_attention(q, k, v, score_mod=o_checkerboard)
    assert 0 < rel_l2(a, b) < 3e-3 and rel_l2(a, t) < 3e-3 and rel_l2(b, t) < 1e-3
    q32, k32, v32 = q.float(), k.float(), v.float()
    assert max_abs(ref_attention(q32, k32, v32, strict=True), ref_attention(q32, k32, v32, strict=False)) == 0


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
def test_rounding_points_against_torch_half_program(dtype):
    """Where the strict oracle rounds through the input dtype is pinned here by a program that torch itself rounds:
    a literal transcription of flaxattention/core/attention.py:27 (Q.K^T computed in the input dtype, then cast to
    fp32), :55 (scale applied after the cast), :97-104 (softmax in fp32) and :105 (P cast to the input dtype, then
    P.V in that dtype) with torch's own 16-bit CPU matrix products, differentiated by torch autograd -- so the
    backward's rounding of dP = dO.V^T (a product in the input dtype) and of dS (the cotangent of the cast in :27,
    after the scale) is placed by autograd, not by the oracle's author.  D = 128: the scale is not a power of two, so
    rounding S before or after it are different numbers.  The oracle must agree with that program to accumulation
    order, and each misplaced rounding point must not."""
    from oracle.flex_oracle import MUTANTS
    q, k, v = seeded_qkv(1, 2, 2, 96, 160, 128, dtype)
    d_o = torch.randn(1, 2, 96, 128, generator=torch.Generator().manual_seed(5)).to(dtype)
    scale = 1.0 / math.sqrt(128.0)
    qq, kk, vv = (t.clone().requires_grad_(True) for t in (q, k, v))
    S = torch.matmul(qq, kk.transpose(-1, -2)).to(torch.float32) * scale
    vis = torch.arange(96).view(96, 1) >= torch.arange(160).view(1, 160)
    S = torch.where(vis, S, torch.full((), -math.inf))
    P = torch.exp(S - torch.logsumexp(S, dim=-1, keepdim=True))
    O = torch.matmul(P.to(dtype), vv)
    O.backward(d_o)
    literal = (O.detach(), qq.grad, kk.grad, vv.grad)

    def distance(mutant):
        o = ref_attention(q, k, v, None, o_causal_mask, scale, strict=True, _mutant=mutant)
        g = ref_attention_bwd(q, k, v, d_o, None, o_causal_mask, scale, strict=True, _mutant=mutant)
        return [rel_l2(a, b) for a, b in zip((o,) + g, literal)]

    own = distance(None)
    # measured 3e-5 (fp16) and 0 ... 1e-4 (bf16): accumulation order flips the last bit of a few entries
    bound = 6e-5 if dtype == torch.float16 else 2e-4
    assert max(own) <= bound, own
    touched = {"s_after_scale": (0, 1, 2, 3), "p_unrounded": (0, 3), "dp_unrounded": (1, 2), "ds_unrounded": (1, 2)}
    for mutant in MUTANTS:
        d = distance(mutant)
        for i in touched[mutant]:
            assert d[i] >= 4 * bound and d[i] >= 4 * own[i], (mutant, i, d, own)
    # and the variant without round trips is not what that program computes either
    loose = [rel_l2(a, b) for a, b in zip(
        (ref_attention(q, k, v, None, o_causal_mask, scale, strict=False),)
        + ref_attention_bwd(q, k, v, d_o, None, o_causal_mask, scale, strict=False), literal)]
    assert min(loose) >= 4 * bound, loose


# ---- backward ----
def _autograd(q, k, v, d_o, bias=None, mult=None, keep=None, scale=None):
    qq, kk, vv = (t.double().clone().requires_grad_(True) for t in (q, k, v))
    G = q.shape[1] // k.shape[1]
    S = qq @ kk.repeat_interleave(G, 1).transpose(-1, -2) * (scale if scale is not None else q.shape[-1] ** -0.5)
    if mult is not None:
        S = S * mult
    if bias is not None:
        S = S + bias
    if keep is not None:
        S = S.masked_fill(~keep, -math.inf)
    O = torch.softmax(S, -1) @ vv.repeat_interleave(G, 1)
    (O * d_o.double()).sum().backward()
    return O, qq.grad, kk.grad, vv.grad


def test_backward_vs_autograd_fp64():
    q, k, v = seeded_qkv(2, 4, 2, 24, 40, 16, torch.float64)
    d_o = torch.randn(2, 4, 24, 16, dtype=torch.float64, generator=torch.Generator().manual_seed(5))
    i, j = torch.arange(24)[:, None], torch.arange(40)[None, :]
    cases = [
        (None, None, dict()),
        (o_alibi(4), o_offset_causal(16), dict(bias=(i - j).double() * torch.exp2(-(torch.arange(4) + 1.0) * 2.0)[:, None, None].double(), keep=(i + 16 >= j))),
        (o_checkerboard, o_sliding_window(7), dict(mult=torch.where((j - i) % 2 == 0, 0.5, 2.0).double(), keep=((i - j <= 7) & (i >= j)))),
    ]
    for sm, mm, kw in cases:
        if "keep" in kw and not kw["keep"].any(-1).all():
            continue
        O, gq, gk, gv = _autograd(q, k, v, d_o, **kw)
        assert max_abs(ref_attention(q, k, v, sm, mm), O) < 1e-12
        dq, dk, dv = ref_attention_bwd(q, k, v, d_o, sm, mm)
        assert max_abs(dq, gq) < 1e-11 and max_abs(dk, gk) < 1e-11 and max_abs(dv, gv) < 1e-11


def test_backward_softcap_finite_differences():
    q, k, v = seeded_qkv(1, 1, 1, 6, 9, 4, torch.float64)
    d_o = torch.randn(1, 1, 6, 4, dtype=torch.float64, generator=torch.Generator().manual_seed(7))
    sm, mm = o_tanh_softcap(0.8), o_offset_causal(3)
    dq, dk, dv = ref_attention_bwd(q, k, v, d_o, sm, mm)
    loss = lambda q_, k_, v_: float((ref_attention(q_, k_, v_, sm, mm) * d_o).sum())
    eps = 1e-6
    for t, gr in ((q, dq), (k, dk), (v, dv)):
        for idx in [(0, 0, 1, 2), (0, 0, 4, 0), (0, 0, 5, 3)]:
            tp, tm = t.clone(), t.clone()
            tp[idx] += eps
            tm[idx] -= eps
            args_p = [tp if x is t else x for x in (q, k, v)]
            args_m = [tm if x is t else x for x in (q, k, v)]
            fd = (loss(*args_p) - loss(*args_m)) / (2 * eps)
            assert abs(fd - float(gr[idx])) < 1e-7


def test_backward_closed_form_sum_loss_and_dead_rows():
    q, k, v = seeded_qkv(1, 2, 2, 16, 16, 8, torch.float64)
    _, P_lse = ref_attention(q, k, v, None, o_causal_mask, return_lse=True)
    S = q @ k.transpose(-1, -2) / math.sqrt(8)
    i = torch.arange(16)
    P = torch.exp(S.masked_fill(i[:, None] < i[None, :], -math.inf) - P_lse[..., None])
    dq, dk, dv = ref_attention_bwd(q, k, v, torch.ones_like(q), None, o_causal_mask)
    # loss = O.sum(): dV[j, :] = sum_i P_ij in every column
    assert max_abs(dv, P.sum(-2)[..., None].expand_as(dv)) < 1e-12
    # rows with no visible key get zero gradient and do not poison the rest
    def some_dead(b, h, q_idx, kv_idx):
        return (q_idx >= kv_idx) & (q_idx % 3 != 0)
    g = ref_attention_bwd(q, k, v, torch.ones_like(q), None, some_dead)
    assert all(torch.isfinite(t).all() for t in g) and torch.count_nonzero(g[0][:, :, 0::3]) == 0


def test_config_sized_slice_runs_in_seconds():
    # one head of benchmark configuration 2 / 3 stays cheap enough for the GPU parity tests
    q, k, v = seeded_qkv(1, 1, 1, 2048, 2048, 64, torch.bfloat16)
    O = ref_attention(q, k, v, o_alibi_config(8), o_causal_mask)
    assert O.shape == (1, 1, 2048, 64) and torch.isfinite(O.float()).all()
