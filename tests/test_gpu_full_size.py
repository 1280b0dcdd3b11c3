"""The benchmark configurations at their full sizes.  The CPU oracle would need gigabytes of dense
temporaries there, so the kernels are held to (a) the oracle on a sample of query rows -- a row of O, lse and dQ
depends on that row of Q and dO and on all of K and V only --, (b) the oracle's dQ, dK and dV on a few whole
(batch, head) pairs, each a dense problem the host can hold, and (c) identities that hold at any size:

    <Q, dQ> = <K, dK>      the loss depends on Q and K through Q K^T only (any score_mod, any mask)
    <V, dV> = <O, dO>      O is linear in V
    sum_j dK_j = 0         under an additive score_mod a common shift of all keys moves every score of a row alike
    V = 1  =>  O = 1, dQ = dK = 0, sum_j dV_j = Lq   rows of P sum to one
"""
import math

import pytest
import torch

import flaxattention_amd as fa
from flaxattention_amd.masks import causal_mask, generate_attention_sink, offset_causal_mask
from flaxattention_amd.mods import generate_alibi_bias, generate_checkerboard, generate_tanh_softcap
from oracle import (max_abs, o_alibi_config, o_causal_mask, o_checkerboard_kv, o_offset_causal, o_sink_window_lt,
                    o_tanh_softcap, ref_attention, ref_attention_bwd, rel_l2)

pytestmark = pytest.mark.gpu


def _inputs(dev, dtype, B, H, Lq, Lkv, D, seed=0):
    g = torch.Generator(device="cpu").manual_seed(seed)
    mk = lambda *s: torch.randn(*s, generator=g, dtype=torch.float32).to(dtype)
    k, q, v, d_o = mk(B, H, Lkv, D), mk(B, H, Lq, D), mk(B, H, Lkv, D), mk(B, H, Lq, D)
    return q, k, v, d_o


def _rows_mods(rows, oscore, omask):
    """Oracle mods for a problem that holds only the sampled query rows: position i there is row rows[i]."""
    rows_t = torch.as_tensor(rows)
    sc = None if oscore is None else (lambda s, b, h, qi, ki: oscore(s, b, h, rows_t[qi.long()].to(qi.dtype), ki))
    mk = None if omask is None else (lambda b, h, qi, ki: omask(b, h, rows_t[qi.long()].to(qi.dtype), ki))
    return sc, mk


def _check_sampled_rows(q, k, v, d_o, out, lse, dq, oscore, omask, dtype, bs, hs, rows):
    sc, mk = _rows_mods(rows, oscore, omask)

    def head_mods(h0):   # the oracle sees one head at a time: head index 0 there is head h0
        s2 = None if sc is None else (lambda s, b, h, qi, ki: sc(s, b, h + h0, qi, ki))
        m2 = None if mk is None else (lambda b, h, qi, ki: mk(b, h + h0, qi, ki))
        return s2, m2
    # the stated tolerance for 16-bit inputs, in the kernels' default numerics (fp16 "fast", bf16 "parity")
    tol = tol_grad = 1e-3
    for b in bs:
        for h in hs:
            s2, m2 = head_mods(h)
            qs, ks, vs, gs = q[b:b + 1, h:h + 1, rows], k[b:b + 1, h:h + 1], v[b:b + 1, h:h + 1], d_o[b:b + 1, h:h + 1, rows]
            want, want_lse = ref_attention(qs, ks, vs, s2, m2, strict=True, return_lse=True)
            got = out[b:b + 1, h:h + 1, rows].cpu()
            a, r = max_abs(got, want), rel_l2(got, want)
            print(f"  rows of (b{b},h{h}): O max-abs {a:.3e} rel-L2 {r:.3e}", flush=True)
            assert a <= 2e-2 and r <= tol
            assert max_abs(lse[b:b + 1, h:h + 1, rows].cpu(), want_lse) <= 2e-2
            if dq is not None:
                wq, _, _ = ref_attention_bwd(qs, ks, vs, gs, s2, m2, strict=True)
                gq = dq[b:b + 1, h:h + 1, rows].cpu()
                a, r = max_abs(gq, wq), rel_l2(gq, wq)
                print(f"                     dQ max-abs {a:.3e} rel-L2 {r:.3e}", flush=True)
                # one unit in the last place at the largest reference entry where that exceeds the absolute bound
                big = wq.abs().max().item()
                ulp = 2.0 ** (math.floor(math.log2(big)) - (7 if dtype == torch.bfloat16 else 10)) if big > 0 else 0.0
                assert a <= max(2e-2, ulp) and r <= tol_grad


def _check_whole_heads(q, k, v, d_o, dq, dk, dv, oscore, omask, dtype, pairs, tol=1e-3):
    """dK and dV of key j depend on that key and on ALL of Q and dO (through every row's log-sum-exp and delta), so they
    are checked on whole (batch, head) pairs: the oracle's backward of one pair is one dense [Lq, Lkv] problem."""
    for b, h in pairs:
        s2 = None if oscore is None else (lambda s, bb, hh, qi, ki, h0=h: oscore(s, bb, hh + h0, qi, ki))
        m2 = None if omask is None else (lambda bb, hh, qi, ki, h0=h: omask(bb, hh + h0, qi, ki))
        sl = (slice(b, b + 1), slice(h, h + 1))
        want = ref_attention_bwd(q[sl], k[sl], v[sl], d_o[sl], s2, m2, strict=True)
        for name, got, w in zip(("dQ", "dK", "dV"), (dq, dk, dv), want):
            g = got[sl].cpu()
            a, r = max_abs(g, w), rel_l2(g, w)
            big = w.abs().max().item()
            ulp = 2.0 ** (math.floor(math.log2(big)) - (7 if dtype == torch.bfloat16 else 10)) if big > 0 else 0.0
            print(f"  whole head (b{b},h{h}): {name} max-abs {a:.3e} rel-L2 {r:.3e} (largest entry {big:.1f})", flush=True)
            assert a <= max(2e-2, ulp) and r <= tol, (name, b, h, a, r)


def _inner(a, b):
    return (a.double() * b.double()).sum(dim=(-1, -2))   # per (batch, head)


def _check_identities(q, k, v, d_o, out, dq, dk, dv, additive):
    """Differences are measured against the sum of the absolute products, which is what rounding noise scales with."""
    qk, kk = _inner(q, dq), _inner(k, dk)
    vv, oo = _inner(v, dv), _inner(out, d_o)
    s1 = ((qk - kk).abs() / _inner(q.abs(), dq.abs())).max().item()
    s2 = ((vv - oo).abs() / _inner(v.abs(), dv.abs())).max().item()
    print(f"  <Q,dQ> vs <K,dK>: {s1:.2e}   <V,dV> vs <O,dO>: {s2:.2e}", flush=True)
    assert s1 <= 2e-3 and s2 <= 2e-3
    if additive:
        shift = dk.double().sum(dim=-2).abs().max().item() / dk.double().abs().sum(dim=-2).max().item()
        print(f"  |sum_j dK_j| / sum_j |dK_j|: {shift:.2e}", flush=True)
        assert shift <= 2e-3


def _fwd_bwd(dev, q, k, v, d_o, score, bm):
    qd, kd, vd = (t.to(dev).requires_grad_(True) for t in (q, k, v))
    out, lse = fa.flax_attention(qd, kd, vd, score_mod=score, block_mask=bm, return_lse=True)
    out.backward(d_o.to(dev))
    return out.detach(), lse.detach(), qd.grad, kd.grad, vd.grad


ROWS = [0, 1, 31, 32, 127, 128, 1000, 1023, 1024, 2047]


def test_config2_full_size(dev):
    """fp16 [8,8,2048,64], checkerboard by kv parity, no mask, forward + backward."""
    print("case config 2 full size", flush=True)
    q, k, v, d_o = _inputs(dev, torch.float16, 8, 8, 2048, 2048, 64)
    out, lse, dq, dk, dv = _fwd_bwd(dev, q, k, v, d_o, generate_checkerboard(2.0, 0.5, "kv"), None)
    _check_sampled_rows(q, k, v, d_o, out, lse, dq, o_checkerboard_kv, None, torch.float16, (0, 7), (0, 5), ROWS)
    _check_whole_heads(q, k, v, d_o, dq, dk, dv, o_checkerboard_kv, None, torch.float16, ((0, 0), (7, 5)))
    _check_identities(q, k, v, d_o, out.cpu(), dq.cpu(), dk.cpu(), dv.cpu(), additive=False)
    # V = 1: every row of P sums to one
    ones = torch.ones_like(v)
    o1, _, dq1, dk1, dv1 = _fwd_bwd(dev, q, k, ones, torch.ones_like(d_o), generate_checkerboard(2.0, 0.5, "kv"), None)
    assert max_abs(o1.cpu(), torch.ones_like(q)) <= 2e-3
    assert dq1.abs().max().item() <= 2e-3 and dk1.abs().max().item() <= 2e-3
    assert (dv1.double().sum(dim=-2).cpu() - 2048).abs().max().item() <= 2048 * 2e-3


def test_config3_full_size(dev):
    """bf16 [8,8,2048,64], ALiBi 2^(-8(h+1)/H) * (kv - q), causal block mask, forward + backward."""
    print("case config 3 full size", flush=True)
    q, k, v, d_o = _inputs(dev, torch.bfloat16, 8, 8, 2048, 2048, 64)
    bm = fa.create_block_mask(causal_mask, 1, 1, 2048, 2048, device=dev)
    out, lse, dq, dk, dv = _fwd_bwd(dev, q, k, v, d_o, generate_alibi_bias(8, -1.0), bm)
    _check_sampled_rows(q, k, v, d_o, out, lse, dq, o_alibi_config(8), o_causal_mask, torch.bfloat16, (0, 7), (0, 7), ROWS)
    _check_whole_heads(q, k, v, d_o, dq, dk, dv, o_alibi_config(8), o_causal_mask, torch.bfloat16, ((0, 0), (7, 7)))
    _check_identities(q, k, v, d_o, out.cpu(), dq.cpu(), dk.cpu(), dv.cpu(), additive=True)


def test_config4_full_size(dev):
    """bf16 [4,16,8192,128], causal window 1024 + 4 sink keys, tanh soft-cap 50: forward and dQ on sampled rows, all
    three gradients on one whole head, the rest through the identities."""
    print("case config 4 full size", flush=True)
    q, k, v, d_o = _inputs(dev, torch.bfloat16, 4, 16, 8192, 8192, 128)
    bm = fa.create_block_mask(generate_attention_sink(1024, 3), 1, 1, 8192, 8192, device=dev)
    # 175 partial + 420 full tiles of 128 x 128 per head (closed form of this mask at this size)
    assert int(bm.kv_num_blocks.sum().item()) == 175 and int(bm.full_kv_num_blocks.sum().item()) == 420
    out, lse, dq, dk, dv = _fwd_bwd(dev, q, k, v, d_o, generate_tanh_softcap(50.0), bm)
    rows = [0, 3, 4, 127, 1023, 1024, 1025, 1028, 4095, 4096, 8191]
    _check_sampled_rows(q, k, v, d_o, out, lse, dq, o_tanh_softcap(50.0), o_sink_window_lt(1024, 4), torch.bfloat16,
                        (0, 3), (0, 15), rows)
    # one whole head of 8192 x 8192 entries (a few GB of fp32 temporaries on the host)
    _check_whole_heads(q, k, v, d_o, dq, dk, dv, o_tanh_softcap(50.0), o_sink_window_lt(1024, 4), torch.bfloat16, ((3, 9),))
    _check_identities(q, k, v, d_o, out.cpu(), dq.cpu(), dk.cpu(), dv.cpu(), additive=False)


@pytest.mark.parametrize("Lq", [1, 16, 64])
def test_config5_full_size(dev, Lq):
    """fp16 Q [8,8,Lq,64] against KV [8,8,16384,64], ALiBi, offset-causal: decode kernel vs the oracle on two heads,
    vs the forward kernel everywhere, and independent of the split count."""
    print(f"case config 5 full size q_len {Lq}", flush=True)
    Lkv = 16384
    q, k, v, _ = _inputs(dev, torch.float16, 8, 8, Lq, Lkv, 64)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    score = generate_alibi_bias(8, -1.0)
    bm = fa.create_block_mask(offset_causal_mask(Lkv - Lq), 1, 1, Lq, Lkv, device=dev)
    out, lse = fa.flax_attention(qd, kd, vd, score_mod=score, block_mask=bm, return_lse=True)
    out16 = fa.flax_attention(qd, kd, vd, score_mod=score, block_mask=bm, kernel_options={"decode_splits": 16})
    pre = fa.flax_attention(qd, kd, vd, score_mod=score, block_mask=bm, kernel_options={"decode": False})
    assert max_abs(out.cpu(), out16.cpu()) <= 2e-3 and max_abs(out.cpu(), pre.cpu()) <= 4e-3
    for b, h in ((0, 0), (7, 7)):
        oal = o_alibi_config(8)
        want, want_lse = ref_attention(q[b:b + 1, h:h + 1], k[b:b + 1, h:h + 1], v[b:b + 1, h:h + 1],
                                       lambda s, bb, hh, qi, ki: oal(s, bb, hh + h, qi, ki), o_offset_causal(Lkv - Lq),
                                       strict=True, return_lse=True)
        a, r = max_abs(out[b:b + 1, h:h + 1].cpu(), want), rel_l2(out[b:b + 1, h:h + 1].cpu(), want)
        print(f"  (b{b},h{h}): O max-abs {a:.3e} rel-L2 {r:.3e}", flush=True)
        assert a <= 2e-2 and r <= 1e-3
        assert max_abs(lse[b:b + 1, h:h + 1].cpu(), want_lse) <= 2e-2


@pytest.mark.parametrize("dtype,D,B,H,L", [(torch.float16, 128, 33, 32, 16384), (torch.float32, 128, 33, 32, 16384),
                                           (torch.bfloat16, 256, 17, 32, 16384)],
                         ids=["f16_d128_tuned", "f32_d128_simple", "bf16_d256_simple"])
def test_tensors_beyond_2_31_elements(dev, dtype, D, B, H, L):
    """Q, K, V, O and the gradients hold more than 2^31 elements each (and more than 2^32 bytes), so every row address
    of the last batch element lies beyond what 32 bits reach.  The (batch, head) pairs of a call are independent
    and their tile schedules identical, so the last pair's slice of the big call must equal, bit for bit, a call on
    that slice alone (whose addresses are small): forward, lse, dQ, dK, dV under a causal block mask."""
    assert B * H * L * D > 2 ** 31
    g = torch.Generator(device=dev).manual_seed(5)
    mk = lambda: torch.randn((B, H, L, D), generator=g, dtype=torch.float32 if dtype == torch.float32 else torch.float16,
                             device=dev).to(dtype)
    q, k, v = (mk().requires_grad_(True) for _ in range(3))
    d_o = mk()
    bm = fa.create_block_mask(causal_mask, 1, 1, L, L, device=dev)
    score = generate_alibi_bias(H, -1.0)
    out, lse = fa.flax_attention(q, k, v, score_mod=score, block_mask=bm, return_lse=True)
    gq, gk, gv = torch.autograd.grad(out, (q, k, v), d_o)
    b, h = B - 1, H - 1
    qs, ks, vs = (t[b:b + 1, h:h + 1].detach().clone().requires_grad_(True) for t in (q, k, v))
    # head H-1 of H has the ALiBi slope 2^-8, and so has head 0 of 1
    shifted = generate_alibi_bias(1, -1.0)
    # (one pair alone would be split over the keys to fill the GPU, which sums in another order: switched off)
    out1, lse1 = fa.flax_attention(qs, ks, vs, score_mod=shifted, block_mask=bm, return_lse=True,
                                   kernel_options={"split_kv": False})
    gq1, gk1, gv1 = torch.autograd.grad(out1, (qs, ks, vs), d_o[b:b + 1, h:h + 1].clone())
    torch.cuda.synchronize()
    for name, big, small in (("O", out, out1), ("lse", lse, lse1), ("dQ", gq, gq1), ("dK", gk, gk1), ("dV", gv, gv1)):
        sl = big[b:b + 1, h:h + 1]
        assert torch.equal(sl, small), f"{name}: slice of the big call differs from the call on the slice"
