"""CPU oracle: a restatement of the reference's dense FlexAttention path.

TEST INFRASTRUCTURE ONLY -- never imported by the shipped package.  Only
tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg use it, and
only as the checker.

What is restated (citations are into the reference tree):

* score/mask mods          flaxattention/masks/causal.py:4-5,
                           flaxattention/masks/sliding_window.py:7-22,
                           flaxattention/masks/attention_sink.py:6-24,
                           flaxattention/mods/alibi.py:5-20,
                           examples/benchmark.py:16-22 (checkerboard)
* block-mask builder       flaxattention/core/blockmask.py:57-64 (ordering),
                           253-274, 277-322 (dense mask), 335-369 (block
                           reduction), 400-455 (entry, rounding rules)
* dense attention          flaxattention/core/attention.py:14-65 (scores,
                           scale, mods, -inf masking), 67-106 (GQA repeat,
                           logsumexp, masked softmax, PV, base-2 LSE),
                           169-218 (defaults and the natural-log LSE)
* backward                 reverse-mode differentiation of the lines above,
                           written out by hand with the dtype round-trips the
                           forward implies (the reference relies on jax.grad)

Parity pinning status (what checks each function independently of this file):

* ref_create_block_mask: pinned by torch.nn.attention.flex_attention's
  create_block_mask on CPU (same algorithm) and by hand-derived vectors in
  tests/golden/block_mask_vectors.json.
* ref_attention forward:  pinned by torch SDPA (identity / causal / boolean
  masks / additive ALiBi bias), torch flex_attention on CPU (the comparator
  the reference's own tests use, tests/attention_test.py:52-63), an fp64
  brute-force loop on tiny inputs, and algebraic invariants.
* ref_attention_bwd: pinned by torch autograd through an fp64 dense forward
  and by finite differences.
* strict=True, placement of the 16-bit rounding points (S before the scale, P,
  dP, dS after the scale): pinned by a literal transcription of
  attention.py:27, 55, 97-105 with torch's own fp16 / bf16 CPU matrix products,
  differentiated by torch autograd (so autograd, not this file's author, places
  the backward's roundings), and by four deliberately misplaced roundings
  (MUTANTS below) that the test must tell apart from the real thing.
* PARITY UNPINNED: whether the reference's XLA executable really performs the
  input-dtype round trips on S, P, dP and dS (``strict=True``) or elides them
  (``strict=False``).  Both variants are provided; no fixture can decide.
* PARITY UNPINNED: the gradient on fully masked rows (defined here as 0).
"""
from __future__ import annotations

import math
from typing import Callable, Optional

import numpy as np
import torch

__all__ = [
    "o_noop_mask", "o_causal_mask", "o_offset_causal", "o_sliding_window",
    "o_attention_sink", "o_sink_window_lt", "o_full_masked", "o_and_masks",
    "o_or_masks", "o_identity", "o_alibi", "o_alibi_config", "o_checkerboard",
    "o_checkerboard_kv", "o_tanh_softcap", "o_rel_bias",
    "ref_create_mask", "ref_create_block_mask", "ref_attention",
    "ref_attention_bwd", "truth_attention", "max_abs", "rel_l2", "seeded_qkv",
]


# --------------------------------------------------------------------------
# mods.  Every mod is a broadcasting function of torch tensors; the reference
# maps scalar functions over (b, h, q, kv) with four nested vmaps
# (flaxattention/core/common.py:41-80), which is the same thing.
# --------------------------------------------------------------------------
def o_noop_mask(b, h, q_idx, kv_idx):
    """blockmask.py:20-27."""
    return torch.ones((), dtype=torch.bool)


def o_causal_mask(b, h, q_idx, kv_idx):
    """masks/causal.py:4-5."""
    return q_idx >= kv_idx


def o_offset_causal(offset: int):
    """Causal mask aligned to the last query position (decode): the query row
    i sits at absolute position i + offset."""
    def mask(b, h, q_idx, kv_idx):
        return q_idx + offset >= kv_idx
    return mask


def o_and_masks(*mods):
    """blockmask.py:386-397."""
    def mask(b, h, q_idx, kv_idx):
        r = torch.ones((), dtype=torch.bool)
        for m in mods:
            r = r & m(b, h, q_idx, kv_idx)
        return r
    return mask


def o_or_masks(*mods):
    """blockmask.py:372-383."""
    def mask(b, h, q_idx, kv_idx):
        r = torch.zeros((), dtype=torch.bool)
        for m in mods:
            r = r | m(b, h, q_idx, kv_idx)
        return r
    return mask


def o_sliding_window(window: int):
    """masks/sliding_window.py:7-22."""
    def win(b, h, q_idx, kv_idx):
        return q_idx - kv_idx <= window
    return o_and_masks(win, o_causal_mask)


def o_attention_sink(window: int, sink: int = 4):
    """masks/attention_sink.py:6-24 (note the inclusive ``kv_idx <= sink``)."""
    def win(b, h, q_idx, kv_idx):
        return q_idx - kv_idx <= window

    def snk(b, h, q_idx, kv_idx):
        return kv_idx <= sink
    return o_and_masks(o_or_masks(snk, win), o_causal_mask)


def o_sink_window_lt(window: int, sink: int = 4):
    """The benchmark-config spelling: |q-kv| <= window, causal, and
    ``kv_idx < sink`` always visible."""
    def win(b, h, q_idx, kv_idx):
        return q_idx - kv_idx <= window

    def snk(b, h, q_idx, kv_idx):
        return kv_idx < sink
    return o_and_masks(o_or_masks(snk, win), o_causal_mask)


def o_full_masked(b, h, q_idx, kv_idx):
    """tests/attention_test.py:72-73 (``fullmask``)."""
    return torch.zeros((), dtype=torch.bool)


def o_identity(score, b, h, q_idx, kv_idx):
    """attention.py:109-116."""
    return score


def o_alibi(H: int):
    """mods/alibi.py:15-18: score + (q_idx - kv_idx) * exp2(-((h+1)*8/H))."""
    def mod(score, b, h, q_idx, kv_idx):
        slope = torch.exp2(-((h + 1).to(torch.float32) * 8.0 / H))
        return score + (q_idx - kv_idx).to(torch.float32) * slope
    return mod


def o_alibi_config(H: int):
    """The benchmark-config sign: slope * (kv_idx - q_idx)."""
    def mod(score, b, h, q_idx, kv_idx):
        slope = torch.exp2(-((h + 1).to(torch.float32) * 8.0 / H))
        return score + (kv_idx - q_idx).to(torch.float32) * slope
    return mod


def o_checkerboard(score, b, h, q_idx, kv_idx):
    """examples/benchmark.py:16-22: parity of (k_idx - q_idx) with floor-mod,
    even -> x0.5, odd -> x2.0."""
    par = torch.remainder(kv_idx - q_idx, 2)
    score = torch.where(par == 0, score * 0.5, score)
    score = torch.where(par == 1, score * 2.0, score)
    return score


def o_checkerboard_kv(score, b, h, q_idx, kv_idx):
    """The benchmark-config spelling: kv_idx odd -> x0.5, even -> x2.0."""
    par = torch.remainder(kv_idx + 0 * q_idx, 2)
    return torch.where(par == 1, score * 0.5, score * 2.0)


def o_tanh_softcap(cap: float):
    """cap * tanh(score / cap) (not in the reference; defined by the
    benchmark configuration)."""
    def mod(score, b, h, q_idx, kv_idx):
        return cap * torch.tanh(score / cap)
    return mod


def o_rel_bias(slope: float):
    """score + slope * (kv_idx - q_idx): head-independent relative-position
    bias (not in the reference; named by the build goal)."""
    def mod(score, b, h, q_idx, kv_idx):
        return score + (kv_idx - q_idx).to(torch.float32) * slope
    return mod


# --------------------------------------------------------------------------
# block mask
# --------------------------------------------------------------------------
def _idx(n, pos, nd=4):
    shape = [1] * nd
    shape[pos] = n
    return torch.arange(n, dtype=torch.int32).reshape(shape)


def ref_create_mask(mod_fn, B, H, Q_LEN, KV_LEN, n_args: Optional[int] = None) -> np.ndarray:
    """Dense bool mask [B,H,Q,KV] (blockmask.py:277-322).  A five-argument
    score_mod is run on zeros and masks where the result is -inf (307-315)."""
    B = 1 if B is None else B
    H = 1 if H is None else H
    b, h, m, n = _idx(B, 0), _idx(H, 1), _idx(Q_LEN, 2), _idx(KV_LEN, 3)
    if n_args is None:
        import inspect
        n_args = sum(1 for p in inspect.signature(mod_fn).parameters.values()
                     if p.default is inspect.Parameter.empty)
    if n_args == 5:
        out = mod_fn(torch.zeros(B, H, Q_LEN, KV_LEN), b, h, m, n)
        mask = ~torch.isneginf(out)
    else:
        mask = mod_fn(b, h, m, n)
        if not torch.is_tensor(mask):
            mask = torch.tensor(bool(mask))
    mask = torch.broadcast_to(mask.to(torch.bool), (B, H, Q_LEN, KV_LEN))
    return mask.numpy()


def _dense_to_ordered(dense: np.ndarray):
    """blockmask.py:57-64: row sums, and a stable descending argsort of the
    0/1 row (selected ids ascending, then the unselected ids ascending)."""
    dense = dense.astype(np.int32)
    num = dense.sum(axis=-1).astype(np.int32)
    idx = np.argsort(-dense, axis=-1, kind="stable").astype(np.int32)
    return num, idx


def _ordered_to_dense_correct(num, idx):
    rows, cols = idx.shape[-2], idx.shape[-1]
    dense = np.zeros(idx.shape, dtype=np.int32)
    sel = np.arange(cols)[None, :] < num.reshape(-1, rows)[..., None]
    flat_idx = idx.reshape(-1, rows, cols)
    flat_dense = dense.reshape(-1, rows, cols)
    for p in range(flat_idx.shape[0]):
        for r in range(rows):
            flat_dense[p, r, flat_idx[p, r][sel[p, r]]] = 1
    return flat_dense.reshape(idx.shape)


def ref_create_block_mask(mask_mod, B, H, Q_LEN, KV_LEN, BLOCK_SIZE=128) -> dict:
    """blockmask.py:419-455 and everything it calls.

    Returns a dict of int32 arrays: kv_num_blocks, kv_indices,
    full_kv_num_blocks, full_kv_indices (bit-exact targets); q_* lists as the
    *correct* transposes (what torch's original computes); refq_* lists as the
    reference really produces them -- blockmask.py:46-47 discards the scatter,
    so its dense matrix is all zeros: every count is 0 and every index row is
    arange.  Also BLOCK_SIZE, which the reference always reports as (128,128)
    (blockmask.py:449-454 does not forward the sizes), and the sizes actually
    used for the reduction.
    """
    B = 1 if B is None else B
    H = 1 if H is None else H
    if isinstance(BLOCK_SIZE, int):
        QB = KVB = BLOCK_SIZE
    else:
        QB, KVB = BLOCK_SIZE
    if Q_LEN < 128:
        QB = Q_LEN
    else:
        Q_LEN = (Q_LEN + QB - 1) // QB * QB
    KV_LEN = (KV_LEN + KVB - 1) // KVB * KVB
    mask = ref_create_mask(mask_mod, B, H, Q_LEN, KV_LEN)
    m = mask.reshape(B, H, Q_LEN // QB, QB, KV_LEN // KVB, KVB).transpose(0, 1, 2, 4, 3, 5)
    s = m.sum(axis=(-2, -1), dtype=np.int64)
    full = (s == QB * KVB).astype(np.int8)
    partial = ((s > 0) & (s < QB * KVB)).astype(np.int8)
    kv_num, kv_idx = _dense_to_ordered(partial)
    fkv_num, fkv_idx = _dense_to_ordered(full)
    q_num, q_idx = _dense_to_ordered(np.swapaxes(partial, -1, -2))
    fq_num, fq_idx = _dense_to_ordered(np.swapaxes(full, -1, -2))
    zeros_t = np.zeros(np.swapaxes(partial, -1, -2).shape, dtype=np.int8)
    rq_num, rq_idx = _dense_to_ordered(zeros_t)
    return dict(
        kv_num_blocks=kv_num, kv_indices=kv_idx,
        full_kv_num_blocks=fkv_num, full_kv_indices=fkv_idx,
        q_num_blocks=q_num, q_indices=q_idx,
        full_q_num_blocks=fq_num, full_q_indices=fq_idx,
        refq_num_blocks=rq_num, refq_indices=rq_idx,
        BLOCK_SIZE=(128, 128), used_block_size=(QB, KVB),
        partial=partial, full=full,
    )


# --------------------------------------------------------------------------
# dense attention
# --------------------------------------------------------------------------
def _rt(x: torch.Tensor, dtype, strict: bool) -> torch.Tensor:
    """Round an fp32 tensor through ``dtype`` (no-op in non-strict mode)."""
    if not strict or dtype in (torch.float32, torch.float64):
        return x
    return x.to(dtype).to(x.dtype)


def _mods_for_slice(score_mod, mask_mod, b0, nb, Hq, M, N):
    b = (_idx(nb, 0) + b0)
    return b, _idx(Hq, 1), _idx(M, 2), _idx(N, 3)


# Test hook: deliberately WRONG placements of the 16-bit rounding points, so that the test that pins the
# placement (tests/test_oracle_cpu.py::test_rounding_points_against_torch_half_program) can show that it
# would notice each of them.  Never set outside that test.
MUTANTS = ("s_after_scale", "p_unrounded", "dp_unrounded", "ds_unrounded")


def _forward_slice(q, k, v, score_mod, mask_mod, scale, strict, b0, want_grad_mod=False, _mutant=None):
    """q,k,v: [nb,H,*,*] slices already GQA-expanded.  Returns fp32 tensors
    X (post-mod, -inf masked), P (normalised), lse (natural), and optionally
    dmod/dS."""
    dtype = q.dtype
    wp = torch.float64 if dtype == torch.float64 else torch.float32
    nb, Hq, M, _ = q.shape
    N = k.shape[2]
    # attention.py:27 -- matmul in the input dtype, then cast to fp32
    S = torch.matmul(q.to(wp), k.to(wp).transpose(-1, -2))
    if _mutant == "s_after_scale":
        S = _rt(S * scale, dtype, strict)
    else:
        S = _rt(S, dtype, strict)
        S = S * scale                                # attention.py:55
    b, h, m, n = _mods_for_slice(score_mod, mask_mod, b0, nb, Hq, M, N)
    mask = mask_mod(b, h, m, n)                      # attention.py:57-58
    if not torch.is_tensor(mask):
        mask = torch.tensor(bool(mask))
    mask = torch.broadcast_to(mask.to(torch.bool), S.shape)
    gmod = None
    if want_grad_mod:
        Sg = S.detach().clone().requires_grad_(True)
        Y = score_mod(Sg, b, h, m, n)
        (gmod,) = torch.autograd.grad(Y.sum(), Sg)
        Y = Y.detach()
    else:
        Y = score_mod(S, b, h, m, n)
    Y = Y.to(wp)
    X = torch.where(mask, Y, torch.full((), -math.inf, dtype=wp))  # attention.py:59-63
    mx = X.max(dim=-1, keepdim=True).values
    dead = torch.isneginf(mx)
    mx0 = torch.where(dead, torch.zeros_like(mx), mx)
    E = torch.exp(X - mx0)
    Z = E.sum(dim=-1, keepdim=True)
    lse = torch.where(dead, mx, mx0 + torch.log(Z)).squeeze(-1)      # attention.py:97-99
    P = torch.where(dead, torch.zeros_like(E), E / torch.where(dead, torch.ones_like(Z), Z))  # :104
    return X, P, lse, mask, gmod


def _expand_gqa(x, G):
    return x if G == 1 else torch.repeat_interleave(x, G, dim=1)   # attention.py:80-82


def ref_attention(q, k, v, score_mod=None, mask_mod=None, scale=None, strict=True,
                  return_lse=False, batch_chunk: int = 1, _mutant=None):
    """flax_attention (attention.py:169-218) on CPU.  ``mask_mod`` is the
    scalar mask function (the only field of the block mask the reference's
    dense path reads, attention.py:45).  Returns O in the input dtype and,
    optionally, the natural-log LSE [B,H,Lq] in fp32 (-inf on dead rows)."""
    score_mod = score_mod or o_identity
    mask_mod = mask_mod or o_noop_mask
    if scale is None:
        scale = 1.0 / math.sqrt(q.shape[-1])
    dtype = q.dtype
    wp = torch.float64 if dtype == torch.float64 else torch.float32
    G = q.shape[1] // k.shape[1]
    outs, lses = [], []
    for b0 in range(0, q.shape[0], batch_chunk):
        sl = slice(b0, b0 + batch_chunk)
        kk, vv = _expand_gqa(k[sl], G), _expand_gqa(v[sl], G)
        _, P, lse, _, _ = _forward_slice(q[sl], kk, vv, score_mod, mask_mod, scale, strict, b0, _mutant=_mutant)
        O = torch.matmul(_rt(P, dtype, strict and _mutant != "p_unrounded"), vv.to(wp))          # attention.py:105
        outs.append(O.to(dtype))
        lses.append(lse)
    O = torch.cat(outs, 0)
    if return_lse:
        return O, torch.cat(lses, 0)
    return O


def ref_attention_bwd(q, k, v, dO, score_mod=None, mask_mod=None, scale=None, strict=True,
                      batch_chunk: int = 1, _mutant=None):
    """Gradients (dQ, dK, dV) of sum(O * dO) for ref_attention, i.e. what
    jax.grad yields through attention.py:14-106 with the dtype round trips of
    the forward transposed: dP and dS pass through the input dtype in strict
    mode.  Rows with no visible key get zero gradient."""
    score_mod = score_mod or o_identity
    mask_mod = mask_mod or o_noop_mask
    if scale is None:
        scale = 1.0 / math.sqrt(q.shape[-1])
    dtype = q.dtype
    wp = torch.float64 if dtype == torch.float64 else torch.float32
    Hkv = k.shape[1]
    G = q.shape[1] // Hkv
    dQs, dKs, dVs = [], [], []
    for b0 in range(0, q.shape[0], batch_chunk):
        sl = slice(b0, b0 + batch_chunk)
        kk, vv = _expand_gqa(k[sl], G), _expand_gqa(v[sl], G)
        qq, dd = q[sl], dO[sl].to(wp)
        _, P, _, mask, gmod = _forward_slice(qq, kk, vv, score_mod, mask_mod, scale, strict, b0,
                                             want_grad_mod=True, _mutant=_mutant)
        Pd = _rt(P, dtype, strict and _mutant != "p_unrounded")
        dV = torch.matmul(Pd.transpose(-1, -2), dd)
        dP = _rt(torch.matmul(dd, vv.to(wp).transpose(-1, -2)), dtype, strict and _mutant != "dp_unrounded")
        delta = (P * dP).sum(dim=-1, keepdim=True)
        dX = P * (dP - delta)
        dS = torch.where(mask, dX * gmod.to(wp), torch.zeros_like(dX)) * scale
        dS = _rt(dS, dtype, strict and _mutant != "ds_unrounded")
        dQ = torch.matmul(dS, kk.to(wp))
        dK = torch.matmul(dS.transpose(-1, -2), qq.to(wp))
        if G > 1:
            nb = dK.shape[0]
            dK = dK.reshape(nb, Hkv, G, *dK.shape[2:]).sum(2)
            dV = dV.reshape(nb, Hkv, G, *dV.shape[2:]).sum(2)
        dQs.append(dQ.to(dtype)); dKs.append(dK.to(dtype)); dVs.append(dV.to(dtype))
    return torch.cat(dQs, 0), torch.cat(dKs, 0), torch.cat(dVs, 0)


def truth_attention(q, k, v, dO=None, score_mod=None, mask_mod=None, scale=None, batch_chunk=1):
    """fp64 dense evaluation on the same (dtype-valued) inputs: no rounding
    anywhere.  Returns O (and dQ,dK,dV when dO is given) in fp64."""
    q64, k64, v64 = q.double(), k.double(), v.double()
    O = ref_attention(q64, k64, v64, score_mod, mask_mod, scale if scale is not None
                      else 1.0 / math.sqrt(q.shape[-1]), strict=False, batch_chunk=batch_chunk)
    if dO is None:
        return O
    g = ref_attention_bwd(q64, k64, v64, dO.double(), score_mod, mask_mod,
                          scale if scale is not None else 1.0 / math.sqrt(q.shape[-1]),
                          strict=False, batch_chunk=batch_chunk)
    return (O,) + g


# --------------------------------------------------------------------------
# helpers shared by tests and the bench
# --------------------------------------------------------------------------
def max_abs(a, b) -> float:
    return (a.double() - b.double()).abs().max().item() if a.numel() else 0.0


def rel_l2(a, b) -> float:
    """||a-b||_2 / ||b||_2 (b is the oracle)."""
    d = (a.double() - b.double()).norm().item()
    n = b.double().norm().item()
    return d / n if n > 0 else d


def seeded_qkv(B, Hq, Hkv, Lq, Lkv, D, dtype, Dv=None):
    """Standard-normal Q/K/V: seed 0 -> key, 1 -> query, 2 -> value as in
    tests/attention_test.py:32-40, drawn in fp32 and cast to ``dtype``.  The
    reference's threefry streams cannot be reproduced without JAX; parity is
    defined on identical inputs to both sides."""
    Dv = D if Dv is None else Dv

    def draw(seed, shape):
        g = torch.Generator().manual_seed(seed)
        return torch.randn(shape, generator=g, dtype=torch.float32).to(dtype)
    k = draw(0, (B, Hkv, Lkv, D))
    q = draw(1, (B, Hq, Lq, D))
    v = draw(2, (B, Hkv, Lkv, Dv))
    return q, k, v
