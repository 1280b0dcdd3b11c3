"""Seeded differential sweep on the GPU: the matrix-core kernels (tuned, simple, decode, split forward) against the
faithful vector-ALU kernels of the same library, which tests/test_gpu_attention.py holds to the oracle at the stated
tolerances.  Both sides follow the same rounding points, so they must agree to about twice the stated relative-L2
bound (1e-3 for 16-bit inputs, 1e-4 for float32); where a gradient vanishes identically (a row that sees one key has
P = 1 and dS = 0) both hold rounding noise and an absolute bound applies."""
import math
import random

import pytest
import torch

import flaxattention_amd as fa
from flaxattention_amd.core.common import MaskMod
from flaxattention_amd.masks import causal_mask, generate_attention_sink, generate_sliding_window, offset_causal_mask
from flaxattention_amd.mods import generate_alibi_bias, generate_checkerboard, generate_rel_bias, generate_tanh_softcap

pytestmark = pytest.mark.gpu


def _rel_l2(a, b):
    a, b = a.float(), b.float()
    n = b.norm().item()
    return (a - b).norm().item() / n if n > 0 else (a - b).norm().item()


def _agree(name, a, b, dtype, fast_bf16):
    tol = 1e-2 if fast_bf16 else (2e-4 if dtype == torch.float32 else 2.5e-3)
    e = _rel_l2(a, b)
    small = (a.float() - b.float()).abs().max().item() <= (5e-5 if dtype == torch.float32 else 5e-3)
    assert torch.isfinite(a.float()).all(), f"{name}: not finite"
    assert math.isfinite(e) and (e <= tol or small), f"{name}: rel-L2 {e:.3e} against the faithful kernels (bound {tol:g})"


def _agree_lse(a, b):
    dead = torch.isneginf(b)
    assert torch.equal(torch.isneginf(a), dead), "lse: rows without visible keys differ"
    if (~dead).any():
        # one unit in the last place of a score rounded through fp16 at magnitude 32 .. 64 is 0.03
        assert (a[~dead] - b[~dead]).abs().max().item() <= 4e-2, "lse"


def _score(r, Hq, kinds):
    sk = r.choice(kinds)
    return sk, {"none": None, "alibi": generate_alibi_bias(Hq, -1.0), "softcap": generate_tanh_softcap(r.choice([5.0, 30.0])),
                "relbias": generate_rel_bias(0.01), "checker": generate_checkerboard(2.0, 0.5, "kv"),
                "square": (lambda s, b, h, q, k: s - 0.05 * s * s)}[sk]


@pytest.mark.parametrize("seed", range(60))
def test_forward_backward_against_faithful_kernels(dev, seed):
    r = random.Random(seed)
    dtype = r.choice([torch.float16, torch.bfloat16, torch.float32])
    D = r.choice([32, 64, 64, 96, 128, 128, 192, 256] if dtype != torch.float32 else [32, 64, 96, 128])
    Dv = D if r.random() < 0.8 else r.choice([d for d in (16, 32, 64, 128) if d <= D])
    B, Hkv, G = r.randint(1, 3), r.randint(1, 3), r.choice([1, 1, 2, 4])
    Hq = Hkv * G
    Lq = r.choice([1, 3, 17, 64, 65, 100, 128, 129, 200, 300, 513])
    Lkv = r.choice([1, 5, 63, 64, 128, 200, 333, 512, 777, 1024, 1500, 2300])
    mk = r.choice(["none", "causal", "offset", "window", "sink", "bitmap", "doc"])
    if mk == "none":
        mask = None
    elif mk == "causal":
        mask = causal_mask
    elif mk == "offset":
        mask = offset_causal_mask(Lkv - Lq)
    elif mk == "window":
        mask = generate_sliding_window(r.choice([16, 100, 400]))
    elif mk == "sink":
        mask = generate_attention_sink(r.choice([32, 200]), 4)
    elif mk == "bitmap":
        a, b_, c = r.randint(2, 9), r.randint(2, 9), r.randint(5, 13)
        mask = lambda b, h, q_idx, kv_idx: ((q_idx * a + kv_idx * b_ + h) % c) < (c // 2 + 1)   # noqa: E731
    else:
        ids = torch.randint(0, 3, (B, max(Lq, Lkv)), generator=torch.Generator().manual_seed(seed)).sort(dim=1).values.to(dev)
        mask = lambda b, h, q_idx, kv_idx: ids[b, q_idx] == ids[b, kv_idx]   # noqa: E731
    sk, score = _score(r, Hq, ["none", "alibi", "softcap", "relbias", "checker", "square"])
    opts = {}
    if r.random() < 0.25:
        opts["tile_lists"] = False
    if r.random() < 0.3 and dtype != torch.float32:
        opts["numerics"] = r.choice(["parity", "fast"])
    if r.random() < 0.15:
        opts["decode"] = False
    fast_bf16 = dtype == torch.bfloat16 and opts.get("numerics") == "fast"
    g = torch.Generator(device=dev).manual_seed(seed)
    mkt = lambda *s: torch.randn(*s, generator=g, device=dev, dtype=torch.float32).to(dtype)   # noqa: E731
    q, k, v = mkt(B, Hq, Lq, D), mkt(B, Hkv, Lkv, D), mkt(B, Hkv, Lkv, Dv)
    d_o = mkt(B, Hq, Lq, Dv)
    print(f"differential {seed}: {dtype} B{B} Hq{Hq} Hkv{Hkv} Lq{Lq} Lkv{Lkv} D{D} Dv{Dv} mask {mk} score {sk} {opts}", flush=True)
    res = []
    for o in (opts, {"strict": True}):
        qq, kk, vv = (t.clone().requires_grad_(True) for t in (q, k, v))
        bm = fa.create_block_mask(mask, B, Hq, Lq, Lkv, device=dev) if mask is not None else None
        out, lse = fa.flax_attention(qq, kk, vv, score_mod=score, block_mask=bm, enable_gqa=G > 1, return_lse=True, kernel_options=o)
        res.append((out, lse) + torch.autograd.grad(out, (qq, kk, vv), d_o))
    for i, name in enumerate(("O", "lse", "dQ", "dK", "dV")):
        if name == "lse":
            _agree_lse(res[0][i], res[1][i])
        else:
            _agree(name, res[0][i], res[1][i], dtype, fast_bf16)


@pytest.mark.parametrize("seed", range(60))
def test_decode_chunks_and_split_forward_against_faithful_kernels(dev, seed):
    r = random.Random(1000 + seed)
    dtype = r.choice([torch.float16, torch.bfloat16])
    D = r.choice([64, 128, 192, 256])
    cols = 32 if D >= 192 else 64
    B, Hkv, G = r.randint(1, 3), r.randint(1, 3), r.choice([1, 1, 2, 4, 8])
    Hq = Hkv * G
    mode = r.choice(["decode", "decode", "chunks", "split_forward"])
    if mode == "decode":
        Lq = r.randint(1, max(cols // G, 1))
    elif mode == "chunks":
        Lq = r.randint(cols // G + 1, 200)
    else:
        Lq = r.choice([65, 100, 128, 200, 300, 512])
    Lkv = r.choice([512, 640, 1000, 1024, 2047, 3000, 4096, 6001])
    off = Lkv - Lq
    mk = r.choice(["none", "offset", "window", "sink_window", "bitmap"])
    if mk == "none":
        mask = None
    elif mk == "offset":
        mask = offset_causal_mask(off)
    elif mk == "window":
        mask = MaskMod(lo=0, hi=r.choice([100, 700]), sink=-1, q_offset=off, name="window")
    elif mk == "sink_window":
        mask = MaskMod(lo=0, hi=r.choice([100, 700]), sink=4, q_offset=off, name="sink_window")
    else:
        a, b_, c = r.randint(2, 9), r.randint(2, 9), r.randint(5, 13)
        mask = lambda b, h, q_idx, kv_idx: ((q_idx * a + kv_idx * b_ + h) % c) < (c // 2 + 1)   # noqa: E731
    sk, score = _score(r, Hq, ["none", "alibi", "softcap", "relbias", "checker"])
    opts = {"decode": mode != "split_forward"}
    if opts["decode"] and r.random() < 0.5:
        opts["decode_splits"] = r.choice([1, 2, 3, 7, 16, 33, 64])
    if r.random() < 0.25:
        opts["tile_lists"] = False
    if r.random() < 0.3:
        opts["numerics"] = r.choice(["parity", "fast"])
    fast_bf16 = dtype == torch.bfloat16 and opts.get("numerics") == "fast"
    g = torch.Generator(device=dev).manual_seed(seed)
    mkt = lambda *s: torch.randn(*s, generator=g, device=dev, dtype=torch.float32).to(dtype)   # noqa: E731
    q, k, v = mkt(B, Hq, Lq, D), mkt(B, Hkv, Lkv, D), mkt(B, Hkv, Lkv, D)
    print(f"differential {seed}: {mode} {dtype} B{B} Hq{Hq} Hkv{Hkv} Lq{Lq} Lkv{Lkv} D{D} mask {mk} score {sk} {opts}", flush=True)
    res = []
    for o in (opts, {"strict": True}):
        bm = fa.create_block_mask(mask, B, Hq, Lq, Lkv, device=dev) if mask is not None else None
        res.append(fa.flax_attention(q, k, v, score_mod=score, block_mask=bm, enable_gqa=G > 1, return_lse=True, kernel_options=o))
    _agree("O", res[0][0], res[1][0], dtype, fast_bf16)
    _agree_lse(res[0][1], res[1][1])
