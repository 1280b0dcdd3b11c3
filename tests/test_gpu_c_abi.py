"""The C ABI called directly (ctypes, raw pointers), for the promises of include/flexattn.h that the Python layer
never exercises by itself: optional pointers, calls without tile lists, error returns that launch nothing."""
import ctypes as C
import math

import pytest
import torch

from flaxattention_amd import _lib
from oracle import max_abs, o_causal_mask, ref_attention, rel_l2

pytestmark = pytest.mark.gpu

INT_MIN, INT_MAX = -2 ** 31, 2 ** 31 - 1


def _params(q, k, v, o, lo=INT_MIN, hi=INT_MAX):
    B, H, Lq, D = q.shape
    p = _lib.FlexAttnParams()
    p.dtype = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}[q.dtype]
    p.B, p.Hq, p.Hkv, p.Lq, p.Lkv, p.D, p.Dv = B, H, k.shape[1], Lq, k.shape[2], D, v.shape[3]
    for name, t in (("q_stride", q), ("k_stride", k), ("v_stride", v), ("o_stride", o)):
        getattr(p, name)[:] = [t.stride(0), t.stride(1), t.stride(2)]
    p.scale, p.flags = 1.0 / math.sqrt(D), 1   # FLEX_ROUND_S
    p.score.kind = 0
    p.mask.kind, p.mask.lo, p.mask.hi, p.mask.sink = 0, lo, hi, -1
    return p


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _inputs(dev, B, H, Lq, Lkv, D, dtype=torch.float16):
    g = torch.Generator(device="cpu").manual_seed(7)
    mk = lambda *s: torch.randn(*s, generator=g, dtype=torch.float32).to(dtype).to(dev)
    return mk(B, H, Lq, D), mk(B, H, Lkv, D), mk(B, H, Lkv, D)


def test_forward_without_lse_and_without_lists(dev):
    print("case C ABI forward, causal band mask, no lists, lse2 NULL", flush=True)
    L = _lib.lib()
    q, k, v = _inputs(dev, 2, 2, 256, 256, 64)
    o1, o2 = torch.empty_like(q), torch.empty_like(q)
    lse = torch.empty(2, 2, 256, dtype=torch.float32, device=dev)
    p = _params(q, k, v, o1, lo=0)   # d = q - kv >= 0: causal
    assert L.flexattn_fwd(p, q.data_ptr(), k.data_ptr(), v.data_ptr(), o1.data_ptr(), lse.data_ptr(), None, _stream()) == 0
    assert L.flexattn_fwd(p, q.data_ptr(), k.data_ptr(), v.data_ptr(), o2.data_ptr(), None, None, _stream()) == 0
    torch.cuda.synchronize()
    assert torch.equal(o1, o2)
    want, want_lse = ref_attention(q.cpu(), k.cpu(), v.cpu(), None, o_causal_mask, strict=True, return_lse=True)
    assert rel_l2(o1.cpu(), want) <= 1e-3 and max_abs(lse.cpu() * math.log(2.0), want_lse) <= 2e-2


def test_errors_launch_nothing(dev):
    print("case C ABI error returns", flush=True)
    L = _lib.lib()
    q, k, v = _inputs(dev, 1, 2, 128, 128, 64)
    o = torch.full_like(q, 7.0)
    p = _params(q, k, v, o)
    assert L.flexattn_fwd(p, None, k.data_ptr(), v.data_ptr(), o.data_ptr(), None, None, _stream()) != 0
    assert b"null" in L.flexattn_last_error()
    p.Lkv = 0
    assert L.flexattn_fwd(p, q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), None, None, _stream()) != 0
    assert b"non-positive" in L.flexattn_last_error()
    p = _params(q, k, v, o)
    p.Hkv = 3   # 2 query heads do not divide over 3 KV heads
    assert L.flexattn_fwd(p, q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), None, None, _stream()) != 0
    p = _params(q, k, v, o)
    p.q_index_base = 64
    assert L.flexattn_fwd(p, q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), None, None, _stream()) != 0
    p = _params(q, k, v, o)   # decode takes at most 64 query columns
    ws = torch.empty(1 << 20, dtype=torch.uint8, device=dev)
    assert L.flexattn_decode(p, q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), None, 2, ws.data_ptr(), _stream()) != 0
    assert b"at most 64 query columns" in L.flexattn_last_error()
    p.mask.kind = 1   # a bitmap mask without a bitmap
    assert L.flexattn_fwd(p, q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), None, None, _stream()) != 0
    torch.cuda.synchronize()
    assert bool((o == 7.0).all())   # nothing was launched by any of the refused calls


def test_block_mask_build_with_optional_outputs(dev):
    print("case C ABI block-mask build, some outputs NULL", flush=True)
    L = _lib.lib()
    B, H, nq, nkv = 2, 3, 5, 7
    m = _lib.FlexMask()
    m.kind, m.lo, m.hi, m.sink = 0, 0, 200, 3   # causal window of 200 with 4 sink keys
    i32 = dict(dtype=torch.int32, device=dev)
    full = {n: torch.empty(s, **i32) for n, s in (("kv_num", (B, H, nq)), ("kv_idx", (B, H, nq, nkv)),
                                                  ("full_kv_num", (B, H, nq)), ("full_kv_idx", (B, H, nq, nkv)),
                                                  ("q_num", (B, H, nkv)), ("q_idx", (B, H, nkv, nq)),
                                                  ("full_q_num", (B, H, nkv)), ("full_q_idx", (B, H, nkv, nq)))}
    ws = torch.empty(L.flexattn_block_mask_workspace_bytes(B, H, nq, nkv), dtype=torch.uint8, device=dev)
    ptr = lambda t: t.data_ptr()
    order = ("kv_num", "kv_idx", "full_kv_num", "full_kv_idx", "q_num", "q_idx", "full_q_num", "full_q_idx")
    assert L.flexattn_block_mask_build(C.byref(m), B, H, nq, nkv, 128, 128, *[ptr(full[n]) for n in order],
                                       ws.data_ptr(), _stream()) == 0
    only = {n: torch.full_like(full[n], -5) for n in ("kv_num", "full_q_idx")}
    assert L.flexattn_block_mask_build(C.byref(m), B, H, nq, nkv, 128, 128,
                                       *[ptr(only[n]) if n in only else None for n in order],
                                       ws.data_ptr(), _stream()) == 0
    torch.cuda.synchronize()
    assert torch.equal(only["kv_num"], full["kv_num"]) and torch.equal(only["full_q_idx"], full["full_q_idx"])
    # the transposed counts agree with the row counts: same number of partial / full tiles either way
    assert int(full["kv_num"].sum()) == int(full["q_num"].sum())
    assert int(full["full_kv_num"].sum()) == int(full["full_q_num"].sum())
    assert L.flexattn_block_mask_build(C.byref(m), B, H, 0, nkv, 128, 128, *[None] * 8, ws.data_ptr(), _stream()) != 0
    assert L.flexattn_block_mask_build(C.byref(m), B, H, nq, nkv, 128, 128, *[None] * 8, None, _stream()) != 0


def test_decode_with_lists_of_another_granularity(dev):
    """Tile lists built at 128 x 128 (the API's block size) instead of the 128 x 64 the decode kernel walks: the
    kernel must not read them as 64-key tiles.  Result = the call without lists."""
    print("case C ABI decode, lists at 128 x 128", flush=True)
    import flaxattention_amd as fa
    from flaxattention_amd.core.blockmask import build_lists
    from flaxattention_amd.masks import generate_sliding_window
    L = _lib.lib()
    B, H, Lq, Lkv, D = 2, 4, 16, 1024, 64
    q, k, v = _inputs(dev, B, H, Lq, Lkv, D)
    outs = []
    spec = generate_sliding_window(300)
    spec_off = type(spec)(lo=spec.lo, hi=spec.hi, sink=spec.sink, q_offset=Lkv - Lq)
    lists = build_lists(spec_off, 1, 1, 1, Lkv // 128, 128, 128, dev)
    for use_lists in (False, True):
        o = torch.empty_like(q)
        p = _params(q, k, v, o, lo=spec.lo, hi=spec.hi)
        p.mask.q_offset = Lkv - Lq
        if use_lists:
            t = p.tiles
            t.kv_num, t.kv_idx = lists["kv_num_blocks"].data_ptr(), lists["kv_indices"].data_ptr()
            t.full_kv_num, t.full_kv_idx = lists["full_kv_num_blocks"].data_ptr(), lists["full_kv_indices"].data_ptr()
            t.q_block, t.kv_block, t.n_q_blocks, t.n_kv_blocks = 128, 128, 1, Lkv // 128
        ws = torch.empty(L.flexattn_decode_workspace_bytes(p, 4), dtype=torch.uint8, device=dev)
        assert L.flexattn_decode(p, q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), None, 4, ws.data_ptr(), _stream()) == 0
        torch.cuda.synchronize()
        outs.append(o)
    assert torch.equal(outs[0], outs[1])
    want = fa.flax_attention(q, k, v, block_mask=fa.create_block_mask(spec_off, 1, 1, Lq, Lkv, device=dev),
                             kernel_options={"decode": False})
    assert max_abs(outs[0].cpu(), want.cpu()) <= 4e-3


def test_threads_on_their_own_streams(dev):
    """The entry points keep no state between calls: two host threads, each on a stream of its own, run forward +
    backward (tuned, simple and decode kernels) on different problems at the same time; every result equals, bit for
    bit, the one of the same call made alone.  An error in one thread leaves the other thread's error string alone."""
    import threading
    import flaxattention_amd as fa
    from flaxattention_amd.masks import causal_mask
    from flaxattention_amd.mods import generate_alibi_bias
    torch.cuda.synchronize()
    cases = [(torch.float16, 2, 4, 384, 384, 64), (torch.bfloat16, 1, 4, 300, 520, 128),
             (torch.float32, 1, 2, 256, 256, 64), (torch.float16, 2, 4, 8, 2048, 128)]

    def work(seed, out):
        res = []
        for i, (dtype, B, H, Lq, Lkv, D) in enumerate(cases):
            g = torch.Generator(device=dev).manual_seed(100 * seed + i)
            q, k, v = (torch.randn(B, H, L, D, generator=g, device=dev, dtype=torch.float32).to(dtype).requires_grad_(True)
                       for L in (Lq, Lkv, Lkv))
            bm = fa.create_block_mask(causal_mask, 1, 1, Lq, Lkv, device=dev) if Lq == Lkv else None
            o, lse = fa.flax_attention(q, k, v, score_mod=generate_alibi_bias(H, -1.0), block_mask=bm, return_lse=True)
            grads = torch.autograd.grad(o.float().square().sum(), (q, k, v))
            res.append((o.detach(), lse.detach()) + tuple(grads))
        out[seed] = res

    alone = {}
    for seed in (1, 2):
        work(seed, alone)
    torch.cuda.synchronize()
    together, errors = {}, {}

    def threaded(seed):
        try:
            with torch.cuda.stream(torch.cuda.Stream(device=dev)):
                for _ in range(3):
                    work(seed, together)
                if seed == 2:   # an error of this thread's own
                    L = _lib.lib()
                    q, k, v = _inputs(dev, 1, 2, 128, 128, 64)
                    p = _params(q, k, v, torch.empty_like(q))
                    assert L.flexattn_fwd(p, None, k.data_ptr(), v.data_ptr(), q.data_ptr(), None, None, _stream()) != 0
                    errors[seed] = L.flexattn_last_error()
                else:
                    errors[seed] = _lib.lib().flexattn_last_error()
                torch.cuda.current_stream().synchronize()
        except Exception as e:   # pragma: no cover
            errors[seed] = e

    threads = [threading.Thread(target=threaded, args=(s,)) for s in (1, 2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert isinstance(errors[2], bytes) and b"null" in errors[2], errors[2]
    assert isinstance(errors[1], bytes) and b"null" not in errors[1], errors[1]
    for seed in (1, 2):
        for a, b in zip(alone[seed], together[seed]):
            for x, y in zip(a, b):
                assert torch.equal(x, y)
