"""flexattn_decode_static (the decode entry point that allocates nothing and keeps its split-KV partials in a buffer
inside the library image) against flexattn_decode with a caller workspace: same bits, on two calls in a row, the
second on a smaller problem, so that what the first call left in the shared buffer is seen not to matter."""
import math

import pytest
import torch

from flaxattention_amd import _lib

pytestmark = pytest.mark.gpu

INT_MIN, INT_MAX = -2 ** 31, 2 ** 31 - 1
STATIC_BYTES = 16 << 20


def _params(q, k, v, o, q_offset):
    B, Hq, Lq, D = q.shape
    p = _lib.FlexAttnParams()
    p.dtype = {torch.float16: 1, torch.bfloat16: 2}[q.dtype]
    p.B, p.Hq, p.Hkv, p.Lq, p.Lkv, p.D, p.Dv = B, Hq, k.shape[1], Lq, k.shape[2], D, v.shape[3]
    for name, t in (("q_stride", q), ("k_stride", k), ("v_stride", v), ("o_stride", o)):
        getattr(p, name)[:] = [t.stride(0), t.stride(1), t.stride(2)]
    p.scale, p.flags = 1.0 / math.sqrt(D), _lib.FLAG_ROUND_S
    p.score.kind, p.score.p0, p.score.i0 = _lib.SCORE_ALIBI, -1.0, Hq
    # offset-causal band: query row i sits at position i + q_offset
    p.mask.kind, p.mask.lo, p.mask.hi, p.mask.sink, p.mask.q_offset = _lib.MASK_BAND, 0, INT_MAX, -1, q_offset
    return p


def _both(dev, B, Hq, Hkv, Lq, Lkv, D, dtype, splits, seed):
    g = torch.Generator(device="cpu").manual_seed(seed)
    mk = lambda *s: torch.randn(*s, generator=g, dtype=torch.float32).to(dtype).to(dev)
    q, k, v = mk(B, Hq, Lq, D), mk(B, Hkv, Lkv, D), mk(B, Hkv, Lkv, D)
    L = _lib.lib()
    s = torch.cuda.current_stream().cuda_stream
    o_ref, o_new = torch.zeros_like(q), torch.zeros_like(q)
    lse_ref = torch.zeros(B, Hq, Lq, dtype=torch.float32, device=dev)
    lse_new = torch.zeros_like(lse_ref)
    p = _params(q, k, v, o_ref, Lkv - Lq)
    nbytes = L.flexattn_decode_workspace_bytes(p, splits)
    assert 0 < nbytes <= STATIC_BYTES
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    rc = L.flexattn_decode(p, q.data_ptr(), k.data_ptr(), v.data_ptr(), o_ref.data_ptr(), lse_ref.data_ptr(), splits,
                           ws.data_ptr(), s)
    _lib.check(rc, "flexattn_decode")
    rc = L.flexattn_decode_static(p, q.data_ptr(), k.data_ptr(), v.data_ptr(), o_new.data_ptr(), lse_new.data_ptr(),
                                  splits, s)
    _lib.check(rc, "flexattn_decode_static")
    torch.cuda.synchronize()
    assert torch.isfinite(o_ref.float()).all() and o_ref.float().abs().max() > 0
    assert torch.equal(o_ref, o_new), (o_ref.float() - o_new.float()).abs().max().item()
    assert torch.equal(lse_ref, lse_new)


def test_static_decode_matches_workspace_decode_twice(dev):
    print("case flexattn_decode_static: fp16 [4,8,16,64] x KV 4096, 8 splits; then bf16 [2,4(kv 2),1,128] x KV 1000, default splits",
          flush=True)
    _both(dev, 4, 8, 8, 16, 4096, 64, torch.float16, 8, seed=11)
    _both(dev, 2, 4, 2, 1, 1000, 128, torch.bfloat16, 0, seed=12)


def test_static_decode_refuses_what_does_not_fit(dev):
    print("case flexattn_decode_static: partials beyond the built-in buffer are refused, nothing is launched", flush=True)
    L = _lib.lib()
    B, H, Lq, Lkv, D = 16, 16, 64, 8192, 128   # 16384 rows x 64 splits x 130 floats = 545 MB of partials
    q = torch.zeros(B, H, Lq, D, dtype=torch.float16, device=dev)
    k = torch.zeros(B, H, Lkv, D, dtype=torch.float16, device=dev)
    o = torch.full_like(q, 3.0)
    p = _params(q, k, k, o, Lkv - Lq)
    assert L.flexattn_decode_workspace_bytes(p, 64) > STATIC_BYTES
    rc = L.flexattn_decode_static(p, q.data_ptr(), k.data_ptr(), k.data_ptr(), o.data_ptr(), None, 64,
                                  torch.cuda.current_stream().cuda_stream)
    assert rc != 0 and b"exceed" in L.flexattn_last_error()
    torch.cuda.synchronize()
    assert bool((o == 3.0).all())
