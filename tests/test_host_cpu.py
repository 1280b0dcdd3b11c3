"""Host-side logic that needs no GPU: the C-ABI library loads and exports every
symbol the header declares, ctypes structs match the C layout, mask / score
functors fold and evaluate like the oracle's restatements, Python callables
are recognised, and argument validation raises the reference's errors."""
import ctypes
import os
import re
import subprocess
import sys

import pytest
import torch

import flaxattention_amd as fa
from flaxattention_amd import _lib
from flaxattention_amd.core.common import (INT_MAX, INT_MIN, MaskMod, ScoreMod, _fit_band, _get_mod_type,
                                           _ModificationType, _probe_score_mod, pack_bits, resolve_score_mod)
from flaxattention_amd.masks import (causal_mask, generate_attention_sink, generate_sliding_window, offset_causal_mask)
from flaxattention_amd.mods import (checkerboard, generate_alibi_bias, generate_checkerboard, generate_rel_bias,
                                    generate_tanh_softcap)
from oracle import (o_alibi, o_alibi_config, o_attention_sink, o_causal_mask, o_checkerboard, o_checkerboard_kv,
                    o_noop_mask, o_offset_causal, o_rel_bias, o_sink_window_lt, o_sliding_window, o_tanh_softcap)

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "flexattn.h")


def test_library_exports_every_declared_symbol():
    decl = set(re.findall(r"\b(flexattn_[a-z_]+)\s*\(", open(HEADER).read()))
    assert decl == set(_lib.EXPORTS), decl ^ set(_lib.EXPORTS)
    L = _lib.lib()
    for name in decl:
        assert hasattr(L, name), name
    assert L.flexattn_abi_version() == 4
    assert L.flexattn_last_error() is not None


def test_ctypes_structs_match_c_layout(tmp_path):
    src = tmp_path / "layout.c"
    src.write_text('#include <stdio.h>\n#include <stddef.h>\n#include "flexattn.h"\n'
                   'int main(){printf("%zu %zu %zu %zu %zu %zu %zu %zu\\n", sizeof(FlexScoreMod), sizeof(FlexMask),'
                   'sizeof(FlexTileLists), sizeof(FlexAttnParams), offsetof(FlexAttnParams, scale),'
                   'offsetof(FlexAttnParams, score), offsetof(FlexAttnParams, mask), offsetof(FlexAttnParams, tiles_bwd));return 0;}\n')
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
    got = [int(x) for x in subprocess.run([str(exe)], capture_output=True, text=True, check=True).stdout.split()]
    P = _lib.FlexAttnParams
    want = [ctypes.sizeof(_lib.FlexScoreMod), ctypes.sizeof(_lib.FlexMask), ctypes.sizeof(_lib.FlexTileLists),
            ctypes.sizeof(P), P.scale.offset, P.score.offset, P.mask.offset, P.tiles_bwd.offset]
    assert got == want


def test_workspace_and_tile_queries_without_gpu():
    L = _lib.lib()
    assert L.flexattn_block_mask_workspace_bytes(2, 3, 4, 5) >= 2 * 2 * 3 * 4 * 5
    qb, kvb = ctypes.c_int32(), ctypes.c_int32()
    L.flexattn_preferred_tiles(_lib.FLEX_F16, 64, 64, 2048, 2048, 0, ctypes.byref(qb), ctypes.byref(kvb))
    assert (qb.value, kvb.value) == (128, 64)
    L.flexattn_preferred_tiles(_lib.FLEX_BF16, 128, 128, 2048, 2048, 0, ctypes.byref(qb), ctypes.byref(kvb))
    assert (qb.value, kvb.value) == (128, 64)
    L.flexattn_preferred_tiles(_lib.FLEX_F16, 64, 64, 2048, 2048, 1, ctypes.byref(qb), ctypes.byref(kvb))
    assert (qb.value, kvb.value) == (128, 128)
    L.flexattn_preferred_tiles(_lib.FLEX_F32, 64, 64, 2048, 2048, 0, ctypes.byref(qb), ctypes.byref(kvb))
    assert (qb.value, kvb.value) == (128, 64)      # the fp32 matrix-core kernels walk the same lists
    L.flexattn_preferred_tiles(_lib.FLEX_BF16, 256, 256, 2048, 2048, 1, ctypes.byref(qb), ctypes.byref(kvb))
    assert (qb.value, kvb.value) == (128, 128)
    L.flexattn_preferred_tiles(_lib.FLEX_F32, 256, 256, 2048, 2048, 0, ctypes.byref(qb), ctypes.byref(kvb))
    assert (qb.value, kvb.value) == (0, 0)         # generic kernels only: lists are ignored
    # the kernel family is a pure function of the parameters
    p = _lib.FlexAttnParams()
    p.dtype, p.B, p.Hq, p.Hkv, p.Lq, p.Lkv, p.D, p.Dv = _lib.FLEX_F32, 1, 2, 2, 256, 256, 64, 64
    for name in ("q_stride", "k_stride", "v_stride", "o_stride"):
        getattr(p, name)[:] = [2 * 256 * 64, 256 * 64, 64]
    assert L.flexattn_kernel_family(p, 0) == 2 and L.flexattn_kernel_family(p, 1) == 2
    p.flags = _lib.FLAG_STRICT
    assert L.flexattn_kernel_family(p, 0) == 0
    p.flags, p.dtype = 0, _lib.FLEX_BF16
    assert L.flexattn_kernel_family(p, 0) == 1 and L.flexattn_kernel_family(p, 1) == 1
    p.D = p.Dv = 256
    assert L.flexattn_kernel_family(p, 0) == 1     # the 16-bit head sizes above 128 have matrix-core kernels too
    p.D = p.Dv = 512
    assert L.flexattn_kernel_family(p, 0) == 0
    p.dtype, p.D, p.Dv = _lib.FLEX_F32, 256, 256
    assert L.flexattn_kernel_family(p, 0) == 0
    # argument validation happens before anything touches a device
    p = _lib.FlexAttnParams()
    assert L.flexattn_fwd(p, None, None, None, None, None, None, None) != 0
    assert b"flexattn_fwd" in L.flexattn_last_error()


GRID = dict(b=torch.arange(2, dtype=torch.int32).reshape(2, 1, 1, 1), h=torch.arange(4, dtype=torch.int32).reshape(1, 4, 1, 1),
            q=torch.arange(70, dtype=torch.int32).reshape(1, 1, 70, 1), kv=torch.arange(90, dtype=torch.int32).reshape(1, 1, 1, 90))


def same_mask(a, b):
    x = torch.broadcast_to(torch.as_tensor(a(GRID["b"], GRID["h"], GRID["q"], GRID["kv"])), (2, 4, 70, 90))
    y = torch.broadcast_to(torch.as_tensor(b(GRID["b"], GRID["h"], GRID["q"], GRID["kv"])), (2, 4, 70, 90))
    return torch.equal(x.bool(), y.bool())


def test_mask_functors_match_reference_definitions():
    assert same_mask(causal_mask, o_causal_mask)                               # masks/causal.py:4-5
    assert same_mask(generate_sliding_window(10), o_sliding_window(10))        # masks/sliding_window.py:7-22
    assert same_mask(generate_attention_sink(20, 4), o_attention_sink(20, 4))  # masks/attention_sink.py:6-24
    assert same_mask(generate_attention_sink(20, 3), o_sink_window_lt(20, 4))
    assert same_mask(offset_causal_mask(30), o_offset_causal(30))
    assert same_mask(fa.noop_mask, o_noop_mask)
    assert generate_sliding_window(10).__name__ == "sliding_window_10"
    assert generate_attention_sink(32, 4).__name__ == "attention_sink_32_4"


def test_and_or_masks_fold_and_fall_back():
    m = fa.and_masks(causal_mask, generate_sliding_window(10))                 # examples/example.py:40
    assert isinstance(m, MaskMod) and (m.lo, m.hi, m.sink) == (0, 10, -1)
    sink = generate_attention_sink(1024, 4)
    assert (sink.lo, sink.hi, sink.sink) == (0, 1024, 4)
    u = fa.or_masks(causal_mask, generate_sliding_window(5))
    assert same_mask(u, o_causal_mask)

    def odd_rows(b, h, q_idx, kv_idx):
        return q_idx % 2 == 1
    mixed = fa.and_masks(causal_mask, odd_rows)
    assert not isinstance(mixed, MaskMod)
    assert same_mask(mixed, lambda b, h, q, kv: (q >= kv) & (q % 2 == 1))
    with pytest.raises(RuntimeError):
        fa.or_masks(causal_mask, "nope")
    with pytest.raises(RuntimeError):
        fa.and_masks(1, causal_mask)
    assert same_mask(fa.and_masks(), o_noop_mask)
    assert not torch.as_tensor(fa.or_masks()(0, 0, torch.arange(3), torch.arange(3))).any()


def test_band_fit_and_bit_packing():
    q, kv = torch.arange(256).reshape(-1, 1), torch.arange(384).reshape(1, -1)
    for lo, hi, sink in ((0, INT_MAX, -1), (0, 40, -1), (0, 40, 3), (-7, 9, -1), (INT_MIN, INT_MAX, -1)):
        d = q - kv
        m = (d >= lo) & ((d <= hi) | (kv <= sink))
        f = _fit_band(m)
        assert f is not None
        assert torch.equal((d >= f.lo) & ((d <= f.hi) | (kv <= f.sink)), m)
    assert _fit_band((q * 7 + kv) % 5 < 2) is None
    allf = _fit_band(torch.zeros(128, 128, dtype=torch.bool))
    assert allf.lo == INT_MAX
    m = torch.rand(2, 3, 17, 70, generator=torch.Generator().manual_seed(1)) < 0.5
    w = pack_bits(m)
    assert w.shape == (2, 3, 17, 3) and w.dtype == torch.int32
    for kvx in (0, 31, 32, 69):
        assert torch.equal(((w[..., kvx >> 5] >> (kvx & 31)) & 1).bool(), m[..., kvx])


SGRID = dict(s=torch.linspace(-3, 3, 5).reshape(5, 1, 1, 1, 1), b=torch.zeros(1, 1, 1, 1, 1, dtype=torch.int32),
             h=torch.arange(8, dtype=torch.int32).reshape(1, 1, 8, 1, 1), q=torch.arange(9, dtype=torch.int32).reshape(1, 1, 1, 9, 1),
             kv=torch.arange(11, dtype=torch.int32).reshape(1, 1, 1, 1, 11))


def same_score(a, b):
    sh = (5, 1, 8, 9, 11)
    x = torch.broadcast_to(a(SGRID["s"].expand(sh), SGRID["b"], SGRID["h"], SGRID["q"], SGRID["kv"]), sh)
    y = torch.broadcast_to(b(SGRID["s"].expand(sh), SGRID["b"], SGRID["h"], SGRID["q"], SGRID["kv"]), sh)
    return torch.allclose(x, y, rtol=1e-6, atol=1e-6)


def test_score_functors_match_reference_definitions():
    assert same_score(generate_alibi_bias(8), o_alibi(8))                       # mods/alibi.py:15-18
    assert same_score(generate_alibi_bias(8, -1.0), o_alibi_config(8))
    assert same_score(checkerboard, o_checkerboard)                             # examples/benchmark.py:16-22
    assert same_score(generate_checkerboard(2.0, 0.5, "kv"), o_checkerboard_kv)
    assert same_score(generate_tanh_softcap(50.0), o_tanh_softcap(50.0))
    assert same_score(generate_rel_bias(0.1), o_rel_bias(0.1))


def test_untagged_score_mods_are_recognised():
    def my_alibi(score, b, h, q_idx, kv_idx):
        return score + (q_idx - kv_idx) * torch.exp2(-((h + 1) * 8.0 / 8))
    s = resolve_score_mod(my_alibi, 8)
    assert (s.kind, s.p0, s.i0) == (_lib.SCORE_ALIBI, 1.0, 8)
    assert resolve_score_mod(o_checkerboard, 4).key() == (_lib.SCORE_CHECKERBOARD, 0.5, 2.0, 0)
    assert resolve_score_mod(o_checkerboard_kv, 4).key() == (_lib.SCORE_CHECKERBOARD, 2.0, 0.5, 1)
    c = resolve_score_mod(o_tanh_softcap(30.0), 4)
    assert c.kind == _lib.SCORE_TANH_SOFTCAP and abs(c.p0 - 30.0) < 1e-4
    r = resolve_score_mod(o_rel_bias(-0.25), 4)
    assert r.kind == _lib.SCORE_REL_BIAS and abs(r.p0 + 0.25) < 1e-6
    assert resolve_score_mod(lambda s, b, h, q, kv: s, 4).kind == _lib.SCORE_IDENTITY
    assert resolve_score_mod(None, 4).kind == _lib.SCORE_IDENTITY
    assert _probe_score_mod(lambda s, b, h, q, kv: s * s, 4) is None
    # mods that equal a family near the origin only: the family must not be accepted for them
    far = lambda s, b, h, q, kv: torch.where((q - kv).abs() > 64, s - 10.0, s)          # noqa: E731
    late_batch = lambda s, b, h, q, kv: torch.where(b >= 2, s * 0.5, s)                  # noqa: E731
    segments = lambda s, b, h, q, kv: s + ((q // 16) != (kv // 16)) * -5.0               # noqa: E731
    for fn in (far, late_batch, segments):
        assert _probe_score_mod(fn, 4, (4, 4, 256, 256)) is None, fn
        assert _probe_score_mod(fn, 4) is None, fn
    # ... while on a problem that never leaves the region where they agree, the family is the right lowering
    assert _probe_score_mod(late_batch, 4, (2, 4, 64, 64)).kind == _lib.SCORE_IDENTITY
    assert _probe_score_mod(far, 4, (1, 4, 32, 32)).kind == _lib.SCORE_IDENTITY
    with pytest.raises(NotImplementedError):
        resolve_score_mod(lambda s, b, h, q, kv: torch.sin(s), 4)


def test_mod_type_by_arity():
    assert _get_mod_type(lambda b, h, q, kv: True) == _ModificationType.MASK_MOD
    assert _get_mod_type(lambda s, b, h, q, kv: s) == _ModificationType.SCORE_MOD
    assert _get_mod_type(causal_mask) == _ModificationType.MASK_MOD
    assert _get_mod_type(checkerboard) == _ModificationType.SCORE_MOD
    with pytest.raises(AssertionError):
        _get_mod_type(lambda a, b: a)


def test_front_end_validation_raises_reference_errors():
    q, k, v = torch.zeros(1, 4, 8, 16), torch.zeros(1, 2, 8, 16), torch.zeros(1, 2, 8, 16)
    with pytest.raises(ValueError, match="same number of heads"):
        fa.flax_attention(q, k, v)
    with pytest.raises(ValueError, match="same dtype"):
        fa.flax_attention(q, k.half(), v)
    with pytest.raises(NotImplementedError, match="4D"):
        fa.flax_attention(q[0], k[0], v[0], enable_gqa=True)
    with pytest.raises(ValueError, match="embedding dimension"):
        fa.flax_attention(q, k[..., :8], v, enable_gqa=True)
    with pytest.raises(ValueError, match="value embedding dimension"):
        fa.flax_attention(q, k, torch.zeros(1, 2, 8, 32), enable_gqa=True)
    with pytest.raises(ValueError, match="multiple of kv heads"):
        fa.flax_attention(torch.zeros(1, 3, 8, 16), k, v, enable_gqa=True)
    with pytest.raises(ValueError, match="same number of heads"):
        fa.flax_attention_pallas(q, k, v)
    # valid arguments on the CPU: there is no fallback, the call must fail loudly
    with pytest.raises(fa.FlexAttnError, match="no CPU fallback"):
        fa.flax_attention(q, k, v, enable_gqa=True)
    with pytest.raises(ValueError, match="only one of"):
        fa.flax_attention_pallas(q, k, v, mask_mod=causal_mask, block_mod=causal_mask, enable_gqa=True)


def test_product_never_imports_the_oracle():
    code = "import sys; import flaxattention_amd, flaxattention_amd.masks, flaxattention_amd.mods; " \
           "assert not any(m == 'oracle' or m.startswith('oracle.') for m in sys.modules), 'oracle imported'"
    subprocess.run([sys.executable, "-c", code], check=True, cwd=ROOT)
    for dirpath, _, files in os.walk(os.path.join(ROOT, "flaxattention_amd")):
        for f in files:
            if f.endswith((".py", ".hip", ".cuh")):
                text = open(os.path.join(dirpath, f)).read()
                assert "import oracle" not in text and "from oracle" not in text, f


def test_affine_score_mod_lowering_on_cpu():
    """A callable that is affine in the score becomes dense tables; one that is not is refused."""
    import torch
    from flaxattention_amd.core.common import affine_score_mod
    table = torch.randn(3, 9, generator=torch.Generator().manual_seed(1))

    def rel_table(score, b, h, q_idx, kv_idx):
        return score + table[h.long(), (q_idx - kv_idx).clamp(-4, 4).long() + 4]

    def scaled(score, b, h, q_idx, kv_idx):
        return torch.where(q_idx >= kv_idx, score * 0.5, score * 2.0) - 1.5 * b

    # a bias that depends on kv - q only is kept per diagonal: entry (kv - q) + Lq - 1, reached with stride_q = -1
    s = affine_score_mod(rel_table, 2, 3, 6, 7, "cpu")
    assert s.kind == _lib.SCORE_AFFINE and s.mul is None and tuple(s.add.shape) == (1, 3, 12) and s.diag_zero == 5
    c = s.c_struct()
    assert (c.stride_b, c.stride_h, c.stride_q) == (0, 12, -1) and c.mul is None and c.add == s.add.data_ptr() + 4 * 5
    q, kv = torch.arange(6).reshape(6, 1), torch.arange(7).reshape(1, 7)
    assert torch.equal(s.add[0, 2][(kv - q) + 5], table[2][(q - kv).clamp(-4, 4) + 4])

    def per_row(score, b, h, q_idx, kv_idx):   # depends on q and kv separately: stays a dense [.., Lq, Lkv] table
        return score + table[h.long(), (q_idx % 3 + kv_idx % 4).long()]
    s = affine_score_mod(per_row, 2, 3, 6, 7, "cpu")
    assert tuple(s.add.shape) == (1, 3, 6, 7) and s.diag_zero is None
    c = s.c_struct()
    assert (c.stride_b, c.stride_h, c.stride_q) == (0, 42, 7) and c.add == s.add.data_ptr()
    assert torch.equal(s.add[0, 2], table[2][(q % 3 + kv % 4)])
    s = affine_score_mod(scaled, 2, 3, 6, 7, "cpu")
    assert tuple(s.mul.shape) == (2, 1, 6, 7) and torch.equal(s.mul[1, 0], torch.where(q >= kv, 0.5, 2.0))
    assert torch.equal(s.add[1, 0], torch.full((6, 7), -1.5))
    assert affine_score_mod(lambda sc, b, h, q_, k_: sc * sc, 1, 1, 4, 4, "cpu") is None
    assert affine_score_mod(lambda sc, b, h, q_, k_: sc + 0.0 * q_, 1, 1, 4, 4, "cpu").kind == _lib.SCORE_IDENTITY


def test_affine_lowering_checks_the_full_index_range():
    """A score_mod that is affine in the score near the origin of the index space and something else beyond it
    must not be lowered to tables (the reference applies the callable to every element,
    flaxattention/core/attention.py:59-63): the resolver has to refuse it, which hands the call to the
    linearised path."""
    import torch
    from flaxattention_amd.core.common import ScoreModNotLowered, affine_score_mod, resolve_score_mod

    def cap_past_sinks(s, b, h, q, kv):     # identity on the first keys, tanh beyond them
        return torch.where(kv > 100, torch.tanh(s), s)

    def square_for_late_batches(s, b, h, q, kv):
        return torch.where(b >= 2, s * s, s)

    def sine_for_late_rows(s, b, h, q, kv):
        return torch.where(q >= 64, 3 * torch.sin(s), 2 * s)

    cases = [(cap_past_sinks, (1, 2, 256, 256)), (square_for_late_batches, (3, 2, 16, 16)),
             (sine_for_late_rows, (1, 1, 128, 32))]
    for fn, shape in cases:
        assert affine_score_mod(fn, *shape, "cpu") is None, fn.__name__
        with pytest.raises(ScoreModNotLowered):
            resolve_score_mod(fn, shape[1], shape, "cpu")

    # the same shapes of callable with an affine far part are still lowered, and the tables carry the far part
    def scale_past_sinks(s, b, h, q, kv):
        return torch.where(kv > 100, 0.25 * s - 1.0, s)
    spec = affine_score_mod(scale_past_sinks, 1, 2, 256, 256, "cpu")
    assert spec is not None and spec.kind == _lib.SCORE_AFFINE
    assert float(spec.mul[0, 0, 0, 200]) == 0.25 and float(spec.mul[0, 0, 0, 50]) == 1.0
    assert float(spec.add[0, 0, 0, 200]) == -1.0 and float(spec.add[0, 0, 0, 50]) == 0.0


def test_lowering_cache_serves_closures_made_anew():
    """A score_mod written as a lambda inside the training step is a new function object on every call; its lowering
    is found again through its code object and what it captures (numbers by value, tensors by identity and version),
    and is made anew when any of that changes."""
    import torch
    from flaxattention_amd.core import common
    calls = []
    orig = common._probe_score_mod

    def counting(*a, **k):
        calls.append(1)
        return orig(*a, **k)
    common._probe_score_mod = counting
    try:
        def make(f):
            return lambda s, b, h, q, kv: torch.where((kv - q) % 2 == 0, s * f, s * 0.5)
        shape = (1, 4, 64, 64)
        a = common.resolve_score_mod(make(2.0), 4, shape, "cpu")
        b = common.resolve_score_mod(make(2.0), 4, shape, "cpu")
        assert a is b and len(calls) == 1 and a.kind == _lib.SCORE_CHECKERBOARD and a.p0 == 2.0
        c = common.resolve_score_mod(make(3.0), 4, shape, "cpu")          # another captured number: another lowering
        assert c is not a and c.p0 == 3.0 and len(calls) == 2
        assert common.resolve_score_mod(make(2.0), 4, shape, "cpu") is a  # both stay cached side by side
        bias = torch.zeros(4)

        def with_table():
            return lambda s, b, h, q, kv: s + bias[h.long()]
        t1 = common.resolve_score_mod(with_table(), 4, shape, "cpu")
        n = len(calls)
        assert common.resolve_score_mod(with_table(), 4, shape, "cpu") is t1 and len(calls) == n
        bias.add_(1.0)                                                    # in-place update: read again
        t2 = common.resolve_score_mod(with_table(), 4, shape, "cpu")
        assert t2 is not t1 and float(t2.add.reshape(-1)[0]) == 1.0
    finally:
        common._probe_score_mod = orig


def test_utils_score_matrix_and_picture(tmp_path):
    """flaxattention/utils.py:17-49, 58-139: dense post-mod scores / mask of one (batch, head) and its picture."""
    from flaxattention_amd.utils import _name_to_title, create_score_mod, visualize_attention_scores
    from flaxattention_amd.masks import causal_mask
    from flaxattention_amd.mods import generate_alibi_bias
    g = torch.Generator().manual_seed(3)
    q, k = torch.randn(2, 4, 6, 8, generator=g), torch.randn(2, 4, 9, 8, generator=g)
    alibi = generate_alibi_bias(4)
    got = create_score_mod(q[1, 2], k[1, 2], alibi, None, batch_idx=1, head_idx=2)
    assert got.shape == (1, 1, 6, 9)
    qi, ki = torch.arange(6).view(6, 1), torch.arange(9).view(1, 9)
    want = (q[1, 2] @ k[1, 2].T) / 8 ** 0.5 + (qi - ki) * 2.0 ** (-(2 + 1) * 8.0 / 4)   # mods/alibi.py:15-18
    assert torch.allclose(got[0, 0], want, atol=1e-6)
    m = create_score_mod(q[0, 0], k[0, 0], None, causal_mask)
    assert m.dtype == torch.bool and torch.equal(m[0, 0], qi >= ki)
    assert _name_to_title("causal_mask_demo") == "Causal Mask Demo"
    visualize_attention_scores(q, k, mask_mod=causal_mask, name="m", path=tmp_path / "mask_picture", head_idx=1)
    assert (tmp_path / "mask_picture.png").stat().st_size > 1000
    with pytest.raises(AssertionError):
        visualize_attention_scores(q, k)


def test_mask_with_captured_buffer_is_not_indexed_past_the_end():
    """The builder's padded index range (blockmask.py:440-444) must not reach a captured tensor: positions past
    the real lengths are evaluated with clamped indices unless the mod provably computes from its index
    arguments alone; such arithmetic mods still see them as if they were real."""
    import functools
    from flaxattention_amd.core.common import _index_arithmetic_only, dense_mask_on_device
    from flaxattention_amd.masks import causal_mask, generate_sliding_window
    table = torch.zeros(4)
    assert _index_arithmetic_only(lambda b, h, q, kv: (q >= kv) & (q - kv < 7))
    assert _index_arithmetic_only(causal_mask) and _index_arithmetic_only(generate_sliding_window(5))
    assert _index_arithmetic_only(fa.and_masks(causal_mask, lambda b, h, q, kv: kv % 2 == 0))
    assert not _index_arithmetic_only(lambda b, h, q, kv: table[q.long()] > 0)
    assert not _index_arithmetic_only(functools.partial(lambda b, h, q, kv, t: t[q.long()] > 0, t=table))
    assert not _index_arithmetic_only(fa.and_masks(causal_mask, lambda b, h, q, kv: table[kv.long()] > 0))
    doc = torch.arange(96) // 20

    def doc_mask(b, h, q_idx, kv_idx):
        return doc[q_idx.long()] == doc[kv_idx.long()]
    m = dense_mask_on_device(doc_mask, 1, 1, 128, 128, torch.device("cpu"), real=(96, 96))
    assert m.shape == (1, 1, 128, 128)
    qi, ki = torch.arange(128).clamp(max=95).view(128, 1), torch.arange(128).clamp(max=95).view(1, 128)
    assert torch.equal(m[0, 0], doc[qi] == doc[ki])
    causal = dense_mask_on_device(lambda b, h, q, kv: q >= kv, 1, 1, 128, 256, torch.device("cpu"), real=(100, 130))
    assert torch.equal(causal[0, 0], torch.arange(128).view(128, 1) >= torch.arange(256).view(1, 256))


def test_cached_lowerings_follow_captured_tensors():
    """A lowering of a score_mod is reused only while the tensors the callable captures are unchanged."""
    from flaxattention_amd.core.common import _capture_stamp, _stamp_valid
    table = torch.zeros(4)
    fn = lambda s, b, h, q, kv: s + table[h.long()]   # noqa: E731
    stamp = _capture_stamp(fn)
    assert stamp is not None and len(stamp) == 2 and stamp[0][0] is table and _stamp_valid(stamp, _capture_stamp(fn))
    table.add_(1.0)
    assert not _stamp_valid(stamp, _capture_stamp(fn))
    assert _capture_stamp(lambda s, b, h, q, kv: s * 2.0) == [(None, ())]
    window = 3
    band = lambda b, h, q, kv: q - kv <= window   # noqa: E731
    stamp = _capture_stamp(band)
    assert stamp == [(None, (3,))] and _stamp_valid(stamp, _capture_stamp(band))
    window = 5                                    # a rebound closure variable is a different callable in effect
    assert not _stamp_valid(stamp, _capture_stamp(band))
    other = torch.zeros(4)
    fn2 = lambda s, b, h, q, kv: s + other[h.long()]   # noqa: E731
    stamp = _capture_stamp(fn2)
    other = torch.ones(4)                         # rebound to another tensor
    assert not _stamp_valid(stamp, _capture_stamp(fn2))

    class Holder:
        t = torch.ones(2)
    holder = Holder()
    assert _capture_stamp(lambda s, b, h, q, kv: s + holder.t[0]) is None   # state that cannot be seen: never cached


def test_bench_refuses_more_than_one_gpu():
    """The benchmark measures one GPU; asking for more ends with a message instead of a number."""
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=300)
    assert r.returncode != 0 and "one GPU" in r.stderr and r.stdout.strip() == ""


def test_bench_traffic_figures_do_not_outlive_the_kernels():
    """The HBM-traffic figures in bench.py are copied from hardware-counter runs; they are reported only while the
    kernel sources are the ones they were measured for (a hash), and read null after any change to them."""
    import importlib.util
    spec = importlib.util.spec_from_file_location("bench_for_test", os.path.join(ROOT, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    old = bench.TRAFFIC_KERNEL_SHA
    try:
        bench.TRAFFIC_KERNEL_SHA = bench.kernel_sources_sha()      # as right after a counter run
        assert bench.measured_traffic("config2", "bwd_dkv_kernel") == bench.MEASURED_TRAFFIC_BYTES[("config2", "bwd_dkv_kernel")]
        assert bench.measured_traffic("config2", "no_such_kernel") is None
        bench.TRAFFIC_KERNEL_SHA = "0" * 16                         # as after an edit of the kernels
        assert bench.measured_traffic("config2", "bwd_dkv_kernel") is None
    finally:
        bench.TRAFFIC_KERNEL_SHA = old


def test_block_classes_of_a_bitmap():
    """The table the fused kernels consult inside partial tiles: 1 = block entirely visible, 2 = entirely hidden."""
    from flaxattention_amd.core.common import block_classes
    g = torch.Generator().manual_seed(3)
    m = torch.rand(2, 1, 96, 128, generator=g) < 0.5
    m[0, 0, 32:64, 64:96] = True
    m[1, 0, 0:32, 0:32] = False
    m[1, 0, 64:96, 96:128] = True
    m[1, 0, 95, 127] = False      # one hidden entry: mixed
    cls = block_classes(m)
    assert cls.shape == (2, 1, 3, 4) and cls.dtype == torch.int8
    for b in range(2):
        for i in range(3):
            for j in range(4):
                blk = m[b, 0, 32 * i:32 * i + 32, 32 * j:32 * j + 32]
                want = 1 if bool(blk.all()) else (2 if not bool(blk.any()) else 0)
                assert int(cls[b, 0, i, j]) == want
    assert int(cls[0, 0, 1, 2]) == 1 and int(cls[1, 0, 0, 0]) == 2 and int(cls[1, 0, 2, 3]) == 0
