"""Mod plumbing: signatures, arity-based classification and the functor objects
that the HIP kernels understand.

Mirrors flaxattention/core/common.py:7-39 (type aliases, _ModificationType,
_get_mod_type).  The reference maps a *scalar* Python function over
(b, h, q_idx, kv_idx) with four nested vmaps (common.py:41-80); here a mod is
lowered to a small POD functor (FlexScoreMod / FlexMask in include/flexattn.h)
that is evaluated inside the kernels.  The functor objects below are also plain
callables with the reference's scalar signature, so user code that calls or
combines them keeps working; they broadcast over torch tensors, numpy arrays
and Python ints alike.
"""
from __future__ import annotations

import inspect
import math
from enum import Enum
from typing import Any, Callable, Optional, Tuple

import torch

from .. import _lib

Array = torch.Tensor
_score_mod_signature = Callable[[Array, Array, Array, Array, Array], Array]
_mask_mod_signature = Callable[[Array, Array, Array, Array], Array]

INT_MIN, INT_MAX = _lib.INT_MIN, _lib.INT_MAX


class _ModificationType(Enum):
    """common.py:10-19."""
    SCORE_MOD = 1
    MASK_MOD = 2
    UNKNOWN = 3


def _get_mod_type(fn: Callable) -> _ModificationType:
    """common.py:21-39: five positional arguments -> score_mod, four -> mask_mod."""
    if isinstance(fn, ScoreMod):
        return _ModificationType.SCORE_MOD
    if isinstance(fn, MaskMod):
        return _ModificationType.MASK_MOD
    num_positional_args = sum(
        1 for param in inspect.signature(fn).parameters.values()
        if param.default == inspect.Parameter.empty
    )
    assert num_positional_args == 5 or num_positional_args == 4
    if num_positional_args == 5:
        return _ModificationType.SCORE_MOD
    elif num_positional_args == 4:
        return _ModificationType.MASK_MOD
    return _ModificationType.UNKNOWN


# ---------------------------------------------------------------------------
# score_mod functors
# ---------------------------------------------------------------------------
def _f32(x):
    if torch.is_tensor(x):
        return x.to(torch.float32)
    return x


class ScoreMod:
    """A score_mod the fused kernels evaluate in registers.

    kind/p0/p1/i0 are the fields of FlexScoreMod.  Calling the object applies
    the same scalar function to its arguments."""

    def __init__(self, kind: int, p0: float = 0.0, p1: float = 0.0, i0: int = 0, name: str = "score_mod",
                 mul: Optional[torch.Tensor] = None, add: Optional[torch.Tensor] = None, fn: Optional[Callable] = None):
        self.kind, self.p0, self.p1, self.i0 = int(kind), float(p0), float(p1), int(i0)
        self.__name__ = name
        # SCORE_AFFINE: dense fp32 tables [b', h', q', Lkv] (each leading extent 1 or full) and the
        # callable they were read from.  An additive table whose diagonals are constant (a bias that depends
        # on kv_idx - q_idx only) is kept as [b', h', Lq + Lkv - 1] instead, entry (kv - q) + diag_zero: the
        # kernels' address  add + q * stride_q + kv  reaches it with stride_q = -1 from add + diag_zero.
        self.mul, self.add, self.fn = mul, add, fn
        self.diag_zero: Optional[int] = None

    def c_struct(self) -> _lib.FlexScoreMod:
        m = _lib.FlexScoreMod(self.kind, self.p0, self.p1, self.i0, 0)
        t = self.mul if self.mul is not None else self.add
        if t is not None and self.diag_zero is not None:
            m.add = self.add.data_ptr() + 4 * self.diag_zero
            m.stride_b, m.stride_h = (t.stride(i) if t.shape[i] > 1 else 0 for i in range(2))
            m.stride_q = -1
        elif t is not None:
            m.mul = self.mul.data_ptr() if self.mul is not None else None
            m.add = self.add.data_ptr() if self.add is not None else None
            m.stride_b, m.stride_h, m.stride_q = (t.stride(i) if t.shape[i] > 1 else 0 for i in range(3))
        return m

    def key(self):
        if self.kind == _lib.SCORE_AFFINE:
            return (self.kind, id(self.mul), id(self.add))
        return (self.kind, self.p0, self.p1, self.i0)

    def __call__(self, score, b, h, q_idx, kv_idx):
        k = self.kind
        if k == _lib.SCORE_IDENTITY:
            return score
        if k == _lib.SCORE_CHECKERBOARD:
            par = ((kv_idx - q_idx) if self.i0 == 0 else (kv_idx + 0 * q_idx)) % 2
            if torch.is_tensor(par):
                return torch.where(par == 0, score * self.p0, score * self.p1)
            return score * (self.p0 if par == 0 else self.p1)
        if k == _lib.SCORE_ALIBI:
            slope = 2.0 ** (-((_f32(h) + 1) * 8.0 / self.i0))
            return score + _f32(q_idx - kv_idx) * slope * self.p0
        if k == _lib.SCORE_TANH_SOFTCAP:
            if torch.is_tensor(score):
                return self.p0 * torch.tanh(score / self.p0)
            return self.p0 * math.tanh(score / self.p0)
        if k == _lib.SCORE_REL_BIAS:
            return score + _f32(kv_idx - q_idx) * self.p0
        if k == _lib.SCORE_AFFINE:
            return self.fn(score, b, h, q_idx, kv_idx)
        raise ValueError(f"unknown score_mod kind {k}")

    def __repr__(self):
        return f"ScoreMod({self.__name__}, kind={self.kind}, p0={self.p0}, p1={self.p1}, i0={self.i0})"


def _identity(score, batch, head, token_q, token_kv):
    """flaxattention/core/attention.py:109-116."""
    return score


IDENTITY = ScoreMod(_lib.SCORE_IDENTITY, name="identity")


def _probe_score_mod(fn: Callable, H: int, shape: Optional[Tuple[int, int, int, int]] = None,
                     device=None) -> Optional[ScoreMod]:
    """Recognise an untagged Python score_mod as one of the functor families by
    evaluating it on a small grid and checking every family exactly.  A callable that may look
    positions up in captured tensors is only probed inside the real index ranges of `shape`
    (an out-of-range index into a device tensor stops the process), and on the device when it
    cannot take CPU tensors."""
    Pq, Pkv, nb = 7, 9, 2
    Hn = max(int(H), 1)
    shape_in = shape
    if not _index_arithmetic_only(fn):
        if shape is None:
            return None
        nb, Pq, Pkv = min(nb, shape[0]), min(Pq, shape[2]), min(Pkv, shape[3])
    s = torch.tensor([-1.75, -0.5, 0.0, 0.625, 2.5], dtype=torch.float32).reshape(5, 1, 1, 1, 1)
    b = torch.arange(nb, dtype=torch.int32).reshape(1, nb, 1, 1, 1)
    h = torch.arange(Hn, dtype=torch.int32).reshape(1, 1, Hn, 1, 1)
    q = torch.arange(Pq, dtype=torch.int32).reshape(1, 1, 1, Pq, 1)
    kv = torch.arange(Pkv, dtype=torch.int32).reshape(1, 1, 1, 1, Pkv)
    shape5 = (5, nb, Hn, Pq, Pkv)
    out = None
    for where in ("cpu",) + ((device,) if device is not None else ()):
        try:
            res = fn(s.to(where).expand(shape5), b.to(where), h.to(where), q.to(where), kv.to(where))
            if not torch.is_tensor(res):
                return None
            out = torch.broadcast_to(res.to(torch.float32), shape5).cpu()
            s, b, h, q, kv = (t.to(where) for t in (s, b, h, q, kv))
            break
        except Exception:
            continue
    if out is None or Pkv < 2:
        return None
    shape = shape5

    def same(c: ScoreMod) -> bool:
        ref = torch.broadcast_to(_f32(c(s.expand(shape), b, h, q, kv)), shape).cpu()
        return bool(torch.allclose(out, ref, rtol=1e-6, atol=1e-6))

    cands = [IDENTITY]
    # multiplicative checkerboards: read both factors off two grid points
    with torch.no_grad():
        one = out[4] / 2.5  # score 2.5
        for i0 in (0, 1):
            f_even = one[0, 0, 0, 0].item()
            f_odd = one[0, 0, 0, 1].item()
            cands.append(ScoreMod(_lib.SCORE_CHECKERBOARD, f_even, f_odd, i0, name=getattr(fn, "__name__", "checkerboard")))
        bias = out[2]  # score 0
        for sign in (1.0, -1.0):
            cands.append(ScoreMod(_lib.SCORE_ALIBI, sign, 0.0, Hn, name=getattr(fn, "__name__", "alibi")))
        cands.append(ScoreMod(_lib.SCORE_REL_BIAS, bias[0, 0, 0, 1].item(), name=getattr(fn, "__name__", "rel_bias")))
        # tanh soft-cap: cap from the saturated value
        try:
            big = fn(torch.full((1, 1, 1, 1, 1), 1e9, device=s.device), b[:, :1], h[:, :, :1], q[..., :1, :], kv[..., :1])
            cap = float(torch.as_tensor(big).reshape(-1)[0])
            if math.isfinite(cap) and cap > 0:
                cands.append(ScoreMod(_lib.SCORE_TANH_SOFTCAP, cap, 1.0 / cap, name=getattr(fn, "__name__", "tanh_softcap")))
        except Exception:
            pass
    for c in cands:
        if same(c):
            # the corner grid only nominates a family; it is accepted when it reproduces the callable on every
            # position of the problem (a mod that differs from the family only far from the origin, for some
            # batch index or past the first few keys must not be lowered to it)
            full = shape_in if shape_in is not None else (4, Hn, 300, 300)
            where = device if (shape_in is not None and device is not None) else "cpu"
            return c if _same_on_full_range(fn, c, full, where) else None
    return None


def _same_on_full_range(fn: Callable, cand: "ScoreMod", shape: Tuple[int, int, int, int], where,
                        max_elems: int = 1 << 25) -> bool:
    """fn == cand on every (b, h, q_idx, kv_idx) of `shape`, at three score values (the corner grid has
    already pinned how a family depends on the score).  Evaluated in slabs of query rows of at most
    `max_elems` entries; a callable that broadcasts is only evaluated over the axes it really uses."""
    B, H, Lq, Lkv = shape
    b = torch.arange(B, dtype=torch.int32, device=where).reshape(B, 1, 1, 1)
    h = torch.arange(H, dtype=torch.int32, device=where).reshape(1, H, 1, 1)
    kv = torch.arange(Lkv, dtype=torch.int32, device=where).reshape(1, 1, 1, Lkv)
    rows = max(1, min(Lq, max_elems // max(1, B * H * Lkv)))
    try:
        for score in (-1.75, 0.625, 2.5):
            sc = torch.full((1, 1, 1, 1), score, dtype=torch.float32, device=where)
            for q0 in range(0, Lq, rows):
                q = torch.arange(q0, min(q0 + rows, Lq), dtype=torch.int32, device=where).reshape(1, 1, -1, 1)
                got = torch.as_tensor(fn(sc, b, h, q, kv)).to(torch.float32)
                want = _f32(cand(sc, b, h, q, kv))
                if not bool(torch.allclose(got, want.to(got.device), rtol=1e-5, atol=1e-5)):
                    return False
    except Exception:
        return False
    return True


def affine_score_mod(fn: Callable, B: int, H: int, Lq: int, Lkv: int, device) -> Optional[ScoreMod]:
    """Lower a score_mod that is affine in the score, mod(s) = mul[b,h,q,kv] * s + add[b,h,q,kv], to dense
    fp32 tables read off the callable on the device (what attention.py:59-63 evaluates per element;
    captured tensors such as bias tables, attention.py:22-23, are simply part of the callable).
    Returns None when the callable is not affine in the score."""
    # affinity, on a small CPU grid: five score values must lie on one line per (b, h, q, kv)
    P = 5
    s = torch.tensor([-1.75, -0.5, 0.0, 0.625, 2.5], dtype=torch.float32).reshape(5, 1, 1, 1, 1)
    b = torch.arange(min(B, 2), dtype=torch.int32).reshape(1, -1, 1, 1, 1)
    h = torch.arange(H, dtype=torch.int32).reshape(1, 1, H, 1, 1)
    q = torch.arange(min(Lq, P), dtype=torch.int32).reshape(1, 1, 1, -1, 1)
    kv = torch.arange(min(Lkv, P + 2), dtype=torch.int32).reshape(1, 1, 1, 1, -1)
    shape = (5, b.numel(), H, q.numel(), kv.numel())
    out = None
    for where in ("cpu", device):   # a callable that indexes tensors living on the device cannot take CPU indices
        try:
            sw, bw, hw, qw, kw = (t.to(where) for t in (s, b, h, q, kv))
            out = torch.broadcast_to(torch.as_tensor(fn(sw.expand(shape), bw, hw, qw, kw)).to(torch.float32), shape).cpu()
            break
        except Exception:
            continue
    if out is None:
        return None
    a0, c0 = (out[4] - out[2]) / 2.5, out[2]
    if not torch.isfinite(out).all() or not torch.allclose(out, a0 * s + c0, rtol=1e-5, atol=1e-5):
        return None
    # the tables, on the device; a [1,1,1,1] score keeps every extent the callable does not use at 1
    bi = torch.arange(B, dtype=torch.int32, device=device).reshape(B, 1, 1, 1)
    hi = torch.arange(H, dtype=torch.int32, device=device).reshape(1, H, 1, 1)
    qi = torch.arange(Lq, dtype=torch.int32, device=device).reshape(1, 1, Lq, 1)
    ki = torch.arange(Lkv, dtype=torch.int32, device=device).reshape(1, 1, 1, Lkv)
    zero = torch.zeros((1, 1, 1, 1), dtype=torch.float32, device=device)
    add = torch.as_tensor(fn(zero, bi, hi, qi, ki)).to(torch.float32)
    # slope from a wide symmetric difference: the additive part cancels with little rounding left
    mul = (torch.as_tensor(fn(zero + 8.0, bi, hi, qi, ki)).to(torch.float32)
           - torch.as_tensor(fn(zero - 8.0, bi, hi, qi, ki)).to(torch.float32)) / 16.0
    while add.dim() < 4:
        add = add.unsqueeze(0)
    while mul.dim() < 4:
        mul = mul.unsqueeze(0)
    if not (bool(torch.isfinite(add).all()) and bool(torch.isfinite(mul).all())):
        return None
    # The corner grid only says that the callable is affine near the origin of the index space.  The tables are
    # accepted when they reproduce the callable at further scores on EVERY (b, h, q_idx, kv_idx) of the problem: a mod
    # that is affine for the first keys, rows or batch entries and something else beyond them (a soft-cap past a few
    # sink keys, a square for some batch index) must not be lowered to tables.  Row slabs bound the temporaries.
    rows = max(1, min(Lq, _SLAB_ELEMS // max(1, B * H * Lkv)))
    for q0 in range(0, Lq, rows):
        qs = qi[:, :, q0:q0 + rows]
        a_s = add[:, :, q0:q0 + rows] if add.shape[2] == Lq else add
        m_s = mul[:, :, q0:q0 + rows] if mul.shape[2] == Lq else mul
        for s_chk in (0.625, -1.75, 3.25):
            got = torch.as_tensor(fn(zero + s_chk, bi, hi, qs, ki)).to(torch.float32)
            while got.dim() < 4:
                got = got.unsqueeze(0)
            if not bool(torch.allclose(got, m_s * s_chk + a_s, rtol=1e-5, atol=1e-5)):
                return None
    full = (B, H, Lq, Lkv)
    shp = tuple(max(add.shape[i], mul.shape[i]) for i in range(3)) + (Lkv,)
    if any(shp[i] not in (1, full[i]) for i in range(3)):
        return None
    add = None if not bool(add.any()) else torch.broadcast_to(add, shp).contiguous()
    mul = None if bool(((mul - 1).abs() <= 1e-6).all()) else torch.broadcast_to(mul, shp).contiguous()
    if add is None and mul is None:
        return IDENTITY
    spec = ScoreMod(_lib.SCORE_AFFINE, name=getattr(fn, "__name__", "affine_score_mod"), mul=mul, add=add, fn=fn)
    if (mul is None and add.shape[2] == Lq and Lq > 1 and Lkv > 1
            and bool(torch.equal(add[:, :, 1:, 1:], add[:, :, :-1, :-1]))):
        # constant along every diagonal: first column upwards (kv - q = -(Lq-1) .. 0), then first row (1 .. Lkv-1)
        spec.add = torch.cat([add[:, :, :, 0].flip(-1), add[:, :, 0, 1:]], dim=-1).contiguous()
        spec.diag_zero = Lq - 1
    return spec


_score_cache: dict = {}


class ScoreModNotLowered(NotImplementedError):
    """resolve_score_mod: the callable is not one of the functor families and not affine in the score."""


def resolve_score_mod(fn: Optional[Callable], H: int, shape: Optional[Tuple[int, int, int, int]] = None,
                      device=None) -> ScoreMod:
    """Lower a score_mod callable to a kernel functor, or raise.  `shape` = (B, H, Lq, Lkv) and `device`
    allow the dense affine form for callables outside the functor families."""
    if fn is None or fn is _identity:
        return IDENTITY
    if isinstance(fn, ScoreMod):
        return fn
    # a lowering is cached only together with what it was derived from: the callable and the captured tensors
    # at their current versions (a learned bias that the optimizer has updated in place must be read again)
    stamp = _capture_stamp(fn)
    who = _callable_key(fn, stamp)
    key = (who, H, None if shape is None else tuple(shape), str(device))   # a family is verified per problem shape
    hit = _score_cache.get(key)
    if hit is not None and not (_same_callable(hit[0], fn) and stamp is not None and _stamp_valid(hit[2], stamp)):
        hit = None
    if hit is not None and hit[1] is not None:
        return hit[1]
    if hit is None:   # (a cached None says: probed before, not one of the families)
        spec = _probe_score_mod(fn, H, shape, device)
        if stamp is not None:
            if len(_score_cache) > 64:
                _score_cache.clear()
            _score_cache[key] = (fn, spec, stamp)
        if spec is not None:
            return spec
    if shape is not None and device is not None:
        key = ("affine", who) + tuple(shape) + (str(device),)
        hit = _score_cache.get(key)
        if hit is not None and _same_callable(hit[0], fn) and stamp is not None and _stamp_valid(hit[2], stamp):
            return hit[1]
        spec = affine_score_mod(fn, *shape, device)
        if spec is not None:
            if len(_score_cache) > 64:
                _score_cache.clear()
            if stamp is not None:
                _score_cache[key] = (fn, spec, stamp)
            return spec
    raise ScoreModNotLowered(
        "score_mod is neither one of the fused functor families (identity, checkerboard, ALiBi, tanh soft-cap, "
        "relative-position bias) nor affine in the score (mul[b,h,q,kv] * score + add[b,h,q,kv]): it cannot be lowered "
        "to a functor that is independent of the scores (the front-ends then linearise it at the scores of each call)")


# ---------------------------------------------------------------------------
# mask_mod functors
# ---------------------------------------------------------------------------
class MaskMod:
    """A mask_mod the kernels evaluate: either the canonical band form

        d = q_idx + q_offset - kv_idx
        visible = (d >= lo) and (d <= hi or kv_idx <= sink)

    or a packed bitmap made from an arbitrary callable (kind BITS)."""

    def __init__(self, lo: int = INT_MIN, hi: int = INT_MAX, sink: int = -1, q_offset: int = 0,
                 name: str = "mask_mod", bits: Optional[torch.Tensor] = None, fn: Optional[Callable] = None,
                 bits_t: Optional[torch.Tensor] = None, blk: Optional[torch.Tensor] = None):
        self.lo, self.hi, self.sink, self.q_offset = int(lo), int(hi), int(sink), int(q_offset)
        self.bits = bits      # int32 [Bm, Hm, Qp, KVw] on the device, or None
        self.bits_t = bits_t  # the same bitmap packed along the query axis, int32 [Bm, Hm, KVp, Qw], or None
        self.blk = blk        # class of every aligned 32 x 32 block, int8 [Bm, Hm, Qp/32, KVp/32], or None
        self.fn = fn          # the callable a bitmap was made from
        self.__name__ = name

    @property
    def kind(self) -> int:
        return _lib.MASK_BITS if self.bits is not None else _lib.MASK_BAND

    def is_noop(self) -> bool:
        return self.bits is None and self.lo == INT_MIN and self.hi == INT_MAX

    def ensure_transposed(self) -> None:
        """Make the query-packed copy of a bitmap (what the dK/dV kernel reads) if it does not exist yet: large
        bitmaps are lowered without it, so that a forward-only user never holds the second copy.  Built from the
        key-packed words on the device, one (batch, head) slab of rows at a time."""
        if self.bits is None or self.bits_t is not None:
            return
        Bm, Hm, Qp, W = self.bits.shape
        KVp = W * 32
        out = torch.empty((Bm, Hm, KVp, Qp // 32), dtype=torch.int32, device=self.bits.device)
        rows = max(32, min(Qp, (_SLAB_ELEMS // KVp) // 32 * 32))
        for b in range(Bm):
            for h in range(Hm):
                for q0 in range(0, Qp, rows):
                    m = unpack_bits(self.bits[b, h, q0:q0 + rows], KVp)          # [rows, KVp]
                    out[b, h, :, q0 // 32:(q0 + m.shape[0]) // 32] = pack_bits(m.transpose(0, 1).contiguous())
        self.bits_t = out

    def key(self):
        if self.bits is not None:
            return ("bits", self.bits.data_ptr())
        return ("band", self.lo, self.hi, self.sink, self.q_offset)

    def c_struct(self) -> _lib.FlexMask:
        m = _lib.FlexMask()
        m.kind, m.lo, m.hi, m.sink, m.q_offset = self.kind, self.lo, self.hi, self.sink, self.q_offset
        if self.bits is not None:
            Bm, Hm, Qp, W = self.bits.shape
            m.bits = self.bits.data_ptr()
            m.bits_stride_b = 0 if Bm == 1 else Hm * Qp * W
            m.bits_stride_h = 0 if Hm == 1 else Qp * W
            m.bits_stride_q = W
            if self.bits_t is not None:
                _, _, KVp, Wq = self.bits_t.shape
                m.bits_t = self.bits_t.data_ptr()
                m.bits_t_stride_b = 0 if Bm == 1 else Hm * KVp * Wq
                m.bits_t_stride_h = 0 if Hm == 1 else KVp * Wq
                m.bits_t_stride_kv = Wq
            if self.blk is not None:
                _, _, nqb, nkb = self.blk.shape
                m.blk = self.blk.data_ptr()
                m.blk_stride_b = 0 if Bm == 1 else Hm * nqb * nkb
                m.blk_stride_h = 0 if Hm == 1 else nqb * nkb
                m.blk_stride_q = nkb
        return m

    def __call__(self, b, h, q_idx, kv_idx):
        if self.bits is not None:
            return self.fn(b, h, q_idx, kv_idx)
        d = q_idx + self.q_offset - kv_idx
        r = (d >= self.lo)
        if self.hi != INT_MAX:
            r = r & ((d <= self.hi) | ((kv_idx + 0 * q_idx) <= self.sink))
        return r

    def __repr__(self):
        if self.bits is not None:
            return f"MaskMod({self.__name__}, bitmap {tuple(self.bits.shape)})"
        return f"MaskMod({self.__name__}, lo={self.lo}, hi={self.hi}, sink={self.sink}, q_offset={self.q_offset})"


def band_and(a: MaskMod, b: MaskMod) -> Optional[MaskMod]:
    """Intersection of two band masks when it is again a band mask."""
    if a.bits is not None or b.bits is not None or a.q_offset != b.q_offset:
        return None
    lo = max(a.lo, b.lo)
    if a.hi == INT_MAX:
        hi, sink = b.hi, b.sink
    elif b.hi == INT_MAX:
        hi, sink = a.hi, a.sink
    elif a.sink == b.sink:
        hi, sink = min(a.hi, b.hi), a.sink
    elif a.hi == b.hi:
        hi, sink = a.hi, min(a.sink, b.sink)
    else:
        return None
    return MaskMod(lo, hi, sink, a.q_offset, name="and_mask")


def band_or(a: MaskMod, b: MaskMod) -> Optional[MaskMod]:
    """Union of two band masks when it is again a band mask."""
    if a.bits is not None or b.bits is not None or a.q_offset != b.q_offset:
        return None
    if a.lo == INT_MIN and b.lo == INT_MIN:
        return MaskMod(INT_MIN, max(a.hi, b.hi), max(a.sink, b.sink), a.q_offset, name="or_mask")
    if a.lo == INT_MAX:
        return b
    if b.lo == INT_MAX:
        return a
    if (a.hi, a.sink) == (b.hi, b.sink):
        return MaskMod(min(a.lo, b.lo), a.hi, a.sink, a.q_offset, name="or_mask")
    return None


def _pad128(n: int) -> int:
    return (n + 127) // 128 * 128


def _eval_mask(fn: Callable, b, h, q, kv) -> torch.Tensor:
    """fn on broadcastable int32 index tensors -> bool tensor (a five-argument score_mod masks where it
    returns -inf: flaxattention/core/blockmask.py:307-315)."""
    dev = q.device
    if _get_mod_type(fn) == _ModificationType.SCORE_MOD:
        shape = torch.broadcast_shapes(b.shape, h.shape, q.shape, kv.shape)
        out = fn(torch.zeros(shape, device=dev), b, h, q, kv)
        return ~torch.isneginf(torch.as_tensor(out, device=dev))
    m = fn(b, h, q, kv)
    if not torch.is_tensor(m):
        m = torch.tensor(bool(m), device=dev)
    return m.to(torch.bool)


def _scan_captures(fn, tensors: list, depth: int = 0, scalars: Optional[list] = None) -> bool:
    """Walk what `fn` closes over, defaults to or reads from its globals.  Tensors found on the way are
    appended to `tensors` (and numbers / strings to `scalars`, when given); the return value says whether
    everything else was transparent: modules, containers of such, and functions that are themselves
    transparent.  An object of any other kind (an array, a module instance, a bound method) may hold state
    this walk cannot see."""
    import functools
    import types

    def plain(x) -> bool:
        if x is None or isinstance(x, (types.ModuleType, type)):
            return True
        if isinstance(x, (bool, int, float, complex, str, bytes)):
            if scalars is not None:
                scalars.append(x)
            return True
        if torch.is_tensor(x):
            tensors.append(x)
            return True
        if isinstance(x, MaskMod):
            if x.bits is not None:
                tensors.append(x.bits)
            return True
        if isinstance(x, ScoreMod):
            tensors.extend(t for t in (x.mul, x.add) if t is not None)
            return True
        if isinstance(x, (tuple, list, frozenset, set)):
            return all([plain(y) for y in x])
        if isinstance(x, dict):
            return all([plain(y) for y in x.values()])
        if isinstance(x, (types.FunctionType, types.BuiltinFunctionType, functools.partial)):
            return _scan_captures(x, tensors, depth + 1, scalars)
        return False

    if depth > 4:
        return False
    if isinstance(fn, (MaskMod, ScoreMod)):
        return plain(fn)
    if isinstance(fn, functools.partial):
        return all([plain(fn.func), plain(fn.args), plain(fn.keywords)])
    if isinstance(fn, types.BuiltinFunctionType):
        return True
    code = getattr(fn, "__code__", None)
    if code is None or getattr(fn, "__self__", None) is not None:
        return False
    seen = [c.cell_contents for c in (fn.__closure__ or ())]
    seen += list(fn.__defaults__ or ()) + list((fn.__kwdefaults__ or {}).values())
    seen += [fn.__globals__[n] for n in code.co_names if n in fn.__globals__]
    return all([plain(x) for x in seen])


def _index_arithmetic_only(fn) -> bool:
    """True when `fn` provably computes from its index arguments alone: everything it closes over, defaults to
    or reads from its globals is a number, a string, a module or another such function.  Anything else (a
    tensor, an array, an object that may hold one) makes it a mod that may look positions up in a buffer."""
    tensors: list = []
    return _scan_captures(fn, tensors) and not tensors


def _capture_stamp(fn):
    """What a cached lowering of `fn` depends on besides `fn` itself: the captured tensors with their version
    counters and the captured numbers and strings, or None when `fn` holds state that cannot be seen (then
    nothing about it may be cached)."""
    tensors: list = []
    scalars: list = []
    if not _scan_captures(fn, tensors, 0, scalars):
        return None
    return [(t, t._version) for t in tensors] + [(None, tuple(scalars))]


def _callable_key(fn, stamp):
    """Cache key of a callable.  A plain function or lambda whose captures can all be seen is known by its code object
    and by what it captures (numbers and strings by value, tensors by identity), so that a closure made anew for every
    call -- `lambda s, b, h, q, kv: s + bias[h]` inside a training step -- finds the lowering of its predecessor;
    anything else (a partial, a bound method, a callable with hidden state) is known by its identity."""
    code = getattr(fn, "__code__", None)
    if code is None or stamp is None:
        return ("id", id(fn))
    try:
        key = ("code", code, stamp[-1][1], tuple(id(t) for t, _ in stamp[:-1]))
        hash(key)
        return key
    except TypeError:
        return ("id", id(fn))


def _same_callable(cached, fn) -> bool:
    """`fn` is the callable a cache entry was made from, or another instance of the same code (what it captures is
    compared by the caller through the stamps)."""
    if cached is fn:
        return True
    code = getattr(fn, "__code__", None)
    return code is not None and getattr(cached, "__code__", None) is code


def _stamp_valid(stamp, now=None) -> bool:
    """`stamp` (taken when a lowering was cached) still describes the callable: the same tensors at the same
    versions.  `now` is a fresh stamp of the callable (a closure variable may have been rebound to another tensor)."""
    if now is not None:
        if len(now) != len(stamp) or any(a[0] is not b[0] for a, b in zip(now, stamp)) or now[-1][1] != stamp[-1][1]:
            return False
    return all(t._version == v for t, v in stamp[:-1])


def dense_mask_on_device(fn: Callable, B: int, H: int, Q: int, KV: int, device,
                         real: Optional[Tuple[int, int]] = None, b_range: Optional[Tuple[int, int]] = None,
                         h_range: Optional[Tuple[int, int]] = None, q_range: Optional[Tuple[int, int]] = None) -> torch.Tensor:
    """Evaluate a Python mask_mod (or a five-argument score_mod) over the index grid [0,Q) x [0,KV) with
    device tensors.  bool, broadcastable to [B,H,Q,KV].

    `real` = (Q_LEN, KV_LEN) when the grid is the padded one of the block-mask builder, which treats
    positions past the end as if they were real (blockmask.py:440-444).  A mod that looks positions up in
    captured tensors must never be handed such indices (an out-of-range index into a device tensor stops
    the process, and torch accepts CPU index tensors for device tensors, so trying on the CPU first is no
    protection): unless the mod provably computes from its index arguments alone, the part of the grid past
    the real lengths is evaluated with indices clamped to the last real position, which is what an
    out-of-range gather yields under XLA.

    `b_range` / `h_range` / `q_range` restrict the evaluation to a slab (batches [b0,b1), heads [h0,h1), query
    rows [q0,q1)); the result then covers that slab only."""
    b0, b1 = b_range or (0, B)
    h0, h1 = h_range or (0, H)
    q_lo, q_hi = q_range or (0, Q)

    def grid(where, qs, ks, clamp=False):
        q = torch.arange(qs[0], qs[1], dtype=torch.int32, device=where).reshape(1, 1, -1, 1)
        kv = torch.arange(ks[0], ks[1], dtype=torch.int32, device=where).reshape(1, 1, 1, -1)
        if clamp:
            q, kv = q.clamp(max=Qr - 1), kv.clamp(max=KVr - 1)
        b = torch.arange(b0, b1, dtype=torch.int32, device=where).reshape(-1, 1, 1, 1)
        h = torch.arange(h0, h1, dtype=torch.int32, device=where).reshape(1, -1, 1, 1)
        return _eval_mask(fn, b, h, q, kv).to(device)

    Qr, KVr = (Q, KV) if real is None else (min(real[0], Q), min(real[1], KV))
    if q_range is not None:
        # a slab of rows: the same three regions, cut to [q_lo, q_hi)
        clamp = not _index_arithmetic_only(fn)
        m = torch.zeros((b1 - b0, h1 - h0, q_hi - q_lo, KV), dtype=torch.bool, device=device)
        q_mid = min(max(Qr, q_lo), q_hi)   # rows [q_lo, q_mid) are real, [q_mid, q_hi) lie past the end
        if q_mid > q_lo:
            m[:, :, :q_mid - q_lo, :KVr] = grid(device, (q_lo, q_mid), (0, KVr))
            if KVr < KV:
                m[:, :, :q_mid - q_lo, KVr:] = grid(device, (q_lo, q_mid), (KVr, KV), clamp)
        if q_hi > q_mid:
            m[:, :, q_mid - q_lo:, :] = grid(device, (q_mid, q_hi), (0, KV), clamp)
        return m
    core = grid(device, (0, Qr), (0, KVr))
    if Qr == Q and KVr == KV:
        return core

    clamp = not _index_arithmetic_only(fn)

    def beyond(qs, ks):
        return grid(device, qs, ks, clamp)
    pieces = [(core, (0, Qr), (0, KVr))]
    if Qr < Q:
        pieces.append((beyond((Qr, Q), (0, KV)), (Qr, Q), (0, KV)))
    if KVr < KV:
        pieces.append((beyond((0, Qr), (KVr, KV)), (0, Qr), (KVr, KV)))
    Bm = max(t.shape[0] if t.dim() == 4 else 1 for t, _, _ in pieces)
    Hm = max(t.shape[1] if t.dim() == 4 else 1 for t, _, _ in pieces)
    m = torch.zeros((Bm, Hm, Q, KV), dtype=torch.bool, device=device)
    for t, (q0, q1), (k0, k1) in pieces:
        m[:, :, q0:q1, k0:k1] = torch.broadcast_to(t, (Bm, Hm, q1 - q0, k1 - k0))
    return m


def _fit_band(m2: torch.Tensor) -> Optional[MaskMod]:
    """Given a [Q,KV] boolean matrix, find band parameters that reproduce it
    exactly over the whole matrix, if any."""
    Q, KV = m2.shape
    dev = m2.device
    q = torch.arange(Q, device=dev, dtype=torch.int32).reshape(Q, 1)
    kv = torch.arange(KV, device=dev, dtype=torch.int32).reshape(1, KV)
    d = q - kv
    if not bool(m2.any()):
        return MaskMod(INT_MAX, INT_MAX, -1, name="all_false")
    lo = int(d[m2].min())
    if lo <= -(KV - 1):
        lo = INT_MIN
    inside = d >= lo
    hidden = inside & ~m2
    cands = []
    if not bool(hidden.any()):
        cands.append((lo, INT_MAX, -1))
    else:
        hi = int(d[hidden].min()) - 1
        sink = int(torch.broadcast_to(kv, d.shape)[hidden].min()) - 1
        cands.append((lo, hi, sink))
        cands.append((lo, hi, -1))
    for lo_, hi_, sink_ in cands:
        test = (d >= lo_) & ((d <= hi_) | (kv <= sink_))
        if bool((test == m2).all()):
            return MaskMod(lo_, hi_, sink_, name="band")
    return None


def pack_bits(mask: torch.Tensor) -> torch.Tensor:
    """bool [..., KV] -> int32 words [..., ceil(KV/32)], bit (kv & 31) of word kv >> 5."""
    *lead, KV = mask.shape
    W = (KV + 31) // 32
    if W * 32 != KV:
        mask = torch.nn.functional.pad(mask, (0, W * 32 - KV))
    # eight entries to a byte, four bytes (little-endian) to a word: no temporary wider than the mask itself
    weights = torch.tensor([1, 2, 4, 8, 16, 32, 64, 128], dtype=torch.uint8, device=mask.device)
    by = (mask.reshape(*lead, W * 4, 8).to(torch.uint8) * weights).sum(-1, dtype=torch.uint8)
    return by.contiguous().view(torch.int32).reshape(*lead, W)


def unpack_bits(words: torch.Tensor, n: int) -> torch.Tensor:
    """int32 words [..., W] -> bool [..., n]: the inverse of pack_bits."""
    *lead, W = words.shape
    by = words.contiguous().view(torch.uint8).reshape(*lead, W * 4, 1)
    shifts = torch.arange(8, dtype=torch.uint8, device=words.device)
    return ((by >> shifts) & 1).to(torch.bool).reshape(*lead, W * 32)[..., :n]


def block_classes(mask: torch.Tensor) -> torch.Tensor:
    """bool [..., Q, KV] (both multiples of 32) -> int8 [..., Q/32, KV/32]: 1 where a 32 x 32 block is entirely set,
    2 where it is entirely clear, 0 otherwise (the kernels' kBlockAll / kBlockNone / kBlockMixed)."""
    *lead, Q, KV = mask.shape
    count = mask.reshape(*lead, Q // 32, 32, KV // 32, 32).sum(dim=(-3, -1), dtype=torch.int32)
    cls = torch.zeros_like(count, dtype=torch.int8)
    cls[count == 1024] = 1
    cls[count == 0] = 2
    return cls.contiguous()


def resolve_mask_mod(fn: Optional[Callable], B: int, H: int, Q: int, KV: int, device,
                     real: Optional[Tuple[int, int]] = None) -> MaskMod:
    """Lower a mask_mod callable to a kernel functor that is exact on the
    index range [0, pad128(Q)) x [0, pad128(KV)).  Tagged functors pass
    through; any other callable is evaluated densely on the device once and
    either recognised as a band mask (checked against every entry) or kept as
    a packed bitmap.  `real` gives the true sequence lengths when Q / KV are already rounded up."""
    if fn is None:
        return MaskMod(name="noop_mask")
    if isinstance(fn, MaskMod) and fn.bits is None:
        return fn
    if isinstance(fn, MaskMod):
        Bm, Hm, Qp, W = fn.bits.shape
        if Qp >= _pad128(Q) and W * 32 >= _pad128(KV) and Bm in (1, B) and Hm in (1, H):
            return fn
        fn = fn.fn
    Qp, KVp = _pad128(Q), _pad128(KV)
    # the dense evaluation is remembered per callable, shape and the captured tensors at their versions
    stamp = _capture_stamp(fn)
    key = (_callable_key(fn, stamp), B, H, Q, KV, str(device), real)
    hit = _mask_cache.get(key)
    if hit is not None and _same_callable(hit[0], fn) and stamp is not None and _stamp_valid(hit[2], stamp):
        return hit[1]
    spec = _lower_mask_callable(fn, B, H, Q, KV, Qp, KVp, device, real)
    if stamp is not None:
        if len(_mask_cache) > 32:
            _mask_cache.clear()
        _mask_cache[key] = (fn, spec, stamp)
    return spec


_mask_cache: dict = {}


_SLAB_ELEMS = 1 << 24          # mask entries evaluated at a time (the callable's own temporaries scale with this)
_FIT_ELEMS = 1 << 25           # entries of the first rows on which band parameters are fitted
_EAGER_T_BYTES = 64 << 20      # bitmaps up to this size get their query-packed copy right away


def _bh_extents(fn: Callable, B: int, H: int, device) -> Tuple[int, int]:
    """Which of the batch and head extents the callable's result has at all (1 = it broadcasts): read off the shape
    it returns for a single position."""
    if B == 1 and H == 1:
        return 1, 1
    one = dense_mask_on_device(fn, B, H, 1, 1, device, real=(1, 1))
    Bm = one.shape[0] if one.dim() == 4 else 1
    Hm = one.shape[1] if one.dim() == 4 else 1
    return (B if Bm > 1 else 1), (H if Hm > 1 else 1)


def _band_equals_bitmap(band: MaskMod, words: torch.Tensor, rows: int) -> bool:
    """The band functor reproduces every bit of the key-packed bitmap `words` [Qp, W]."""
    Qp, W = words.shape
    dev = words.device
    kv = torch.arange(W * 32, dtype=torch.int32, device=dev).reshape(1, -1)
    zero = torch.zeros((), dtype=torch.int32, device=dev)
    for q0 in range(0, Qp, rows):
        q = torch.arange(q0, min(q0 + rows, Qp), dtype=torch.int32, device=dev).reshape(-1, 1)
        m = torch.broadcast_to(band(zero, zero, q, kv), (q.numel(), W * 32))
        if not bool(torch.equal(pack_bits(m.contiguous()), words[q0:q0 + rows])):
            return False
    return True


def _lower_mask_callable(fn: Callable, B: int, H: int, Q: int, KV: int, Qp: int, KVp: int, device, real) -> MaskMod:
    """Evaluate the callable over the padded index grid one (batch, head, rows) slab at a time -- the dense
    [B,H,Q,KV] mask is never held -- and pack each slab straight into the bitmap words and the classes of its
    32 x 32 blocks.  If every (batch, head) turns out to carry the same mask, it is fitted to the band form or kept
    as one broadcast bitmap."""
    name = getattr(fn, "__name__", "mask_mod")
    real = real or (Q, KV)
    Bm, Hm = _bh_extents(fn, B, H, device)
    rows = max(128, min(Qp, (_SLAB_ELEMS // KVp) // 128 * 128))
    W = KVp // 32
    bits = torch.empty((Bm, Hm, Qp, W), dtype=torch.int32, device=device)
    blk = torch.empty((Bm, Hm, Qp // 32, KVp // 32), dtype=torch.int8, device=device)
    same = True          # every (batch, head) seen so far equals (0, 0)
    for b in range(Bm):
        for h in range(Hm):
            for q0 in range(0, Qp, rows):
                q1 = min(q0 + rows, Qp)
                m = dense_mask_on_device(fn, B, H, Qp, KVp, device, real=real, b_range=(b, b + 1), h_range=(h, h + 1),
                                         q_range=(q0, q1))[0, 0]
                bits[b, h, q0:q1] = pack_bits(m)
                blk[b, h, q0 // 32:q1 // 32] = block_classes(m)
                if same and (b or h):
                    same = bool(torch.equal(bits[b, h, q0:q1], bits[0, 0, q0:q1]))
    if same:
        # the closed band form: parameters are fitted on the first rows (_FIT_ELEMS entries) and then
        # checked against EVERY word of the bitmap, slab by slab; a band whose window is longer than the fitted rows
        # fails that check and stays a bitmap
        bits, blk = bits[:1, :1].contiguous(), blk[:1, :1].contiguous()   # (lets go of the per-(batch, head) arrays)
        fit_rows = min(Qp, max(128, (_FIT_ELEMS // KVp) // 128 * 128))
        band = _fit_band(unpack_bits(bits[0, 0, :fit_rows], KVp))
        if band is not None and _band_equals_bitmap(band, bits[0, 0], rows):
            band.__name__ = name
            return band
    spec = MaskMod(name=name, bits=bits, fn=fn, blk=blk)
    if bits.numel() * 4 <= _EAGER_T_BYTES:
        spec.ensure_transposed()
    return spec
