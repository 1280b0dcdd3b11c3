"""Front-ends: flax_attention, flax_attention_pallas, math_attention.

Same names, arguments, defaults and errors as flaxattention/core/attention.py
(flax_attention 169-218, flax_attention_pallas 220-312, math_attention 67-106,
validators 119-167).  Arrays are torch tensors resident on the MI355X; the
work is done by the HIP kernels behind include/flexattn.h, reached through
ctypes.  Differentiation goes through a torch.autograd.Function that plays the
role of the reference's jax.custom_vjp (kernel/attention.py:166-168, 653):
forward saves (q, k, v, out, lse2), backward returns (dq, dk, dv).

``kernel_options`` (accepted and ignored by the reference, attention.py:179)
selects numerics here:
    {"numerics": "parity" | "fast"}   fused (matrix-core) kernels, 16-bit inputs:
                        "parity": the rounding points of the reference's dense
                        path -- S rounded to the input dtype (attention.py:27),
                        the NORMALISED P rounded before P.V (attention.py:104-105;
                        a two-pass forward), and in the backward dP rounded,
                        delta = sum_j P round(dP), dS rounded after scaling.
                        "fast": one-pass online softmax (the unnormalised P is
                        rounded), delta = sum_d O dO, dP kept in fp32; about 1.5x
                        faster.  Default: "parity" for bfloat16, whose 8-bit
                        mantissa puts "fast" 3e-3 (relative L2) away from the dense
                        path, and "fast" for float16, where it stays within 1e-3.
                        "unrounded": no internal round trip at all -- S is not
                        rounded, P and dS enter the matrix products as a high and
                        a low part (twice the mantissa), delta = sum_j P dP from an
                        unrounded row sweep; only the results are rounded.  What
                        the dense path computes if XLA removes the round trips of
                        attention.py:27, 104-105 (excess-precision simplification);
                        within 1e-4 of that variant of the oracle, about 1.6x the
                        time of "fast".
    {"strict": True}    faithful kernels on the vector ALU: the same rounding
                        points as "parity", any dtype and head size
    {"round_s": bool}   fused kernels: round Q.K^T through the input dtype
                        (default True, as attention.py:27 computes that product
                        in the input dtype)
    {"backend": "generic" | "auto"}
    {"decode": bool}      split-KV decode kernel on / off; by default it is used
                          whenever it applies (fp16/bf16, D = Dv in {64, 128} with
                          at most 64 query rows per KV head or D = Dv in {192, 256}
                          with at most 32, at least 512 keys); True also runs longer queries
                          through it, in chunks of that many rows
    {"decode_splits": n}  force the split-KV decode kernel with n splits
    {"split_kv": bool}    False: the forward kernel never splits a call over the keys
                          (by default it does when the query tiles alone are fewer
                          workgroups than the GPU has compute units); the result of a
                          (batch, head) pair then does not depend on how many pairs
                          the call has, bit for bit
    {"pad_head_dim": bool}  inputs whose head sizes are not among those of the matrix-core kernels
                          (D = Dv in {64, 128}, 16-bit inputs also {192, 256}) but no larger are
                          zero-padded to the next of those (default True)
    {"tile_lists": bool}  False: call the library without tile lists, as a C-ABI caller without a
                          block mask would; every tile is then visited and the mask evaluated in
                          each (default True: lists are built from the mask)
"""
from __future__ import annotations

import math
from typing import Any, Callable, Dict, Optional, Tuple, Union

import torch

from .. import _lib
from .blockmask import BlockMask, _create_empty_block_mask
from .common import (IDENTITY, MaskMod, ScoreMod, ScoreModNotLowered, _identity, _mask_mod_signature,
                     _score_mod_signature, resolve_mask_mod, resolve_score_mod)

Array = torch.Tensor

_DTYPES = {torch.float32: _lib.FLEX_F32, torch.float16: _lib.FLEX_F16, torch.bfloat16: _lib.FLEX_BF16}


def _validate_sdpa_input(query, key, value, attn_mask=None, dropout_p=0.0, is_causal=False, scale=None):
    """attention.py:119-138."""
    if query.dtype != key.dtype or query.dtype != value.dtype:
        raise ValueError(
            f"Expected query, key, and value to have the same dtype, "
            f"but got query.dtype: {query.dtype}, key.dtype: {key.dtype}, "
            f"and value.dtype: {value.dtype} instead."
        )
    if query.dim() < 2 or key.dim() < 2 or value.dim() < 2:
        raise ValueError(
            f"Expected query, key, and value to all be  at least 2 dimensional, but got query.dim: "
            f"{query.dim()}, key.dim: {key.dim()} and value.dim: {value.dim()} instead."
        )


def _validate_embed_dim(query, key, value):
    """attention.py:149-167."""
    if query.shape[-1] != key.shape[-1]:
        raise ValueError(
            f"Expect query and key/value to have the same embedding dimension "
            f"but got E={query.shape[-1]} and E={key.shape[-1]}."
        )
    if value.shape[-1] > query.shape[-1]:
        raise ValueError(
            f"NYI: Currently value embedding dimension must be less than or equal to query embedding dimension. "
            f"Got Ev={value.shape[-1]} and E={query.shape[-1]}."
        )


def _require_device(*ts):
    for t in ts:
        if not t.is_cuda:
            raise _lib.FlexAttnError("flaxattention_amd computes on the HIP device only: got a CPU tensor "
                                     "(there is no CPU fallback)")
    if ts[0].dtype not in _DTYPES:
        raise TypeError(f"unsupported dtype {ts[0].dtype}; use float32, float16 or bfloat16")


class _Plan:
    """Everything but the tensors: the POD the C ABI takes plus what keeps its
    device pointers alive."""

    def __init__(self, q, k, v, score: ScoreMod, mask: MaskMod, block_mask: Optional[BlockMask], scale: float,
                 flags: int, bhld: bool, decode_splits: int = 0):
        # logical [B,H,L,D] views; physical layout may be [B,L,H,D]
        self.B, self.Hq, self.Lq, self.D = q.shape
        self.Hkv, self.Lkv, self.Dv = k.shape[1], k.shape[2], v.shape[3]
        self.dtype = q.dtype
        self.score, self.mask, self.block_mask = score, mask, block_mask
        # decode_splits: > 0 = decode kernel with that many splits, < 0 = decode kernel with the
        # library's default split count, 0 = forward kernel
        self.scale, self.flags, self.decode_splits = float(scale), int(flags), int(decode_splits)
        self.split_kv = True    # the forward kernel may split a call with few query tiles over the keys
        self.fwd_ws_bytes = None   # bytes of split partials the library wants for the forward (asked on first use)
        self.lists = None       # tile lists for the forward / decode kernels
        self.lists_bwd = None   # tile lists for the backward kernels
        self.keep = [mask.bits, score.mul, score.add]
        self._params = {}       # parameter blocks by (strides, rows, row offset): a repeated call fills none

    def params(self, q, k, v, o, q_index_base: int = 0) -> _lib.FlexAttnParams:
        """q / o may be a slice of rows [q_index_base, q_index_base + q.shape[2]) of the planned query
        (decode in chunks); everything else refers to the whole problem.  The block is built once per layout and
        handed out again for the same layout (callers that change a field, as the backward does with d_lse2, copy it)."""
        key = (q.stride(), k.stride(), v.stride(), o.stride(), q.shape[2], int(q_index_base), id(self.score), id(self.mask),
               id(self.lists), id(self.lists_bwd))
        hit = self._params.get(key)
        if hit is not None:
            return hit
        p = self._build_params(q, k, v, o, q_index_base)
        if len(self._params) > 16:
            self._params.clear()
        self._params[key] = p
        return p

    def _build_params(self, q, k, v, o, q_index_base: int = 0) -> _lib.FlexAttnParams:
        p = _lib.FlexAttnParams()
        p.dtype = _DTYPES[self.dtype]
        p.B, p.Hq, p.Hkv, p.Lq, p.Lkv, p.D, p.Dv = self.B, self.Hq, self.Hkv, q.shape[2], self.Lkv, self.D, self.Dv
        p.q_index_base = int(q_index_base)
        for name, t in (("q_stride", q), ("k_stride", k), ("v_stride", v), ("o_stride", o)):
            if t.stride(3) != 1:
                raise _lib.FlexAttnError("the feature axis must be contiguous")
            getattr(p, name)[:] = [t.stride(0), t.stride(1), t.stride(2)]
        p.scale, p.flags = self.scale, self.flags
        p.score = self.score.c_struct()
        p.mask = self.mask.c_struct()
        for L, t in ((self.lists, p.tiles), (self.lists_bwd, p.tiles_bwd)):
            if L is None:
                continue
            t.kv_num, t.kv_idx = L["kv_num_blocks"].data_ptr(), L["kv_indices"].data_ptr()
            t.full_kv_num, t.full_kv_idx = L["full_kv_num_blocks"].data_ptr(), L["full_kv_indices"].data_ptr()
            t.q_num, t.q_idx = L["q_num_blocks"].data_ptr(), L["q_indices"].data_ptr()
            t.full_q_num, t.full_q_idx = L["full_q_num_blocks"].data_ptr(), L["full_q_indices"].data_ptr()
            t.q_block, t.kv_block = L["q_block"], L["kv_block"]
            t.n_q_blocks, t.n_kv_blocks = L["n_q_blocks"], L["n_kv_blocks"]
            t.stride_b = 0 if L["B"] == 1 else L["H"]
            t.stride_h = 0 if L["H"] == 1 else 1
        return p


def _make_plan(q, k, v, score_mod, block_mask: Optional[BlockMask], mask_mod, scale, kernel_options) -> _Plan:
    opts = dict(kernel_options or {})
    B, Hq, Lq, D = q.shape
    Lkv = k.shape[2]
    dev = q.device
    score = resolve_score_mod(score_mod, Hq, (B, Hq, Lq, Lkv), dev)
    if block_mask is not None:
        if block_mask.seq_lengths is not None and (block_mask.seq_lengths[0] < Lq or block_mask.seq_lengths[1] < Lkv):
            raise ValueError(f"block_mask was built for lengths {block_mask.seq_lengths}, "
                             f"but the inputs have Lq={Lq}, Lkv={Lkv}")
        mask = block_mask.resolved_spec(B, Hq, Lq, Lkv, dev)
    else:
        mask = resolve_mask_mod(mask_mod, B, Hq, Lq, Lkv, dev)
    flags = 0
    if opts.get("strict", False):
        flags |= _lib.FLAG_STRICT
    if opts.get("round_s", True) and q.dtype != torch.float32:
        flags |= _lib.FLAG_ROUND_S
    if opts.get("backend", "auto") == "generic":
        flags |= _lib.FLAG_FORCE_GENERIC
    numerics = opts.get("numerics", "parity" if q.dtype == torch.bfloat16 else "fast")
    if numerics not in ("parity", "fast", "unrounded"):
        raise ValueError(f'kernel_options["numerics"] must be "parity", "fast" or "unrounded", got {numerics!r}')
    if numerics == "parity" and q.dtype != torch.float32:
        flags |= _lib.FLAG_PARITY
    if numerics == "unrounded":
        flags = (flags & ~(_lib.FLAG_ROUND_S | _lib.FLAG_STRICT)) | _lib.FLAG_UNROUNDED
    plan = _Plan(q, k, v, score, mask, block_mask, scale, flags, True, _decode_choice(q, k, v, score, flags, opts))
    plan.split_kv = bool(opts.get("split_kv", True))
    # tile lists at the fused kernels' granularity (skipped for a mask that hides nothing)
    if not mask.is_noop() and opts.get("tile_lists", True) and not (flags & (_lib.FLAG_STRICT | _lib.FLAG_FORCE_GENERIC)):
        holder = block_mask if block_mask is not None else _holder_for(mask)
        holder.spec = mask
        for which in (0, 1):
            qb, kvb = _lib.C.c_int32(0), _lib.C.c_int32(0)
            _lib.lib().flexattn_preferred_tiles(_DTYPES[q.dtype], D, v.shape[3], Lq, Lkv, which,
                                                _lib.C.byref(qb), _lib.C.byref(kvb))
            if qb.value > 0:
                lists = holder.tile_lists(qb.value, kvb.value, B, Hq, Lq, Lkv, dev)
                if which == 0:
                    plan.lists = lists
                else:
                    plan.lists_bwd = lists
    return plan


_plans: dict = {}


def _plan_for(q, k, v, score_mod, block_mask: Optional[BlockMask], mask_mod, scale, kernel_options) -> _Plan:
    """_make_plan, remembered for calls that repeat: the same tagged functors (or none), the same BlockMask object,
    shapes, dtype, scale and options give the same plan, so a training loop lowers nothing and looks nothing up after
    its first step.  Untagged Python callables are not remembered here: what they capture may change between calls,
    which their own lowering caches track (common.py)."""
    def fixed(f, cls):
        return f is None or f is _identity or (isinstance(f, cls) and getattr(f, "bits", None) is None
                                               and getattr(f, "kind", 0) != _lib.SCORE_AFFINE)
    src = block_mask.mask_mod if block_mask is not None else None
    if not (fixed(score_mod, ScoreMod) and fixed(mask_mod, MaskMod) and fixed(src, MaskMod)):
        return _make_plan(q, k, v, score_mod, block_mask, mask_mod, scale, kernel_options)
    try:
        key = (id(score_mod), id(block_mask), id(mask_mod), tuple(q.shape), tuple(k.shape), tuple(v.shape), q.dtype,
               q.device, float(scale), tuple(sorted((kernel_options or {}).items())))
        hit = _plans.get(key)
    except TypeError:   # an option value that cannot be hashed
        return _make_plan(q, k, v, score_mod, block_mask, mask_mod, scale, kernel_options)
    if hit is not None and hit[1] is score_mod and hit[2] is block_mask and hit[3] is mask_mod:
        return hit[0]
    plan = _make_plan(q, k, v, score_mod, block_mask, mask_mod, scale, kernel_options)
    if len(_plans) > 64:
        _plans.clear()
    _plans[key] = (plan, score_mod, block_mask, mask_mod)   # the objects are held so that their ids stay theirs
    return plan


def _decode_choice(q, k, v, score: ScoreMod, flags: int, opts: dict) -> int:
    """Split count for the decode kernel (> 0 given, < 0 library default) or 0 for the forward kernel."""
    if int(opts.get("decode_splits", 0)) > 0:
        return int(opts["decode_splits"])
    want = opts.get("decode")
    if want is False:
        return 0
    B, Hq, Lq, D = q.shape
    G = Hq // k.shape[1]
    ok = (q.dtype in (torch.float16, torch.bfloat16) and D == v.shape[3] and D in (64, 128, 192, 256)
          and score.kind != _lib.SCORE_AFFINE
          and not (flags & (_lib.FLAG_STRICT | _lib.FLAG_FORCE_GENERIC | _lib.FLAG_UNROUNDED)))
    if want is True:
        return -1   # the library reports what does not fit
    if not ok:
        return 0
    # more rows than one decode call takes: the forward kernel, which splits a call with few query tiles over the keys
    # (one pass over the KV cache; measured faster than several decode calls of 64 rows: 124 us against 212 us for 256
    # rows x 16384 keys); {"decode": True} still runs such a query through the decode kernel in chunks
    return -1 if (G * Lq <= _decode_columns(D) and k.shape[2] >= 512) else 0


def _decode_columns(D: int) -> int:
    """Query columns (rows x heads per KV head) one decode call takes."""
    return 32 if D > 128 else 64


_holders: dict = {}


def _holder_for(mask: MaskMod) -> BlockMask:
    """A cache object for tile lists of a mask that came without a BlockMask
    (flax_attention_pallas takes a bare mask_mod)."""
    key = mask.key()
    h = _holders.get(key)
    if h is None:
        if len(_holders) > 64:
            _holders.clear()
        dev = mask.bits.device if mask.bits is not None else torch.device("cuda", torch.cuda.current_device())
        h = BlockMask.from_kv_blocks(torch.ones([1, 1, 1], dtype=torch.int32, device=dev),
                                     torch.zeros([1, 1, 1, 1], dtype=torch.int32, device=dev), mask_mod=mask)
        _holders[key] = h
    return h


def _stream(t) -> int:
    """Raw handle of torch's current stream on the tensor's device (the private accessor skips the Stream object
    that torch.cuda.current_stream builds on every call)."""
    raw = getattr(torch._C, "_cuda_getCurrentRawStream", None)
    if raw is not None:
        return raw(t.device.index if t.device.index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(t.device).cuda_stream


class _on_device:
    """torch.cuda.device(dev) only when dev is not already current (entering the context costs ~10 us of host time)."""
    __slots__ = ("ctx",)

    def __init__(self, dev):
        idx = dev.index
        self.ctx = None if idx is None or idx == torch.cuda.current_device() else torch.cuda.device(dev)

    def __enter__(self):
        if self.ctx is not None:
            self.ctx.__enter__()

    def __exit__(self, *exc):
        if self.ctx is not None:
            self.ctx.__exit__(*exc)
        return False


def _run_fwd(plan: _Plan, q, k, v) -> Tuple[Array, Array]:
    L = _lib.lib()
    o = torch.empty((plan.B, plan.Hq, plan.Lq, plan.Dv), dtype=q.dtype, device=q.device)
    lse2 = torch.empty((plan.B, plan.Hq, plan.Lq), dtype=torch.float32, device=q.device)
    p = plan.params(q, k, v, o)
    with _on_device(q.device):
        if plan.decode_splits != 0:
            splits = max(plan.decode_splits, 0)   # 0 asks the library for its default
            rows = max(_decode_columns(plan.D) // (plan.Hq // plan.Hkv), 1)   # query rows one decode call takes
            if plan.Lq <= rows:
                chunks = [(0, plan.Lq, q, o, lse2, p)]
            else:
                # on request ({"decode": True}) a longer query goes through the decode kernel 64 (D = 256: 32)
                # columns at a time, each call seeing its row offset
                chunks = []
                for s0 in range(0, plan.Lq, rows):
                    s1 = min(s0 + rows, plan.Lq)
                    qc, oc = q[:, :, s0:s1], o[:, :, s0:s1]
                    lc = torch.empty((plan.B, plan.Hq, s1 - s0), dtype=torch.float32, device=q.device)
                    chunks.append((s0, s1, qc, oc, lc, plan.params(qc, k, v, oc, q_index_base=s0)))
            ws = None
            for s0, s1, qc, oc, lc, pc in chunks:
                nbytes = L.flexattn_decode_workspace_bytes(pc, splits)
                if ws is None or ws.numel() < nbytes:
                    ws = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=q.device)
                rc = L.flexattn_decode(pc, qc.data_ptr(), k.data_ptr(), v.data_ptr(), oc.data_ptr(), lc.data_ptr(),
                                       splits, ws.data_ptr(), _stream(q))
                _lib.check(rc, "flexattn_decode")
                if lc is not lse2:
                    lse2[:, :, s0:s1] = lc
        else:
            # few query tiles against many keys: with a workspace the library may split the call over the keys
            # (the library decides from the problem and the device's compute units; 0 = no split.  Asked once per plan)
            ws = None
            if plan.split_kv and plan.Lkv >= 1024:
                if plan.fwd_ws_bytes is None:
                    # the size also covers the log-sum-exp hand-over of the parity numerics, which this front end
                    # never needs (it always passes lse2): beyond that part, the bytes are split partials
                    parity = (plan.flags & _lib.FLAG_PARITY) and not (plan.flags & _lib.FLAG_UNROUNDED)
                    lse_part = (plan.B * plan.Hq * plan.Lq * 4 + 255) // 256 * 256 if parity else 0
                    nbytes = int(L.flexattn_fwd_workspace_bytes(p))
                    plan.fwd_ws_bytes = nbytes if nbytes > lse_part else 0
                if plan.fwd_ws_bytes:
                    ws = torch.empty(plan.fwd_ws_bytes, dtype=torch.uint8, device=q.device)
            rc = L.flexattn_fwd(p, q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse2.data_ptr(),
                                ws.data_ptr() if ws is not None else None, _stream(q))
            _lib.check(rc, "flexattn_fwd")
    return o, lse2


def _run_bwd(plan: _Plan, q, k, v, o, lse2, d_o, d_lse2=None) -> Tuple[Array, Array, Array]:
    L = _lib.lib()
    d_o = d_o.contiguous()
    if d_lse2 is not None:
        d_lse2 = d_lse2.to(torch.float32).contiguous()
    dq = torch.empty((plan.B, plan.Hq, plan.Lq, plan.D), dtype=q.dtype, device=q.device)
    dk = torch.empty((plan.B, plan.Hkv, plan.Lkv, plan.D), dtype=q.dtype, device=q.device)
    dv = torch.empty((plan.B, plan.Hkv, plan.Lkv, plan.Dv), dtype=q.dtype, device=q.device)
    if plan.mask.bits is not None and plan.mask.bits_t is None:
        plan.mask.ensure_transposed()   # the dK/dV kernel reads a bitmap mask packed along the query axis
        plan._params.clear()            # parameter blocks made before carry no pointer to the new copy
    p = plan.params(q, k, v, o)
    if d_lse2 is not None:
        p2 = _lib.FlexAttnParams()      # a copy: the cached block is shared with other calls
        _lib.C.memmove(_lib.C.byref(p2), _lib.C.byref(p), _lib.C.sizeof(p))
        p2.d_lse2 = d_lse2.data_ptr()
        p = p2
    with _on_device(q.device):
        ws = torch.empty(max(L.flexattn_bwd_workspace_bytes(p), 256), dtype=torch.uint8, device=q.device)
        rc = L.flexattn_bwd(p, q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse2.data_ptr(), d_o.data_ptr(),
                            dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), ws.data_ptr(), _stream(q))
    _lib.check(rc, "flexattn_bwd")
    return dq, dk, dv


class _FlexAttention(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, plan: _Plan):
        o, lse2 = _run_fwd(plan, q, k, v)
        ctx.save_for_backward(q, k, v, o, lse2)
        ctx.plan = plan
        ctx.set_materialize_grads(False)   # an output the loss does not use arrives as None, not as zeros
        return o, lse2

    @staticmethod
    def backward(ctx, d_o, d_lse2):
        # the log-sum-exp is a differentiable output as in the reference (attention.py:97-106): its cotangent
        # joins the softmax's row term inside the kernels
        q, k, v, o, lse2 = ctx.saved_tensors
        if d_o is None:
            d_o = torch.zeros_like(o)
        dq, dk, dv = _run_bwd(ctx.plan, q, k, v, o, lse2, d_o, d_lse2)
        return dq, dk, dv, None


# ---- score_mods that cannot be lowered to a functor: linearised at the scores of the call ----------------------
_LINEARISE_BYTES = 2 << 30   # dense fp32 temporaries of one batch chunk (scores, mod, derivative, the two tables)


def _linearised_tables(score_fn, q, k, scale: float, b0: int, h0: int = 0):
    """For an arbitrary differentiable scalar score_mod f: the scaled scores S0 of the call (the product computed in
    the input dtype and cast to fp32, then scaled: attention.py:27, 55), Y = f(S0, b, h, q_idx, kv_idx) and
    G = dY/dS0, as the dense fp32 tables of the affine functor  mul * s + add  with mul = G and add = Y - G * S0.
    At s = S0 that is f(S0) exactly, its derivative is f'(S0), and where a kernel's own score differs from S0 in the
    last bit of the input dtype the difference enters to first order.  `b0` / `h0` are the batch and head index of
    q[0, 0] in the whole problem."""
    B, Hq, Lq, _ = q.shape
    G_ = Hq // k.shape[1]
    kk = k if G_ == 1 else k.repeat_interleave(G_, dim=1)   # the reference repeats K for GQA (attention.py:80-82)
    s0 = (torch.matmul(q, kk.transpose(-1, -2)).to(torch.float32) * scale).requires_grad_(True)
    dev = q.device
    b = torch.arange(b0, b0 + B, dtype=torch.int32, device=dev).reshape(B, 1, 1, 1)
    h = torch.arange(h0, h0 + Hq, dtype=torch.int32, device=dev).reshape(1, Hq, 1, 1)
    qi = torch.arange(Lq, dtype=torch.int32, device=dev).reshape(1, 1, Lq, 1)
    ki = torch.arange(k.shape[2], dtype=torch.int32, device=dev).reshape(1, 1, 1, -1)
    with torch.enable_grad():
        y = torch.as_tensor(score_fn(s0, b, h, qi, ki)).to(torch.float32)
        y = torch.broadcast_to(y, s0.shape)
        (g,) = torch.autograd.grad(y.sum(), s0, allow_unused=True)
    if g is None:
        g = torch.zeros_like(s0)
    y, s0 = y.detach(), s0.detach()
    g = torch.where(torch.isfinite(g), g, torch.zeros_like(g))
    add = torch.where(torch.isfinite(y), y - g * s0, y)   # (a mod that returns -inf masks the entry: keep it)
    return g.contiguous(), add.contiguous()


def _linearise_chunks(B: int, Hq: int, Hkv: int, Lq: int, Lkv: int):
    """(b0, b1, h0, h1) slabs of the problem whose dense fp32 temporaries (scores, mod, derivative and the two
    tables: five [Lq, Lkv] planes per head) stay within _LINEARISE_BYTES: whole batch elements while one fits, else
    whole groups of query heads that share a KV head (one group at least: a single head of 8192 x 8192 is 1.3 GB)."""
    per_head = 5 * Lq * Lkv * 4
    G = Hq // Hkv
    if per_head * Hq <= _LINEARISE_BYTES:
        step = max(1, min(B, _LINEARISE_BYTES // max(per_head * Hq, 1)))
        return [(b0, min(b0 + step, B), 0, Hq) for b0 in range(0, B, step)]
    heads = max(G, (_LINEARISE_BYTES // max(per_head, 1)) // G * G)
    return [(b, b + 1, h0, min(h0 + heads, Hq)) for b in range(B) for h0 in range(0, Hq, heads)]


class _FlexAttentionLinearised(torch.autograd.Function):
    """flax_attention for a score_mod outside the functor families and not affine in the score (the reference applies
    any scalar callable, attention.py:59-63).  Per slab of batch elements (or, when one batch element is too large,
    of query-head groups) the callable and its derivative are evaluated at the call's own scores and handed to the
    kernels as the tables of an affine functor; the backward evaluates them again instead of keeping them."""

    @staticmethod
    def forward(ctx, q, k, v, cfg):
        B, Hq, Lq, _ = q.shape
        G = Hq // k.shape[1]
        o = torch.empty((B, Hq, Lq, v.shape[3]), dtype=q.dtype, device=q.device)
        lse2 = torch.empty((B, Hq, Lq), dtype=torch.float32, device=q.device)
        chunks = _linearise_chunks(B, Hq, k.shape[1], Lq, k.shape[2])
        for b0, b1, h0, h1 in chunks:
            qc, kc, vc = q[b0:b1, h0:h1], k[b0:b1, h0 // G:h1 // G], v[b0:b1, h0 // G:h1 // G]
            plan = _FlexAttentionLinearised._chunk_plan(cfg, qc, kc, vc, b0, h0)
            oc, lc = _run_fwd(plan, qc, kc, vc)
            o[b0:b1, h0:h1], lse2[b0:b1, h0:h1] = oc, lc
            plan.score = None   # the tables are not kept for the backward
        ctx.save_for_backward(q, k, v, o, lse2)
        ctx.cfg, ctx.chunks = cfg, chunks
        ctx.set_materialize_grads(False)
        return o, lse2

    @staticmethod
    def _chunk_plan(cfg, qc, kc, vc, b0, h0=0):
        score_fn, block_mask, mask_mod, scale, opts = cfg
        mul, add = _linearised_tables(score_fn, qc, kc, scale, b0, h0)
        score = ScoreMod(_lib.SCORE_AFFINE, name=getattr(score_fn, "__name__", "score_mod"), mul=mul, add=add, fn=score_fn)
        # the mask of this slab: a functor that does not look at the batch (or head) index serves as it is; anything
        # else is the user's callable with the slab's offsets (lowered again for the slab; the lowering is remembered
        # by the callable's code and offsets, so the backward finds the forward's)
        src = block_mask.mask_mod if block_mask is not None else mask_mod
        spec = block_mask.spec if block_mask is not None else (src if isinstance(src, MaskMod) else None)
        if not (isinstance(spec, MaskMod) and (spec.bits is None or (spec.bits.shape[0] == 1 and (h0 == 0 or spec.bits.shape[1] == 1)))):
            spec = None if src is None else (lambda b, h, q_idx, kv_idx: src(b + b0, h + h0, q_idx, kv_idx))
        plan = _make_plan(qc, kc, vc, IDENTITY, None, spec, scale, opts)
        plan.score = score
        plan.keep = [plan.mask.bits, mul, add]
        return plan

    @staticmethod
    def backward(ctx, d_o, d_lse2):
        q, k, v, o, lse2 = ctx.saved_tensors
        if d_o is None:
            d_o = torch.zeros_like(o)
        G = q.shape[1] // k.shape[1]
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        for b0, b1, h0, h1 in ctx.chunks:
            qc, kc, vc = q[b0:b1, h0:h1], k[b0:b1, h0 // G:h1 // G], v[b0:b1, h0 // G:h1 // G]
            plan = _FlexAttentionLinearised._chunk_plan(ctx.cfg, qc, kc, vc, b0, h0)
            dl = None if d_lse2 is None else d_lse2[b0:b1, h0:h1]
            dq[b0:b1, h0:h1], dk[b0:b1, h0 // G:h1 // G], dv[b0:b1, h0 // G:h1 // G] = _run_bwd(
                plan, qc, kc, vc, o[b0:b1, h0:h1], lse2[b0:b1, h0:h1].contiguous(), d_o[b0:b1, h0:h1], dl)
        return dq, dk, dv, None


def _attend_linearised(q, k, v, score_fn, block_mask, mask_mod, scale, kernel_options) -> Tuple[Array, Array]:
    opts = dict(kernel_options or {})
    opts["decode"] = False   # the split-KV decode kernel takes closed-form functors only
    opts.pop("decode_splits", None)
    cfg = (score_fn, block_mask, mask_mod, float(scale), opts)
    return _FlexAttentionLinearised.apply(q, k, v, cfg)


def _attend(plan: _Plan, q, k, v) -> Tuple[Array, Array]:
    if torch.is_grad_enabled() and (q.requires_grad or k.requires_grad or v.requires_grad):
        return _FlexAttention.apply(q, k, v, plan)
    return _run_fwd(plan, q, k, v)   # nothing to differentiate: no need to pay for the autograd wrapper


class _NothingToAttend(torch.autograd.Function):
    """Inputs with no query rows, batches or heads (empty outputs) or with no keys at all: every row is then a
    fully masked row, whose output is 0 and whose log-sum-exp is -inf (attention.py:97-104).  Gradients are zero.
    Nothing is launched; the kernels take positive sizes only."""
    @staticmethod
    def forward(ctx, q, k, v):
        ctx.meta = [(t.shape, t.dtype, t.device) for t in (q, k, v)]
        out = q.new_zeros(*q.shape[:-1], v.shape[-1])
        lse2 = torch.full(q.shape[:-1], float("-inf"), dtype=torch.float32, device=q.device)
        return out, lse2

    @staticmethod
    def backward(ctx, _d_o, _d_lse):
        return tuple(torch.zeros(s, dtype=d, device=dev) for s, d, dev in ctx.meta)


def _nothing_to_attend(query: Array, key: Array) -> bool:
    return query.numel() == 0 or key.shape[1] == 0 or key.shape[2] == 0


def _as_kernel_layout(t: Array) -> Array:
    """The kernels read 16-byte chunks along a contiguous feature axis: anything else (a transposed feature axis, a
    view that starts in the middle of a row) is copied once."""
    if t.stride(-1) != 1:
        t = t.contiguous()
    if t.data_ptr() % 16 != 0 or (not t.is_contiguous() and any(s % 8 != 0 for s in t.stride()[:-1])):
        t = t.clone(memory_format=torch.contiguous_format)
    return t


def _pad_head_dims(q: Array, k: Array, v: Array, kernel_options) -> Tuple[Array, Array, Array]:
    """The matrix-core kernels exist for D = Dv in {64, 128} and, for 16-bit inputs, {192, 256}.  Other head sizes
    up to the largest of those (and Dv < D) are zero-padded to the next one: zero feature columns add nothing to
    Q.K^T, the padded columns of O are dropped by the caller and the padded columns of the gradients are cut off
    by autograd, so the result is the one of the original problem at matrix-core speed.  Opt out with
    kernel_options={"pad_head_dim": False}; the faithful and the generic kernels take any size as it is."""
    opts = kernel_options or {}
    D, Dv = q.shape[-1], v.shape[-1]
    if (q.dtype not in (torch.float16, torch.bfloat16, torch.float32) or opts.get("strict", False)
            or opts.get("backend", "auto") == "generic" or not opts.get("pad_head_dim", True)):
        return q, k, v
    sizes = (64, 128) if q.dtype == torch.float32 else (64, 128, 192, 256)
    Dp = next((s for s in sizes if max(D, Dv) <= s), None)
    if Dp is None or (D == Dp and Dv == Dp):
        return q, k, v
    pad = torch.nn.functional.pad
    return pad(q, (0, Dp - D)), pad(k, (0, Dp - D)), pad(v, (0, Dp - Dv))


def math_attention(query: Array, key: Array, value: Array, score_mod: Callable, block_mask: Tuple, scale: float,
                   kernel_options: Dict[str, Any], score_mod_other_buffers: Tuple = (),
                   mask_mod_other_buffers: Tuple = (), use_pallas: bool = False) -> Tuple[Array, Array]:
    """attention.py:67-106: (output, base-2 logsumexp).  ``block_mask`` is the
    tuple BlockMask.as_tuple() gives; only its last entry (the mask_mod) is
    read, as in the reference (attention.py:45).  Runs the faithful kernels.
    ``score_mod_other_buffers`` / ``mask_mod_other_buffers`` are handed to the mods as
    trailing arguments (attention.py:22-23, 36-44)."""
    mask_mod = block_mask[-1]
    if score_mod_other_buffers:
        inner_score, sbufs = score_mod, tuple(score_mod_other_buffers)
        score_mod = lambda score, b, h, q_idx, kv_idx: inner_score(score, b, h, q_idx, kv_idx, *sbufs)  # noqa: E731
    if mask_mod_other_buffers:
        inner_mask, mbufs = mask_mod, tuple(mask_mod_other_buffers)
        mask_mod = lambda b, h, q_idx, kv_idx: inner_mask(b, h, q_idx, kv_idx, *mbufs)  # noqa: E731
    _require_device(query, key, value)
    q, k, v = map(_as_kernel_layout, (query, key, value))
    opts = dict(kernel_options or {})
    opts.setdefault("strict", True)
    try:
        plan = _make_plan(q, k, v, score_mod, None, mask_mod, scale, opts)
    except ScoreModNotLowered:
        return _attend_linearised(q, k, v, score_mod, None, mask_mod, scale, opts)
    return _attend(plan, q, k, v)


def flax_attention(query: Array, key: Array, value: Array, score_mod: Optional[_score_mod_signature] = None,
                   block_mask: Optional[BlockMask] = None, scale: Optional[float] = None, enable_gqa: bool = False,
                   return_lse: bool = False, kernel_options: Optional[Dict[str, Any]] = None
                   ) -> Union[Array, Tuple[Array, Array]]:
    """attention.py:169-218."""
    _validate_sdpa_input(query, key, value)
    _validate_embed_dim(query, key, value)
    if query.dim() != 4 or key.dim() != 4 or value.dim() != 4:
        raise NotImplementedError("NYI: query, key, and value must be 4D tensors")
    if (not enable_gqa) and query.shape[-3] != key.shape[-3]:
        raise ValueError(
            f"Expect query and key/value to have the same number of heads "
            f"but got Hq={query.shape[-3]} and Hkv={key.shape[-3]}. "
            f"Try setting enable_gqa=True for GQA."
        )
    if enable_gqa:
        Hq = query.shape[1]
        Hkv = key.shape[1]
        if Hq % Hkv != 0:
            raise ValueError(
                f"Expect number of query heads to be a multiple of kv heads for GQA "
                f"but got Hq={Hq} and Hkv={Hkv}."
            )
    _require_device(query, key, value)
    if _nothing_to_attend(query, key):
        out, lse2 = _NothingToAttend.apply(query, key, value)
        return (out, lse2) if return_lse else out
    if score_mod is None:
        score_mod = _identity
    if block_mask is None:
        block_mask = _create_empty_block_mask(query, key)
    if scale is None:
        scale = 1.0 / math.sqrt(query.shape[-1])
    q, k, v = map(_as_kernel_layout, _pad_head_dims(query, key, value, kernel_options))
    try:
        plan = _plan_for(q, k, v, score_mod, block_mask, None, scale, kernel_options)
        out, lse2 = _attend(plan, q, k, v)
    except ScoreModNotLowered:
        out, lse2 = _attend_linearised(q, k, v, score_mod, block_mask, None, scale, kernel_options)
    out = out[..., :value.shape[-1]]
    if return_lse:
        return out, lse2 * math.log(2.0)
    return out


_FAMILIES = {0: "generic", 1: "mfma_16bit", 2: "mfma_f32"}


def kernel_family(query: Array, key: Array, value: Array, score_mod: Optional[_score_mod_signature] = None,
                  block_mask: Optional[BlockMask] = None, scale: Optional[float] = None,
                  kernel_options: Optional[Dict[str, Any]] = None, backward: bool = False) -> str:
    """Which kernels flax_attention runs for these inputs: "generic" (vector ALU), "mfma_16bit" or "mfma_f32"
    (matrix cores).  Asks the library (flexattn_kernel_family) with the parameters the call itself would pass: the
    score_mod and the mask are lowered and the mask's tile lists built as the call would, no attention is computed.
    No counterpart in the reference, which has one dense path (core/attention.py:14-106)."""
    _require_device(query, key, value)
    if score_mod is None:
        score_mod = _identity
    if block_mask is None:
        block_mask = _create_empty_block_mask(query, key)
    if scale is None:
        scale = 1.0 / math.sqrt(query.shape[-1])
    q, k, v = map(_as_kernel_layout, _pad_head_dims(query, key, value, kernel_options))
    try:
        plan = _make_plan(q, k, v, score_mod, block_mask, None, scale, kernel_options)
    except ScoreModNotLowered:
        # linearised at the scores of the call: dense multiplicative and additive tables (FLEX_SCORE_AFFINE)
        opts = dict(kernel_options or {})
        opts["tile_lists"] = opts.get("tile_lists", True)
        plan = _make_plan(q, k, v, _identity, block_mask, None, scale, opts)
        plan.score = ScoreMod(_lib.SCORE_AFFINE, mul=torch.ones((1, 1, 1, 1), device=q.device), add=None)
    o_like = torch.empty((q.shape[0], q.shape[1], q.shape[2], v.shape[3]), dtype=q.dtype, device="meta")
    p = plan.params(q, k, v, o_like)
    return _FAMILIES[_lib.lib().flexattn_kernel_family(_lib.C.byref(p), 1 if backward else 0)]


def flax_attention_pallas(query: Array, key: Array, value: Array, score_mod: Optional[_score_mod_signature] = None,
                          mask_mod: Optional[_mask_mod_signature] = None, block_q: int = 64, block_k: int = 64,
                          sm_scale: Optional[float] = None, bhln: bool = True, enable_gqa: bool = False,
                          block_mask: Optional[BlockMask] = None, block_mod: Optional[_mask_mod_signature] = None,
                          kernel_options: Optional[Dict[str, Any]] = None) -> Array:
    """attention.py:220-312: the fused-kernel front-end.  ``bhln=True`` takes
    [B,H,L,D]; ``bhln=False`` takes [B,L,H,D] (read in place through strides).
    ``block_q`` / ``block_k`` are accepted for compatibility; tile shapes are
    chosen by the kernels.  ``block_mask=`` (a BlockMask) and the README's
    spelling ``block_mod=`` are accepted next to ``mask_mod=``.  Unlike the
    reference kernel (kernel/attention.py:233-235 indexes K/V with the q-head
    id) GQA works here."""
    if block_mod is not None:
        if mask_mod is not None:
            raise ValueError("pass only one of mask_mod= and block_mod=")
        mask_mod = block_mod
    if not bhln:
        query, key, value = (t.transpose(1, 2) for t in (query, key, value))
    _validate_sdpa_input(query, key, value)
    _validate_embed_dim(query, key, value)
    if query.dim() != 4 or key.dim() != 4 or value.dim() != 4:
        raise NotImplementedError("NYI: query, key, and value must be 4D tensors")
    if (not enable_gqa) and query.shape[1] != key.shape[1]:
        raise ValueError(
            f"Expect query and key/value to have the same number of heads "
            f"but got Hq={query.shape[1]} and Hkv={key.shape[1]}. "
            f"Try setting enable_gqa=True for GQA."
        )
    if enable_gqa:
        Hq, Hkv = query.shape[1], key.shape[1]
        if Hq % Hkv != 0:
            raise ValueError(
                f"Expect number of query heads to be a multiple of kv heads for GQA "
                f"but got Hq={Hq} and Hkv={Hkv}."
            )
    _require_device(query, key, value)
    if sm_scale is None:
        sm_scale = 1 / math.sqrt(query.shape[-1])
    if block_mask is not None and mask_mod is not None:
        raise ValueError("pass only one of block_mask= and mask_mod=")
    if _nothing_to_attend(query, key):
        out, _ = _NothingToAttend.apply(query, key, value)
        return out if bhln else out.transpose(1, 2)
    q, k, v = map(_as_kernel_layout, _pad_head_dims(query, key, value, kernel_options))
    try:
        plan = _plan_for(q, k, v, score_mod, block_mask, mask_mod, sm_scale, kernel_options)
        out, _ = _attend(plan, q, k, v)
    except ScoreModNotLowered:
        out, _ = _attend_linearised(q, k, v, score_mod, block_mask, mask_mod, sm_scale, kernel_options)
    out = out[..., :value.shape[-1]]
    return out if bhln else out.transpose(1, 2)
