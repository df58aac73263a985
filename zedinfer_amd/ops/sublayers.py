"""Checked launches of the kernels behind sublayers that the first architectures do not have: the layer norm (alone,
or on a sublayer's output with the residual addition), what stands between a q/k/v projection with a short
convolution and attention, the router that takes the largest logits, the feed-forward activations without a SiLU
gate, the soft cap of logits, and a conversion between storage types."""
from __future__ import annotations

from typing import Optional

import torch

from . import _lib
from .functional import _check_cache, _code, _gpu, _i32, _p, _rows, _stream
from .mixing import MOE_MAX_EXPERTS, _f32

CONV_MAX_TAPS = 16
CONV_MAX_CHANNELS = 15360


def _terms(x: torch.Tensor, what: str):
    """(splits, stride between splits, row stride, rows, width) of [n, H] rows or a stack [S, n, H] of float32 terms."""
    if x.dim() == 3:
        if x.dtype != torch.float32 or not x.is_contiguous():
            raise ValueError(f"{what}: a stack of terms must be contiguous float32 [S, n, width]")
        return int(x.shape[0]), int(x.shape[1] * x.shape[2]), int(x.shape[2]), int(x.shape[1]), int(x.shape[2])
    ld, width = _rows(x, what)
    return 1, 0, ld, int(x.shape[0]), width


def layer_norm(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float,
               out: Optional[torch.Tensor] = None, out_dtype: Optional[torch.dtype] = None,
               resid: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """y = (x - mean) / sqrt(mean((x - mean)^2) + eps) * weight + bias over the rows of x [n, H], in float32; x may be
    a stack [S, n, H] of float32 terms, added in rising order first.  With ``resid`` (float32 [n, H], changed in
    place): resid += y, and ``out`` (optional then) receives the new residual rows in its own type.  Without
    ``resid``: ``out`` receives y."""
    _gpu("layer_norm", x, weight, bias, out, resid)
    splits, split_stride, ldx, n, H = _terms(x, "layer_norm x")
    for name, t in (("weight", weight), ("bias", bias)):
        if t.dim() != 1 or t.numel() != H or not t.is_contiguous() or t.dtype != weight.dtype:
            raise ValueError(f"layer_norm: {name} must be a contiguous [{H}] tensor, gain and bias of one type")
    if resid is not None and (resid.dtype != torch.float32 or tuple(resid.shape) != (n, H) or not resid.is_contiguous()):
        raise ValueError(f"layer_norm: the residual stream must be a contiguous float32 [{n}, {H}] tensor")
    if out is None and resid is None:
        out = torch.empty((n, H), dtype=out_dtype or (x.dtype if x.dim() == 2 else torch.float32), device=x.device)
    ldo = 0
    if out is not None:
        ldo, Ho = _rows(out, "layer_norm out")
        if tuple(out.shape) != (n, H):
            raise ValueError("layer_norm: out has the wrong shape")
    if not eps > 0:
        raise ValueError("layer_norm: eps must be positive")
    _lib.call("zi_layer_norm", _p(out), _code(out, "layer_norm out") if out is not None else 0, ldo, _p(resid), _p(x),
              _code(x, "layer_norm x"), splits, split_stride, ldx, _p(weight), _p(bias), _code(weight, "layer_norm weight"),
              n, H, float(eps), _stream())
    return out


def conv_state_floats(channels: int, taps: int) -> int:
    """Floats of a request's state for a convolution of ``taps`` taps over ``channels`` channels: its last
    taps - 1 input rows (at least one float, so that the slot exists)."""
    return max(1, (int(taps) - 1) * int(channels))


def conv_qkv(proj: torch.Tensor, bias: Optional[torch.Tensor], conv_w: torch.Tensor, state: torch.Tensor,
             q_norm: torch.Tensor, k_norm: torch.Tensor, eps: float, table: Optional[torch.Tensor], tok_seq: torch.Tensor,
             entry_start: torch.Tensor, entry_slot: torch.Tensor, slots: Optional[torch.Tensor],
             kcache: Optional[torch.Tensor], vcache: Optional[torch.Tensor], nh: int, nkv: int, dim: int, vdim: int,
             head: int, taps: int, q_out: torch.Tensor, move_tail: bool = False) -> torch.Tensor:
    """Rows of proj [n, nh*dim + nkv*dim + nkv*vdim] (q | k | v, any storage type, or a stack [S, n, ...] of float32
    partial sums) plus ``bias`` pass, per channel, a
    causal convolution of ``taps`` taps (``conv_w`` [channels, taps]; rows before the step come from the request's
    tail in ``state`` [slots, >= (taps-1) * channels]), q and k an RMS norm over all their channels at once (gains
    ``q_norm`` / ``k_norm``), and a split-half rotation of the first R dims of every head by ``table`` [n, R/2, 2].
    The queries go to ``q_out`` [n, nh*head]; keys and values, where the caches are given, into the paged cache at
    ``slots`` (a token whose slot is negative stores nothing), whose heads hold ``head`` >= dim, vdim values (the
    rest zero).  ``move_tail`` (only when every entry brings one token): the new tails are written here too, for
    tokens that have a slot, and ``conv_tail`` is not needed.  Everything float32 but the stores."""
    _gpu("conv_qkv", proj, bias, conv_w, state, q_norm, k_norm, table, tok_seq, entry_start, entry_slot, slots, kcache,
         vcache, q_out)
    splits, split_stride, ld, n, width = _terms(proj, "conv_qkv proj")
    Qd, Kd, Vd = nh * dim, nkv * dim, nkv * vdim
    C = Qd + Kd + Vd
    if width != C:
        raise ValueError(f"conv_qkv: proj must be [n, {C}], got width {width}")
    if not (1 <= taps <= CONV_MAX_TAPS) or C > CONV_MAX_CHANNELS:
        raise ValueError(f"conv_qkv: at most {CONV_MAX_TAPS} taps and {CONV_MAX_CHANNELS} channels ({taps}, {C})")
    _f32(conv_w, "conv_qkv conv_w", (C, taps))
    _f32(q_norm, "conv_qkv q_norm", (Qd,))
    _f32(k_norm, "conv_qkv k_norm", (Kd,))
    if bias is not None:
        _f32(bias, "conv_qkv bias", (C,))
    if state.dtype != torch.float32 or state.dim() != 2 or not state.is_contiguous() or state.shape[1] < (taps - 1) * C:
        raise ValueError(f"conv_qkv: state must be contiguous float32 [slots, >= {(taps - 1) * C}]")
    rot = 0
    if table is not None:
        _f32(table, "conv_qkv table")
        if table.dim() != 3 or table.shape[0] != n or table.shape[2] != 2 or 2 * table.shape[1] > dim:
            raise ValueError("conv_qkv: the table must be [n, R/2, 2] with R within the head")
        rot = 2 * int(table.shape[1])
    _i32(tok_seq, "conv_qkv tok_seq", n)
    _i32(entry_start, "conv_qkv entry_start")
    _i32(entry_slot, "conv_qkv entry_slot", entry_start.numel())
    ldq, wq = _rows(q_out, "conv_qkv q_out")
    if tuple(q_out.shape) != (n, nh * head) or head < max(dim, vdim):
        raise ValueError(f"conv_qkv: q_out must be [n, {nh * head}] with heads of at least {max(dim, vdim)} values")
    pages = ps = 0
    if slots is not None:
        _i32(slots, "conv_qkv slots", n)
    if kcache is not None:
        if slots is None:
            raise ValueError("conv_qkv: a cache needs the tokens' slots")
        pages, ps = _check_cache(kcache, vcache, nkv, head, q_out.dtype, "conv_qkv")
    if move_tail and slots is None:
        raise ValueError("conv_qkv: moving the tail needs the tokens' slots")
    _lib.call("zi_conv_qkv", _p(q_out), _code(q_out, "conv_qkv q_out"), ldq, _p(kcache),
              _p(vcache if kcache is not None else None), _p(proj), _code(proj, "conv_qkv proj"), ld, splits, split_stride,
              _p(bias), _p(conv_w), _p(state), int(state.stride(0)), int(bool(move_tail)), _p(q_norm), _p(k_norm),
              float(eps), _p(table), rot, n, _p(tok_seq),
              _p(entry_start), _p(entry_slot), _p(slots), pages * ps, nh, nkv, dim, vdim, head, taps, max(ps, 1), _stream())
    return q_out


def conv_tail(state: torch.Tensor, proj: torch.Tensor, bias: Optional[torch.Tensor], entry_start: torch.Tensor,
              entry_len: torch.Tensor, entry_slot: torch.Tensor, taps: int, slots: Optional[torch.Tensor] = None) -> None:
    """After ``conv_qkv`` has read the old tails: the last taps - 1 rows of proj + bias of every entry's sequence so
    far become the new tail in the entry's state slot.  With ``slots`` (every token's place in the cache) the tokens
    that have none (negative; they stand behind an entry's own) do not count, and an entry without any token of its
    own leaves its slot's tail as it is."""
    _gpu("conv_tail", state, proj, bias, entry_start, entry_len, entry_slot, slots)
    splits, split_stride, ld, n, C = _terms(proj, "conv_tail proj")
    if slots is not None:
        _i32(slots, "conv_tail slots", n)
    if state.dtype != torch.float32 or state.dim() != 2 or not state.is_contiguous() or state.shape[1] < (taps - 1) * C:
        raise ValueError(f"conv_tail: state must be contiguous float32 [slots, >= {(taps - 1) * C}]")
    if bias is not None:
        _f32(bias, "conv_tail bias", (C,))
    E = entry_start.numel()
    for name, t in (("entry_start", entry_start), ("entry_len", entry_len), ("entry_slot", entry_slot)):
        _i32(t, f"conv_tail {name}", E)
    if not (1 <= taps <= CONV_MAX_TAPS):
        raise ValueError(f"conv_tail: at most {CONV_MAX_TAPS} taps")
    _lib.call("zi_conv_tail", _p(state), int(state.stride(0)), _p(proj), _code(proj, "conv_tail proj"), ld, splits,
              split_stride, _p(bias),
              _p(entry_start), _p(entry_len), _p(entry_slot), _p(slots), E, C, taps, _stream())


def relu_squared(z: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out = relu(z)^2, z [n, I] with dense rows or a stack [S, n, I] of float32 partial sums."""
    _gpu("relu_squared", z, out)
    splits, split_stride, ldz, n, I = _terms(z, "relu_squared z")
    ldo, Io = _rows(out, "relu_squared out")
    if tuple(out.shape) != (n, I):
        raise ValueError("relu_squared: out has the wrong shape")
    _lib.call("zi_relu_squared", _p(out), _code(out, "relu_squared out"), ldo, _p(z), _code(z, "relu_squared z"), ldz,
              splits, split_stride, n, I, _stream())
    return out


def clamped_glu(gate: torch.Tensor, up: torch.Tensor, limit: float, out: torch.Tensor, alpha: float = 1.702) -> torch.Tensor:
    """out = g sigmoid(alpha g) (u + 1) with g = min(gate, limit), u = clamp(up, -limit, limit); gate and up [n, I]
    with dense rows (column slices of one product are fine), or the same slices [S, n, I] of a stack of float32 partial
    sums, which are added first."""
    _gpu("clamped_glu", gate, up, out)
    splits, split_stride = 1, 0
    if gate.dim() == 3:
        if gate.dtype != torch.float32 or up.dtype != torch.float32 or gate.shape != up.shape or gate.stride() != up.stride() \
                or gate.stride(2) != 1:
            raise ValueError("clamped_glu: stacks of partial sums must be float32 slices of one stack")
        splits, split_stride = int(gate.shape[0]), int(gate.stride(0))
        gate, up = gate[0], up[0]
    ldg, I = _rows(gate, "clamped_glu gate")
    ldu, Iu = _rows(up, "clamped_glu up")
    ldo, Io = _rows(out, "clamped_glu out")
    n = gate.shape[0]
    if gate.dtype != up.dtype or I != Iu or I != Io or up.shape[0] != n or out.shape[0] != n:
        raise ValueError("clamped_glu: gate, up and out must agree in shape, gate and up in type")
    if not limit > 0:
        raise ValueError("clamped_glu: the limit must be positive")
    _lib.call("zi_clamped_glu", _p(out), _code(out, "clamped_glu out"), ldo, _p(gate), _p(up), _code(gate, "clamped_glu"),
              ldg, ldu, splits, split_stride, n, I, float(limit), float(alpha), _stream())
    return out


def softcap(x: torch.Tensor, cap: float) -> torch.Tensor:
    """In place: x <- cap * tanh(x / cap) for a contiguous float32 tensor."""
    _gpu("softcap", x)
    if x.dtype != torch.float32 or not x.is_contiguous() or not cap > 0:
        raise ValueError("softcap: a contiguous float32 tensor and a positive cap")
    _lib.call("zi_softcap", _p(x), x.numel(), float(cap), _stream())
    return x


def convert(x: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out = x in out's storage type (both contiguous, of one shape)."""
    _gpu("convert", x, out)
    if x.shape != out.shape or not x.is_contiguous() or not out.is_contiguous():
        raise ValueError("convert: x and out must be contiguous and of one shape")
    _lib.call("zi_convert", _p(out), _code(out, "convert out"), _p(x), _code(x, "convert x"), x.numel(), _stream())
    return out


def moe_route_top(z: torch.Tensor, bias: Optional[torch.Tensor], top: int, idx: torch.Tensor, wt: torch.Tensor) -> None:
    """z [n, E] float32 router logits (plus ``bias`` [E], float32): the ``top`` largest of every row (the lowest
    index among equals) into ``idx`` [n, top], the softmax over those chosen logits into ``wt``."""
    _gpu("moe_route_top", z, bias, idx, wt)
    _f32(z, "moe_route_top z")
    n, E = z.shape
    if bias is not None:
        _f32(bias, "moe_route_top bias", (E,))
    _f32(wt, "moe_route_top wt", (n, top))
    _i32(idx, "moe_route_top idx", n * top)
    if not (0 < top <= E <= MOE_MAX_EXPERTS):
        raise ValueError(f"moe_route_top: top {top} of {E} experts (at most {MOE_MAX_EXPERTS})")
    _lib.call("zi_moe_route_top", _p(idx), _p(wt), _p(z), _p(bias), n, E, top, _stream())
