"""Multi-stream residuals (hyper-connections), grouped RMS norm, token shift, gated sublayer results and the tanh-GELU
gate: the row kernels of csrc/stream_ops.hip (libhydra_mix.so).

The residual is a float tensor x [n_tokens, n_streams, width]; a sublayer reads `stream_norm` of it and writes back
through `stream_update`.  One stream with in = mix = out = 1 is the ordinary pre-norm residual.  Activations (what the
matrix products read and write) are float32 or bfloat16."""
from dataclasses import dataclass
from typing import Optional

import torch
from torch import Tensor

from hydrainfer_amd import _lib


def _ptr(t: Optional[Tensor]):
    return None if t is None else t.data_ptr()


def _f32(t: Optional[Tensor], name: str) -> None:
    if t is not None and (t.dtype != torch.float32 or not t.is_contiguous()):
        raise _lib.HydraHipError(f"{name} must be a contiguous float32 tensor")


def _act_code(dtype: torch.dtype) -> int:
    if dtype not in (torch.float32, torch.bfloat16):
        raise _lib.HydraHipError(f"stream ops: activations are float32 or bfloat16, not {dtype}")
    return _lib._DTYPE[dtype]


@dataclass
class SequenceState:
    """Where the rows that a sequence carries from one step to the next live, and which sequences a batch holds.
    state: float32 [n_slots, n_rows_per_slot, width] (memory.state_slots.StateSlotManager); slots: int32 [n_seq];
    tok_seq: int32 [n_tokens] sequence of each token of the batch."""
    state: Tensor
    slots: Tensor
    tok_seq: Tensor


def stream_embed(ids: Tensor, table: Tensor, scale: float, n_streams: int) -> Tensor:
    """x[t, s, :] = table[ids[t]] * scale for every stream s (float32)."""
    _lib.require_gpu(ids, table)
    if ids.dim() != 1 or ids.dtype not in (torch.int32, torch.int64) or not ids.is_contiguous():
        raise _lib.HydraHipError("stream_embed: ids must be a contiguous 1-D int32 / int64 tensor")
    if table.dim() != 2 or not table.is_contiguous():
        raise _lib.HydraHipError("stream_embed: table must be contiguous [vocab, width]")
    x = torch.empty((ids.shape[0], n_streams, table.shape[1]), dtype=torch.float32, device=table.device)
    _lib.mix_check(_lib.mix_lib().hxm_stream_embed(
        x.data_ptr(), table.data_ptr(), ids.data_ptr(), 1 if ids.dtype == torch.int64 else 0, float(scale), ids.shape[0],
        int(n_streams), table.shape[1], table.shape[0], _act_code(table.dtype), _lib.current_stream()), "stream_embed")
    return x


def stream_norm(x: Tensor, in_w: Tensor, norm_w: Tensor, groups: int, eps: float, dtype: torch.dtype,
                rows: Optional[Tensor] = None, shift_w: Optional[Tensor] = None, seq: Optional[SequenceState] = None,
                state_row: int = 0, q_cu: Optional[Tensor] = None, positions: Optional[Tensor] = None,
                want_plain: bool = True):
    """h = grouped_rms_norm(sum_s in_w[s] x[:, s, :]) * norm_w.  Without shift_w: returns h [n_out, width] (`rows`
    selects rows of x).  With shift_w: returns (h or None, hs) with hs = h + (h_prev - h) * shift_w, h_prev the h of
    the token before in the same sequence — across steps through row `state_row` of the sequence's state slot, which
    is left holding the h of the sequence's last token of this batch."""
    _lib.require_gpu(x, in_w, norm_w, rows, shift_w)
    _f32(x, "x"); _f32(in_w, "in_w"); _f32(norm_w, "norm_w"); _f32(shift_w, "shift_w")
    if x.dim() != 3 or in_w.numel() != x.shape[1] or norm_w.numel() != x.shape[2]:
        raise _lib.HydraHipError("stream_norm: x [n_tokens, n_streams, width], in_w [n_streams], norm_w [width]")
    T, S, W = x.shape
    n_out = T if rows is None else rows.numel()
    if rows is not None and (rows.dtype != torch.int32 or not rows.is_contiguous()):
        raise _lib.HydraHipError("stream_norm: rows must be contiguous int32")
    code = _act_code(dtype)
    h = torch.empty((n_out, W), dtype=dtype, device=x.device) if (want_plain or shift_w is None) else None
    hs = None
    args_state = [None, 0, None, None, None, None]
    if shift_w is not None:
        if seq is None or q_cu is None or positions is None or rows is not None:
            raise _lib.HydraHipError("stream_norm: the token shift needs the batch's sequences (seq, q_cu, positions) and all rows")
        st = seq.state
        if st.dtype != torch.float32 or st.dim() != 3 or st.shape[2] != W or not st.is_contiguous() or not 0 <= state_row < st.shape[1]:
            raise _lib.HydraHipError("stream_norm: state must be contiguous float32 [n_slots, rows, width]")
        for t, name, n in ((seq.slots, "slots", q_cu.numel() - 1), (seq.tok_seq, "tok_seq", T), (q_cu, "q_cu", q_cu.numel()),
                           (positions, "positions", T)):
            if t.dtype != torch.int32 or not t.is_contiguous() or t.numel() != n:
                raise _lib.HydraHipError(f"stream_norm: {name} must be contiguous int32 [{n}]")
        _lib.require_gpu(st, seq.slots, seq.tok_seq, q_cu, positions)
        hs = torch.empty((T, W), dtype=dtype, device=x.device)
        args_state = [st.data_ptr() + state_row * W * 4, st.shape[1] * W, seq.tok_seq.data_ptr(), q_cu.data_ptr(),
                      positions.data_ptr(), seq.slots.data_ptr()]
    _lib.mix_check(_lib.mix_lib().hxm_stream_norm(
        x.data_ptr(), in_w.data_ptr(), norm_w.data_ptr(), int(groups), float(eps), _ptr(rows), n_out, S, W, _ptr(h),
        _ptr(shift_w), _ptr(hs), *args_state, code, _lib.current_stream()), "stream_norm")
    return h if shift_w is None else (h, hs)


def stream_update(x: Tensor, y: Tensor, mix: Tensor, out_w: Tensor, gate_pre: Optional[Tensor] = None,
                  gate_b: Optional[Tensor] = None) -> None:
    """In place: x[:, t, :] <- sum_s mix[s, t] x[:, s, :] + out_w[t] * y * sigmoid(gate_pre + gate_b) (no gate_pre: * 1)."""
    _lib.require_gpu(x, y, mix, out_w, gate_pre, gate_b)
    _f32(x, "x"); _f32(mix, "mix"); _f32(out_w, "out_w"); _f32(gate_b, "gate_b")
    T, S, W = x.shape
    if y.dim() != 2 or y.shape[0] != T or y.shape[1] < W or y.stride(1) != 1:
        raise _lib.HydraHipError("stream_update: y must be [n_tokens, >= width] with a contiguous last dimension")
    if gate_pre is not None and (gate_pre.dtype != y.dtype or gate_pre.dim() != 2 or gate_pre.shape[0] != T
                                 or gate_pre.shape[1] < W or gate_pre.stride(1) != 1):
        raise _lib.HydraHipError("stream_update: gate_pre must look like y")
    if mix.numel() != S * S or out_w.numel() != S or (gate_b is not None and gate_b.numel() != W):
        raise _lib.HydraHipError("stream_update: mix [n_streams, n_streams], out_w [n_streams], gate_b [width]")
    _lib.mix_check(_lib.mix_lib().hxm_stream_update(
        x.data_ptr(), y.data_ptr(), y.stride(0), _ptr(gate_pre), gate_pre.stride(0) if gate_pre is not None else 0,
        _ptr(gate_b), mix.data_ptr(), out_w.data_ptr(), T, S, W, _act_code(y.dtype), _lib.current_stream()), "stream_update")


def stream_update_norm(x: Tensor, y: Tensor, mix: Tensor, out_w: Tensor, gate_pre: Optional[Tensor], gate_b: Optional[Tensor],
                       in_next: Tensor, norm_next: Tensor, groups: int, eps: float) -> Tensor:
    """stream_update(x, y, mix, out_w, gate_pre, gate_b) and then stream_norm(x, in_next, norm_next, ...) of the next
    sublayer (one without a token shift), as one launch.  Returns h [n_tokens, width] of y's dtype."""
    _lib.require_gpu(x, y, mix, out_w, gate_pre, gate_b, in_next, norm_next)
    _f32(x, "x"); _f32(mix, "mix"); _f32(out_w, "out_w"); _f32(gate_b, "gate_b"); _f32(in_next, "in_next"); _f32(norm_next, "norm_next")
    T, S, W = x.shape
    if y.dim() != 2 or y.shape[0] != T or y.shape[1] < W or y.stride(1) != 1:
        raise _lib.HydraHipError("stream_update_norm: y must be [n_tokens, >= width] with a contiguous last dimension")
    if gate_pre is not None and (gate_pre.dtype != y.dtype or gate_pre.dim() != 2 or gate_pre.shape[0] != T
                                 or gate_pre.shape[1] < W or gate_pre.stride(1) != 1):
        raise _lib.HydraHipError("stream_update_norm: gate_pre must look like y")
    if mix.numel() != S * S or out_w.numel() != S or in_next.numel() != S or norm_next.numel() != W or \
            (gate_b is not None and gate_b.numel() != W):
        raise _lib.HydraHipError("stream_update_norm: mix [S, S], out_w / in_next [S], norm_next / gate_b [width]")
    h = torch.empty((T, W), dtype=y.dtype, device=x.device)
    _lib.mix_check(_lib.mix_lib().hxm_stream_update_norm(
        x.data_ptr(), y.data_ptr(), y.stride(0), _ptr(gate_pre), gate_pre.stride(0) if gate_pre is not None else 0,
        _ptr(gate_b), mix.data_ptr(), out_w.data_ptr(), in_next.data_ptr(), norm_next.data_ptr(), int(groups), float(eps),
        h.data_ptr(), T, S, W, _act_code(y.dtype), _lib.current_stream()), "stream_update_norm")
    return h


def gelu_tanh_and_mul(gate: Tensor, up: Tensor) -> Tensor:
    """gelu_tanh(gate) * up in one pass; gelu_tanh(z) = 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))."""
    _lib.require_gpu(gate, up)
    if gate.dim() != 2 or gate.shape != up.shape or gate.stride(1) != 1 or up.stride(1) != 1 or gate.dtype != up.dtype:
        raise _lib.HydraHipError("gelu_tanh_and_mul: gate/up must be 2-D, same shape and dtype, contiguous last dim")
    out = torch.empty(gate.shape, dtype=gate.dtype, device=gate.device)
    _lib.mix_check(_lib.mix_lib().hxm_gelu_tanh_and_mul(
        out.data_ptr(), gate.data_ptr(), up.data_ptr(), gate.shape[0], gate.shape[1], gate.stride(0), up.stride(0),
        _act_code(gate.dtype), _lib.current_stream()), "gelu_tanh_and_mul")
    return out
