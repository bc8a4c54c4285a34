"""Gated linear recurrence with a matrix state per head — HGRN2 (csrc/gated_recurrence.hip, libhydra_mix.so):
    f = low + (1 - low) * sigmoid(f_pre + f_bias),  S <- diag(f) S + (1 - f) v^T,  o = S^T silu(q_pre),
    out = o / sqrt(mean(o^2) + eps) * norm_w   over each head's value channels.
The state S [heads, dim, vdim] of a sequence lives in float32 in its state slot between steps; a portion that starts at
position 0 starts from zeros without reading the slot."""
import torch
from torch import Tensor

from hydrainfer_amd import _lib
from hydrainfer_amd._C.kernel.stream_ops import SequenceState


def gated_recurrence(q_pre: Tensor, f_pre: Tensor, v: Tensor, f_bias: Tensor, low: Tensor, norm_w: Tensor, eps: float,
                     seq: SequenceState, state_row: int, q_cu: Tensor, positions: Tensor, heads: int, dim: int,
                     vdim: int, max_q_len: int = 0) -> Tensor:
    """q_pre, f_pre: [n_tokens, heads * dim]; v: [n_tokens, heads * vdim] (views of one projection will do: contiguous rows).
    seq.state: float32 [n_slots, n_rows, >= heads * dim * vdim]; this layer's state is row `state_row` of a slot.
    max_q_len: the longest portion of the batch when known (1: every sequence brings one token — a decode step's kernel).
    Returns [n_tokens, heads * vdim] in the inputs' dtype."""
    _lib.require_gpu(q_pre, f_pre, v, f_bias, low, norm_w, seq.state, seq.slots, q_cu, positions)
    T = q_pre.shape[0]
    dt = q_pre.dtype
    if dt not in (torch.float32, torch.bfloat16):
        raise _lib.HydraHipError(f"gated_recurrence: activations are float32 or bfloat16, not {dt}")
    for t, n, name in ((q_pre, heads * dim, "q_pre"), (f_pre, heads * dim, "f_pre"), (v, heads * vdim, "v")):
        if t.dim() != 2 or t.shape != (T, n) or t.stride(1) != 1 or t.dtype != dt:
            raise _lib.HydraHipError(f"gated_recurrence: {name} must be [n_tokens, {n}] with contiguous rows, one dtype")
    for t, n, name in ((f_bias, heads * dim, "f_bias"), (low, heads * dim, "low"), (norm_w, vdim, "norm_w")):
        if t.dtype != torch.float32 or not t.is_contiguous() or t.numel() != n:
            raise _lib.HydraHipError(f"gated_recurrence: {name} must be contiguous float32 [{n}]")
    st = seq.state
    if st.dtype != torch.float32 or st.dim() != 3 or not st.is_contiguous() or st.shape[2] < heads * dim * vdim or \
            not 0 <= state_row < st.shape[1]:
        raise _lib.HydraHipError("gated_recurrence: state must be contiguous float32 [n_slots, rows, >= heads * dim * vdim]")
    n_seq = q_cu.numel() - 1
    for t, n, name in ((q_cu, n_seq + 1, "q_cu"), (positions, T, "positions"), (seq.slots, n_seq, "slots")):
        if t.dtype != torch.int32 or not t.is_contiguous() or t.numel() != n:
            raise _lib.HydraHipError(f"gated_recurrence: {name} must be contiguous int32 [{n}]")
    out = torch.empty((T, heads * vdim), dtype=dt, device=q_pre.device)
    base = st.data_ptr() + 4 * state_row * st.stride(1)
    n_ws = _lib.mix_lib().hxm_gated_recurrence_workspace(T, int(heads), int(dim), int(vdim))
    ws = torch.empty(max(n_ws, 1), dtype=torch.float32, device=q_pre.device)      # partial results of the key channels' parts
    _lib.mix_check(_lib.mix_lib().hxm_gated_recurrence(
        out.data_ptr(), q_pre.data_ptr(), q_pre.stride(0), f_pre.data_ptr(), f_pre.stride(0), v.data_ptr(), v.stride(0),
        f_bias.data_ptr(), low.data_ptr(), norm_w.data_ptr(), float(eps), base, st.stride(0), q_cu.data_ptr(),
        positions.data_ptr(), seq.slots.data_ptr(), n_seq, T, int(heads), int(dim), int(vdim), int(max_q_len), ws.data_ptr(), n_ws,
        _lib._DTYPE[dt], _lib.current_stream()), "gated_recurrence")
    return out
