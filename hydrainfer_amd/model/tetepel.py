"""Tetepel — a decoder-only language model made of mechanisms the Llama path does not have:

  * the residual is `streams` copies x_1 .. x_s (hyper-connections): a sublayer reads u = sum_s in[s] x_s and its result y
    enters every stream, x_t <- sum_s mix[s, t] x_s + out[t] y; the model's output is the sum of the streams;
  * norms are RMS norms over `groups` equal consecutive parts of the vector;
  * the mixer's input is shifted towards the previous token's, hs = h + (h_prev - h) * shift (h_prev is carried from step to
    step in a state slot of the sequence, one row per layer run);
  * a sublayer's result is gated by sigmoid(W_rg h + b) of its own (unshifted) input;
  * the mixer is attention through low-rank latents without positions: cq = norm(W_dq hs), q = W_uq cq; c = norm(W_dkv hs)
    is all a token leaves in the cache; per head k = W_uk c, v = W_uv c; softmax over a sliding window; every head's result
    is gated by sigmoid(W_g hs); W_o on the concatenated heads;
  * the feed-forward is W_down(gelu_tanh(W_gate h) * W_up h);
  * a span of layers can be run several times in a row with the same weights (every run has its own cache plane and its
    own state row);
  * logits = embed . norm(sum of the streams), the input embedding being embed[token] * scale.

Every size and constant comes from config.json (`TetepelShape.from_config`), every tensor from model.safetensors under
the names of `TetepelForCausalLM.from_state_dict`.  Residual streams, norms, shifts, gates, scores and softmax weights are
float; the matrix products run in the model's dtype (bfloat16 with float accumulation, or float32).

The compute path: library GEMMs (torch.matmul / bmm) and the kernels of libhydra_mix.so (_C.kernel.stream_ops,
_C.kernel.latent_attn).  The attention kernel works in the latent space: q~ = W_uk^T q per head (a batched GEMM), then
multi-query attention over the cached rows c, then o = W_uv (sum_j p_j c_j) (a batched GEMM) — keys and values are
never materialised.  The model plugs into the engine through the interface LlamaForCausalLM has: forward_hidden /
forward_logits / forward over (token ids, position ids, LanguageModelParameters)."""
import json
import math
import os
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch
from torch import Tensor

from hydrainfer_amd._C.kernel.latent_attn import latent_attention, latent_norm_cache
from hydrainfer_amd._C.kernel.stream_ops import (SequenceState, gelu_tanh_and_mul, stream_embed, stream_norm,
                                                  stream_update, stream_update_norm)

ARCHITECTURE = "Tetepel"


@dataclass
class LatentAttentionSpec:
    heads: int
    dim: int                      # query / key size per head
    vdim: int                     # value size per head
    kv_rank: int                  # the cached latent
    q_rank: int                   # the query's latent
    scale: float
    window: Optional[int] = None  # position i sees j with 0 <= i - j < window; None: every j <= i


@dataclass
class TetepelLayer:
    type: str
    mixer: LatentAttentionSpec
    ff: Optional[int]             # dense feed-forward size, None: the layer has no feed-forward


@dataclass
class TetepelShape:
    vocab_size: int
    hidden_size: int
    layers: List[TetepelLayer]
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    norm_eps: float = 1e-6
    norm_groups: int = 1
    streams: int = 1
    embedding_scale: float = 1.0
    run_order: List[int] = field(default_factory=list)     # the layer behind every layer run, loops unrolled
    max_position_embeddings: Optional[int] = None          # no positional table: sequences are as long as the cache allows

    def __post_init__(self):
        n = len(self.layers)
        if not (0 <= self.loop_start <= self.loop_stop <= n) or self.loop_times < 1:
            raise ValueError(f"loop {self.loop_start}..{self.loop_stop} x {self.loop_times} does not fit {n} layers")
        if self.hidden_size % self.norm_groups:
            raise ValueError("norm groups must divide the width")
        self.run_order = (list(range(self.loop_start)) + list(range(self.loop_start, self.loop_stop)) * self.loop_times
                          + list(range(self.loop_stop, n)))

    # what the engine's cache pool and parameter builders ask of a model's shape
    @property
    def num_hidden_layers(self) -> int:          # cache planes: one per layer RUN
        return len(self.run_order)

    @property
    def num_attention_heads(self) -> int:
        return max(l.mixer.heads for l in self.layers)

    @property
    def num_key_value_heads(self) -> int:        # one latent row per token
        return 1

    @property
    def head_dim(self) -> int:                   # width of a cache row: the widest latent
        return max(l.mixer.kv_rank for l in self.layers)

    @classmethod
    def from_config(cls, cfg: dict) -> "TetepelShape":
        if cfg.get("architecture") != ARCHITECTURE:
            raise ValueError(f"not a {ARCHITECTURE} configuration: {cfg.get('architecture')!r}")
        layers = []
        for i, l in enumerate(cfg["layers"]):
            if l["type"] != "latent_attention":
                raise ValueError(f"layer {i}: unknown mixer type {l['type']!r}")
            m = l["mixer"]
            mask = m.get("mask")
            mlp = l.get("mlp")
            if mlp is not None and mlp.get("kind", "dense") != "dense":
                raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
            layers.append(TetepelLayer(l["type"], LatentAttentionSpec(
                heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]), kv_rank=int(m["kv_rank"]),
                q_rank=int(m["q_rank"]), scale=float(m["scale"]),
                window=int(mask["size"]) if mask and mask.get("size") else None),
                ff=int(mlp["ff"]) if mlp is not None else None))
        loop = cfg.get("loop") or {}
        norm = cfg.get("norm") or {}
        return cls(vocab_size=int(cfg["vocab"]), hidden_size=int(cfg["width"]), layers=layers,
                   loop_start=int(loop.get("start", 0)), loop_stop=int(loop.get("stop", loop.get("start", 0))),
                   loop_times=int(loop.get("times", 1)), norm_eps=float(norm.get("eps", 1e-6)),
                   norm_groups=int(norm.get("groups", 1)), streams=int(cfg.get("streams", 1)),
                   embedding_scale=float((cfg.get("embedding") or {}).get("scale", 1.0)))

    def to_config(self) -> dict:
        return {"architecture": ARCHITECTURE, "vocab": self.vocab_size, "width": self.hidden_size,
                "streams": self.streams, "embedding": {"scale": self.embedding_scale},
                "norm": {"eps": self.norm_eps, "groups": self.norm_groups},
                "loop": {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times},
                "layers": [{"type": l.type,
                            "mixer": {"heads": l.mixer.heads, "dim": l.mixer.dim, "vdim": l.mixer.vdim,
                                      "kv_rank": l.mixer.kv_rank, "q_rank": l.mixer.q_rank, "scale": l.mixer.scale,
                                      "mask": {"size": l.mixer.window} if l.mixer.window else None},
                            "mlp": {"kind": "dense", "ff": l.ff} if l.ff else None} for l in self.layers]}


def tensor_shapes(shape: TetepelShape) -> Dict[str, tuple]:
    """Name -> shape of every tensor of a checkpoint of this shape (linear weights are [out, in])."""
    W, S = shape.hidden_size, shape.streams
    out = {"embed": (shape.vocab_size, W), "final.norm": (W,)}
    for i, l in enumerate(shape.layers):
        m, p = l.mixer, f"l{i}."
        out.update({p + "norm1": (W,), p + "mix.dq": (m.q_rank, W), p + "mix.dq.norm": (m.q_rank,),
                    p + "mix.uq": (m.heads * m.dim, m.q_rank), p + "mix.dkv": (m.kv_rank, W),
                    p + "mix.dkv.norm": (m.kv_rank,), p + "mix.uk": (m.heads * m.dim, m.kv_rank),
                    p + "mix.uv": (m.heads * m.vdim, m.kv_rank), p + "mix.g": (m.heads, W),
                    p + "mix.o": (W, m.heads * m.vdim), p + "shift": (W,), p + "rg1": (W, W), p + "rg1.b": (W,),
                    p + "hc1.in": (S,), p + "hc1.out": (S,), p + "hc1.mix": (S, S)})
        if l.ff:
            out.update({p + "norm2": (W,), p + "mlp.gate": (l.ff, W), p + "mlp.up": (l.ff, W), p + "mlp.down": (W, l.ff),
                        p + "rg2": (W, W), p + "rg2.b": (W,), p + "hc2.in": (S,), p + "hc2.out": (S,),
                        p + "hc2.mix": (S, S)})
    return out


class _Sub:
    """The stream side of one sublayer: how it reads the streams, normalises, gates its result and writes back."""
    __slots__ = ("hc_in", "hc_mix", "hc_out", "norm", "rg_b", "has_gate")


class _LayerWeights:
    __slots__ = ("sub1", "sub2", "shift", "w_in", "dq_norm", "dkv_norm", "uq", "uk", "uv_t", "o", "w_ff", "down", "rg1")


class TetepelForCausalLM:
    supports_graph_decode = False      # the engine's captured decode step is built around the Llama launch sequence

    def __init__(self, shape: TetepelShape, dtype: torch.dtype, device, state: Dict[str, Tensor]):
        if dtype not in (torch.float32, torch.bfloat16):
            raise ValueError("Tetepel runs in bfloat16 or float32")
        self.shape, self.dtype, self.device = shape, dtype, torch.device(device)
        self.state = state
        self.layer_trace: Optional[List[Tensor]] = None    # tests: when a list, the sum of the streams after every layer run
        dev, S = self.device, shape.streams
        f32 = lambda t: t.to(device=dev, dtype=torch.float32).contiguous()
        act = lambda t: t.to(device=dev, dtype=dtype).contiguous()
        self.embed_table = act(state["embed"])
        self.final_norm = f32(state["final.norm"])
        self.ones = torch.ones(S, dtype=torch.float32, device=dev)
        self.eye = torch.eye(S, dtype=torch.float32, device=dev).contiguous()
        self.lw: List[_LayerWeights] = []
        for i, l in enumerate(shape.layers):
            m, p = l.mixer, f"l{i}."
            w = _LayerWeights()

            def sub(q: int) -> _Sub:
                s = _Sub()
                if p + f"hc{q}.in" in state:
                    s.hc_in, s.hc_mix, s.hc_out = (f32(state[p + f"hc{q}.{k}"]) for k in ("in", "mix", "out"))
                elif S == 1:          # one stream and no mixing weights: the plain residual sum
                    s.hc_in, s.hc_mix, s.hc_out = self.ones, self.eye, self.ones
                else:
                    raise KeyError(p + f"hc{q}.in")
                s.norm = f32(state[p + f"norm{q}"])
                s.has_gate = p + f"rg{q}" in state
                s.rg_b = (f32(state[p + f"rg{q}.b"]) if p + f"rg{q}.b" in state else None) if s.has_gate else None
                return s

            w.sub1 = sub(1)
            w.shift = f32(state[p + "shift"]) if p + "shift" in state else None
            w.w_in = act(torch.cat([state[p + "mix.dq"], state[p + "mix.dkv"], state[p + "mix.g"]], dim=0))
            w.dq_norm, w.dkv_norm = f32(state[p + "mix.dq.norm"]), f32(state[p + "mix.dkv.norm"])
            w.uq = act(state[p + "mix.uq"])
            w.uk = act(state[p + "mix.uk"].reshape(m.heads, m.dim, m.kv_rank))                       # q~_h = q_h @ uk[h]
            w.uv_t = act(state[p + "mix.uv"].reshape(m.heads, m.vdim, m.kv_rank).transpose(1, 2))    # o_h = l_h @ uv_t[h]
            w.o = act(state[p + "mix.o"])
            w.rg1 = act(state[p + "rg1"]) if w.sub1.has_gate else None
            w.sub2 = w.w_ff = w.down = None
            if l.ff:
                w.sub2 = sub(2)
                parts = [state[p + "mlp.gate"], state[p + "mlp.up"]] + ([state[p + "rg2"]] if w.sub2.has_gate else [])
                w.w_ff = act(torch.cat(parts, dim=0))
                w.down = act(state[p + "mlp.down"])
            self.lw.append(w)

    # ------------------------------------------------------------------ construction
    @classmethod
    def from_state_dict(cls, shape: TetepelShape, sd: Dict[str, Tensor], dtype, device) -> "TetepelForCausalLM":
        want = tensor_shapes(shape)
        # a checkpoint without shift / result-gate tensors has no such mechanism; one stream needs no mixing weights
        optional = lambda k: k.split(".", 1)[-1].split(".")[0] in ("shift", "rg1", "rg2") or (
            shape.streams == 1 and k.split(".", 1)[-1].startswith("hc"))
        missing = [k for k in want if k not in sd and not optional(k)]
        if missing:
            raise RuntimeError(f"{len(missing)} tensors missing from the checkpoint, e.g. {missing[:3]}")
        for k, shp in want.items():
            if k in sd and tuple(sd[k].shape) != shp:
                raise RuntimeError(f"tensor {k}: shape {tuple(sd[k].shape)} in the checkpoint, {shp} by config.json")
        return cls(shape, dtype, device, {k: sd[k] for k in want if k in sd})

    @classmethod
    def random_init(cls, shape: TetepelShape, dtype, device, seed: int = 0) -> "TetepelForCausalLM":
        """Random weights of a size that keeps activations O(1): linears N(0, 1/fan_in), norm weights near 1, stream
        weights near an averaging mix."""
        g = torch.Generator().manual_seed(seed)
        sd = {}
        for k, shp in tensor_shapes(shape).items():
            leaf = k.split(".", 1)[-1]
            if leaf in ("norm1", "norm2", "norm", "mix.dq.norm", "mix.dkv.norm") or k == "final.norm":
                t = 1.0 + 0.1 * torch.randn(shp, generator=g)
            elif leaf == "shift":
                t = torch.rand(shp, generator=g)
            elif leaf.endswith(".b"):
                t = 0.5 * torch.randn(shp, generator=g)
            elif leaf.startswith("hc"):
                S = shape.streams
                t = {"in": torch.full(shp, 1.0 / S), "out": torch.ones(shp),
                     "mix": torch.eye(S) * 0.7 + 0.3 / S}[leaf.split(".")[1]] + 0.1 * torch.randn(shp, generator=g)
            elif k == "embed":
                t = torch.randn(shp, generator=g) / math.sqrt(shp[1])
            else:
                t = torch.randn(shp, generator=g) / math.sqrt(shp[-1])
            sd[k] = t.to(torch.bfloat16)      # checkpoints hold bfloat16
        return cls(shape, dtype, device, sd)

    # ------------------------------------------------------------------ what the engine asks
    def cache_spec(self) -> dict:
        """Planes and row size of the paged cache this model needs: one latent row per token and layer run."""
        sh = self.shape
        return {"n_layers": sh.num_hidden_layers, "n_tokens": 1, "n_heads": 1, "head_size": sh.head_dim}

    def state_spec(self) -> Optional[dict]:
        """Rows a sequence carries from step to step: the mixer input of its last token, per layer run."""
        if all(w.shift is None for w in self.lw):
            return None
        return {"rows": self.shape.num_hidden_layers, "width": self.shape.hidden_size}

    def prepare_decode(self, max_rows: int = 64, keep_row_major: bool = True) -> None:
        """Nothing to prepare: decode steps run on the same weights as portions of prompts."""

    def weight_bytes(self) -> int:
        """Bytes of matrix weights a decode step streams (looped layers every time they run) + the output embedding."""
        e = torch.empty((), dtype=self.dtype).element_size()
        n = self.embed_table.numel()
        for li in self.shape.run_order:
            w = self.lw[li]
            n += sum(t.numel() for t in (w.w_in, w.uq, w.uk, w.uv_t, w.o, w.rg1, w.w_ff, w.down) if t is not None)
        return n * e

    def embed(self, input_ids: Tensor) -> Tensor:
        return input_ids

    # ------------------------------------------------------------------ forward
    def _mixer(self, run: int, li: int, x: Tensor, position_ids: Tensor, ap, seq: SequenceState) -> Optional[Tensor]:
        """The mixer sublayer of layer run `run`; returns the feed-forward's input when the layer has one (the streams'
        update and the feed-forward's read side are one launch)."""
        sh, w, m, dt = self.shape, self.lw[li], self.shape.layers[li].mixer, self.dtype
        T, H, D, V, R = x.shape[0], m.heads, m.dim, m.vdim, m.kv_rank
        s1 = w.sub1
        if w.shift is not None:
            h, hs = stream_norm(x, s1.hc_in, s1.norm, sh.norm_groups, sh.norm_eps, dt, shift_w=w.shift, seq=seq,
                                state_row=run, q_cu=ap.q_cu_seq_lens, positions=position_ids, want_plain=s1.has_gate)
        else:
            h = hs = stream_norm(x, s1.hc_in, s1.norm, sh.norm_groups, sh.norm_eps, dt)
        proj = torch.matmul(hs, w.w_in.t())                                   # [T, q_rank | kv_rank | heads]
        cache = ap.kv_cache.key_cache                                         # [n_blocks, block_size, 1, row]
        cq = latent_norm_cache(proj, 0, m.q_rank, m.q_rank, R, w.dq_norm, w.dkv_norm, sh.norm_eps, ap.new_cache_slots, cache)
        q = torch.matmul(cq, w.uq.t()).view(T, H, D)
        q_lat = torch.bmm(q.transpose(0, 1), w.uk)                            # [H, T, R]: the queries in the latent space
        o_lat = torch.empty_like(q_lat)
        latent_attention(q_lat.transpose(0, 1), cache, seq.tok_seq, position_ids, ap.q_cu_seq_lens, ap.block_tables,
                         ap.cu_blocks_lens, m.scale, m.window, ap.q_max_seq_len, gate_pre=proj[:, m.q_rank + R:],
                         out=o_lat.transpose(0, 1), max_kv_len=ap.kv_max_seq_len)
        o = torch.bmm(o_lat, w.uv_t)                                          # [H, T, V]
        y = torch.matmul(o.transpose(0, 1).reshape(T, H * V), w.o.t())
        gate_pre = torch.matmul(h, w.rg1.t()) if s1.has_gate else None
        if w.sub2 is not None:
            return stream_update_norm(x, y, s1.hc_mix, s1.hc_out, gate_pre, s1.rg_b, w.sub2.hc_in, w.sub2.norm,
                                      sh.norm_groups, sh.norm_eps)
        stream_update(x, y, s1.hc_mix, s1.hc_out, gate_pre, s1.rg_b)
        return None

    def _feed_forward(self, li: int, x: Tensor, h: Tensor) -> None:
        w, ff = self.lw[li], self.shape.layers[li].ff
        s2 = w.sub2
        gu = torch.matmul(h, w.w_ff.t())                                      # [T, gate | up | result gate]
        act = gelu_tanh_and_mul(gu[:, :ff], gu[:, ff:2 * ff])
        y = torch.matmul(act, w.down.t())
        stream_update(x, y, s2.hc_mix, s2.hc_out, gu[:, 2 * ff:] if s2.has_gate else None, s2.rg_b)

    def forward_hidden(self, input_ids: Tensor, position_ids: Tensor, model_params) -> Tensor:
        """The normalised sum of the streams [n_selected, width] of model_params.selected_token_ids (all rows if None).
        Every token's latent goes to the cache and every sequence's state slot is brought up to date."""
        sh = self.shape
        if input_ids.dtype not in (torch.int32, torch.int64):
            raise ValueError("Tetepel takes token ids (its embedding is scaled and copied into the streams)")
        seq = model_params.sequence_state
        if position_ids.dtype != torch.int32:
            position_ids = position_ids.to(torch.int32)
        if seq is None:
            if self.state_spec() is not None:
                raise ValueError("Tetepel with a token shift needs LanguageModelParameters.sequence_state (the batch's "
                                 "sequences and their state slots)")
            # no state rows: the sequence of every token follows from the batch's portion lengths (no host round trip)
            q_cu = model_params.attention_params[0].q_cu_seq_lens
            tok_seq = torch.repeat_interleave(torch.arange(q_cu.numel() - 1, device=q_cu.device), q_cu.diff().long(),
                                              output_size=input_ids.shape[0]).to(torch.int32)
            seq = SequenceState(None, None, tok_seq)
        x = stream_embed(input_ids.contiguous(), self.embed_table, sh.embedding_scale, sh.streams)
        for run, li in enumerate(sh.run_order):
            h_ff = self._mixer(run, li, x, position_ids, model_params.attention_params[run], seq)
            if sh.layers[li].ff:
                self._feed_forward(li, x, h_ff)
            if self.layer_trace is not None:
                self.layer_trace.append(x.sum(dim=1))
        sel = model_params.selected_token_ids
        rows = sel.to(torch.int32).contiguous() if sel is not None else None
        return stream_norm(x, self.ones, self.final_norm, sh.norm_groups, sh.norm_eps, self.dtype, rows=rows)

    def forward_logits(self, input_ids: Tensor, position_ids: Tensor, model_params) -> Tensor:
        """float32 logits [n_selected, vocab]: the embedding table itself (without its scale) applied to the output."""
        x = self.forward_hidden(input_ids, position_ids, model_params)
        return torch.matmul(x, self.embed_table.t()).float()

    def forward(self, input_ids: Tensor, position_ids: Tensor, model_params) -> Tensor:
        """Greedy token ids of the selected rows, like the framework's other models."""
        return torch.argmax(self.forward_logits(input_ids, position_ids, model_params), dim=-1)

    __call__ = forward


def read_shape(model_path: str) -> TetepelShape:
    with open(os.path.join(model_path, "config.json")) as f:
        return TetepelShape.from_config(json.load(f))
