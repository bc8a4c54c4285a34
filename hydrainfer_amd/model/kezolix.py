"""Kezolix — a decoder-only hybrid of recurrent and attention layers with a depth-averaged residual:

  * x = embed[token] + pos[position] (a learned position table);
  * every sublayer sits between two layer norms (weight, no bias): x <- x + m * norm_b(sublayer(norm_a(x))), m a constant;
  * depth average: with X_0 the embedding output and X_(i+1) the result of layer i, the input of layer i + 1 (and of the
    output head after the last) is sum_{j <= i+1} dwa_i[j] X_j — the levels X_j of a step are kept in one float stack;
  * mixer `attention`: grouped-query attention, ONE RMS norm over the whole query projection and one over the whole key
    projection (all heads at once), no rotation, score = q . k * scale - slope_h (i - j) with slope_h = 2^(-8 (h + 1) / H),
    a chunked mask (i sees j <= i of its own chunk, chunks counted from position 0) or a plain causal one; a layer with
    `kv_from: j` has no key / value tensors and reads the cache planes layer j wrote in the same step;
  * mixer `hgrn2`: a gated linear recurrence with a matrix state per head, f = low + (1 - low) sigmoid(W_f h + b),
    S <- diag(f) S + (1 - f) v^T, o = S^T silu(W_q h), RMS norm of o per head; the float state of a sequence lives in its
    state slot between steps (one row per recurrent layer);
  * feed-forward `dense`: W_down PolyNorm(W_up h); `moe`: softmax router (choice = score + correction, weights = the
    chosen scores over their sum, times a scale), squared-ReLU experts, and a shared expert gated by sigmoid(w_sg . h);
    or none;
  * logits = head . norm(x).

Every size and constant comes from config.json (`KezolixShape.from_config`), every tensor from model.safetensors under
the names of `tensor_shapes`.  The residual, norms, routers, scores, softmax weights, gates and recurrent state are float;
the matrix products run in the model's dtype (bfloat16 with float accumulation, or float32).

The compute path: library GEMMs (torch.matmul) for the dense projections and the kernels of libhydra_mix.so
(_C.kernel.depth_ops, .biased_attn, .recurrence, .moe_mix).  The model plugs into the engine through the interface
LlamaForCausalLM has: forward_hidden / forward_logits / forward over (token ids, position ids, LanguageModelParameters);
`cache_spec` asks the block manager for one key and one value plane per attention layer that owns its keys, `state_spec`
asks the state-slot manager for one row per recurrent layer."""
import json
import math
import os
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch
from torch import Tensor

from hydrainfer_amd._C.kernel.biased_attn import biased_attention, qk_norm_cache
from hydrainfer_amd._C.kernel.depth_ops import depth_norm, embed_positions, poly_norm, relu_squared
from hydrainfer_amd._C.kernel.moe_mix import grouped_linear, moe_combine, moe_plan, route_softmax_topk
from hydrainfer_amd._C.kernel.recurrence import gated_recurrence
from hydrainfer_amd._C.kernel.stream_ops import SequenceState

ARCHITECTURE = "Kezolix"
SLOPE_EXPONENT = 8.0          # slope_h = 2^(-SLOPE_EXPONENT (h + 1) / H)


@dataclass
class MixerSpec:
    type: str                         # "attention" | "hgrn2"
    heads: int
    dim: int                          # query / key size per head
    vdim: int                         # value size per head
    kv_heads: int = 0                 # attention: key / value heads (0: as many as heads)
    scale: float = 1.0                # attention
    chunk: Optional[int] = None       # attention: size of the mask's chunks (or of its window); None: every j <= i
    kv_from: Optional[int] = None     # attention: the layer whose keys and values this one reads
    mask: str = "chunk"               # attention, with a size: "chunk" (i sees j <= i of its own chunk) | "window" (0 <= i - j < size)

    def __post_init__(self):
        if self.type == "attention":
            self.kv_heads = self.kv_heads or self.heads
            if self.heads % self.kv_heads:
                raise ValueError("attention: heads must be a multiple of kv_heads")


@dataclass
class FeedForwardSpec:
    kind: str                         # "dense" | "moe"
    ff: int = 0                       # dense: inner size; moe: an expert's inner size
    experts: int = 0
    top: int = 0
    router_scale: float = 1.0
    shared_ff: Optional[int] = None   # moe: inner size of the shared expert, None: there is none


@dataclass
class KezolixLayer:
    mixer: MixerSpec
    mlp: Optional[FeedForwardSpec]


@dataclass
class KezolixShape:
    vocab_size: int
    hidden_size: int
    layers: List[KezolixLayer]
    max_position_embeddings: int = 2048
    norm_eps: float = 1e-5
    residual_mult: float = 1.0
    cache_plane: Dict[int, int] = field(default_factory=dict)    # attention layer -> the cache plane it reads (its own or its lender's)
    state_row: Dict[int, int] = field(default_factory=dict)      # recurrent layer -> its row of a state slot

    def __post_init__(self):
        self.cache_plane, self.state_row = {}, {}
        for i, l in enumerate(self.layers):
            m = l.mixer
            if m.type == "attention":
                if m.kv_from is None:
                    self.cache_plane[i] = len(set(self.cache_plane.values()))
                else:
                    j = m.kv_from
                    src = self.layers[j].mixer if 0 <= j < i else None
                    if src is None or src.type != "attention" or src.kv_from is not None:
                        raise ValueError(f"layer {i}: kv_from {j} is not an earlier attention layer with keys of its own")
                    if (src.kv_heads, src.dim, src.vdim) != (m.kv_heads, m.dim, m.vdim):
                        raise ValueError(f"layer {i}: its key / value shape differs from layer {j}'s")
                    self.cache_plane[i] = self.cache_plane[j]
            elif m.type == "hgrn2":
                self.state_row[i] = len(self.state_row)
            else:
                raise ValueError(f"layer {i}: unknown mixer type {m.type!r}")

    # what the engine's cache pool and parameter builders ask of a model's shape
    @property
    def num_hidden_layers(self) -> int:          # cache planes: one per attention layer with keys of its own
        return max(1, len(set(self.cache_plane.values())))

    @property
    def num_attention_heads(self) -> int:
        return max([l.mixer.heads for l in self.layers if l.mixer.type == "attention"] or [1])

    @property
    def num_key_value_heads(self) -> int:
        return max([l.mixer.kv_heads for l in self.layers if l.mixer.type == "attention"] or [1])

    @property
    def head_dim(self) -> int:                   # width of a cached head: the larger of key and value rows
        return max([max(l.mixer.dim, l.mixer.vdim) for l in self.layers if l.mixer.type == "attention"] or [1])

    @classmethod
    def from_config(cls, cfg: dict) -> "KezolixShape":
        if cfg.get("architecture") != ARCHITECTURE:
            raise ValueError(f"not a {ARCHITECTURE} configuration: {cfg.get('architecture')!r}")
        layers = []
        for i, l in enumerate(cfg["layers"]):
            m, kind = l["mixer"], l["type"]
            if kind == "attention":
                mask = m.get("mask") or {}
                mask_kind = str(mask.get("kind") or mask.get("type") or "chunk").lower()
                if mask_kind in ("chunk", "chunked", "chunks", "block"):
                    mask_kind = "chunk"
                elif mask_kind in ("window", "sliding", "sliding_window", "local"):
                    mask_kind = "window"
                elif mask_kind in ("causal", "none", "full"):
                    mask, mask_kind = {}, "chunk"
                else:
                    raise ValueError(f"layer {i}: unknown mask kind {mask_kind!r}")
                mixer = MixerSpec(kind, int(m["heads"]), int(m["dim"]), int(m["vdim"]), int(m.get("kv_heads") or m["heads"]),
                                  float(m.get("scale", 1.0)), int(mask["size"]) if mask.get("size") else None,
                                  int(m["kv_from"]) if m.get("kv_from") is not None else None, mask_kind)
            elif kind == "hgrn2":
                mixer = MixerSpec(kind, int(m["heads"]), int(m["dim"]), int(m["vdim"]))
            else:
                raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
            mlp, spec = l.get("mlp"), None
            if mlp is not None:
                if mlp.get("kind", "dense") == "dense":
                    spec = FeedForwardSpec("dense", int(mlp["ff"]))
                elif mlp["kind"] == "moe":
                    r, sh = mlp["router"], mlp.get("shared")
                    spec = FeedForwardSpec("moe", int(mlp["expert"]["ff"]), int(r["experts"]), int(r["top"]),
                                           float(r.get("scale", 1.0)), int(sh["ff"]) if sh else None)
                else:
                    raise ValueError(f"layer {i}: unknown feed-forward kind {mlp['kind']!r}")
            layers.append(KezolixLayer(mixer, spec))
        return cls(vocab_size=int(cfg["vocab"]), hidden_size=int(cfg["width"]), layers=layers,
                   max_position_embeddings=int(cfg["max_positions"]), norm_eps=float((cfg.get("norm") or {}).get("eps", 1e-5)),
                   residual_mult=float(cfg.get("residual_mult", 1.0)))

    def to_config(self) -> dict:
        out = []
        for l in self.layers:
            m = l.mixer
            mixer = {"heads": m.heads, "dim": m.dim, "vdim": m.vdim}
            if m.type == "attention":
                mixer.update({"kv_heads": m.kv_heads, "scale": m.scale})
                if m.chunk:
                    mixer["mask"] = {"size": m.chunk} if m.mask == "chunk" else {"kind": m.mask, "size": m.chunk}
                if m.kv_from is not None:
                    mixer["kv_from"] = m.kv_from
            mlp = None
            if l.mlp is not None and l.mlp.kind == "dense":
                mlp = {"kind": "dense", "ff": l.mlp.ff}
            elif l.mlp is not None:
                mlp = {"kind": "moe", "expert": {"ff": l.mlp.ff},
                       "router": {"experts": l.mlp.experts, "top": l.mlp.top, "scale": l.mlp.router_scale}}
                if l.mlp.shared_ff:
                    mlp["shared"] = {"ff": l.mlp.shared_ff}
            out.append({"type": m.type, "mixer": mixer, "mlp": mlp})
        return {"architecture": ARCHITECTURE, "vocab": self.vocab_size, "width": self.hidden_size,
                "max_positions": self.max_position_embeddings, "norm": {"eps": self.norm_eps},
                "residual_mult": self.residual_mult, "layers": out}


def tensor_shapes(shape: KezolixShape) -> Dict[str, tuple]:
    """Name -> shape of every tensor of a checkpoint of this shape (linear weights are [out, in])."""
    W = shape.hidden_size
    out = {"embed": (shape.vocab_size, W), "pos": (shape.max_position_embeddings, W), "final.norm": (W,),
           "head": (shape.vocab_size, W)}
    for i, l in enumerate(shape.layers):
        m, p = l.mixer, f"l{i}."
        out.update({p + "norm1": (W,), p + "norm1b": (W,), p + "dwa": (i + 2,)})
        if m.type == "attention":
            out.update({p + "mix.q": (m.heads * m.dim, W), p + "mix.q.norm": (m.heads * m.dim,), p + "mix.o": (W, m.heads * m.vdim)})
            if m.kv_from is None:
                out.update({p + "mix.k": (m.kv_heads * m.dim, W), p + "mix.k.norm": (m.kv_heads * m.dim,),
                            p + "mix.v": (m.kv_heads * m.vdim, W)})
        else:
            out.update({p + "mix.q": (m.heads * m.dim, W), p + "mix.f": (m.heads * m.dim, W), p + "mix.f.b": (m.heads * m.dim,),
                        p + "mix.lower": (m.heads * m.dim,), p + "mix.v": (m.heads * m.vdim, W), p + "mix.norm": (m.vdim,),
                        p + "mix.o": (W, m.heads * m.vdim)})
        f = l.mlp
        if f is None:
            continue
        out.update({p + "norm2": (W,), p + "norm2b": (W,)})
        if f.kind == "dense":
            out.update({p + "mlp.up": (f.ff, W), p + "mlp.down": (W, f.ff), p + "mlp.act": (4,)})
        else:
            for e in range(f.experts):
                out.update({p + f"mlp.e{e}.up": (f.ff, W), p + f"mlp.e{e}.down": (W, f.ff)})
            out.update({p + "mlp.router": (f.experts, W), p + "mlp.correction": (f.experts,)})
            if f.shared_ff:
                out.update({p + "mlp.shared.up": (f.shared_ff, W), p + "mlp.shared.down": (W, f.shared_ff),
                            p + "mlp.shared.sg": (1, W)})
    return out


OPTIONAL_LEAVES = ("dwa", "mlp.correction")      # a checkpoint without them: no depth average / no choice bias


class _LayerWeights:
    __slots__ = ("norm1", "norm1b", "norm2", "norm2b", "dwa", "w_in", "q_norm", "k_norm", "slopes", "f_bias", "low", "o_norm",
                 "o", "up", "down", "coef", "router", "correction", "sh_up", "sh_down")


class KezolixForCausalLM:
    supports_graph_decode = False      # the engine's captured decode step is built around the Llama launch sequence

    def __init__(self, shape: KezolixShape, dtype: torch.dtype, device, state: Dict[str, Tensor]):
        if dtype not in (torch.float32, torch.bfloat16):
            raise ValueError("Kezolix runs in bfloat16 or float32")
        self.shape, self.dtype, self.device = shape, dtype, torch.device(device)
        self.state = state
        self.layer_trace: Optional[List[Tensor]] = None    # tests: when a list, what every layer passes on (after the depth average)
        dev = self.device
        f32 = lambda t: t.to(device=dev, dtype=torch.float32).contiguous()
        act = lambda t: t.to(device=dev, dtype=dtype).contiguous()
        self.embed_table, self.pos_table = act(state["embed"]), act(state["pos"])
        self.final_norm, self.head = f32(state["final.norm"]), act(state["head"])
        self.lw: List[_LayerWeights] = []
        for i, l in enumerate(shape.layers):
            m, p = l.mixer, f"l{i}."
            w = _LayerWeights()
            for s in _LayerWeights.__slots__:
                setattr(w, s, None)
            w.norm1, w.norm1b = f32(state[p + "norm1"]), f32(state[p + "norm1b"])
            w.dwa = f32(state[p + "dwa"]) if p + "dwa" in state else None
            if m.type == "attention":
                parts = [state[p + "mix.q"]] + ([state[p + "mix.k"], state[p + "mix.v"]] if m.kv_from is None else [])
                w.w_in = act(torch.cat(parts, dim=0))
                w.q_norm = f32(state[p + "mix.q.norm"])
                w.k_norm = f32(state[p + "mix.k.norm"]) if m.kv_from is None else None
                w.slopes = torch.tensor([2.0 ** (-SLOPE_EXPONENT * (h + 1) / m.heads) for h in range(m.heads)],
                                        dtype=torch.float64).to(device=dev, dtype=torch.float32)
            else:
                w.w_in = act(torch.cat([state[p + "mix.q"], state[p + "mix.f"], state[p + "mix.v"]], dim=0))
                w.f_bias, w.low, w.o_norm = f32(state[p + "mix.f.b"]), f32(state[p + "mix.lower"]), f32(state[p + "mix.norm"])
            w.o = act(state[p + "mix.o"])
            f = l.mlp
            if f is not None:
                w.norm2, w.norm2b = f32(state[p + "norm2"]), f32(state[p + "norm2b"])
                if f.kind == "dense":
                    w.up, w.down, w.coef = act(state[p + "mlp.up"]), act(state[p + "mlp.down"]), f32(state[p + "mlp.act"])
                else:
                    w.up = act(torch.stack([state[p + f"mlp.e{e}.up"] for e in range(f.experts)]))        # [E, ff, W]
                    w.down = act(torch.stack([state[p + f"mlp.e{e}.down"] for e in range(f.experts)]))    # [E, W, ff]
                    rows = [state[p + "mlp.router"]] + ([state[p + "mlp.shared.sg"].reshape(1, -1)] if f.shared_ff else [])
                    w.router = f32(torch.cat(rows, dim=0))                                               # [E (+ 1), W]
                    w.correction = f32(state[p + "mlp.correction"]) if p + "mlp.correction" in state else None
                    if f.shared_ff:
                        w.sh_up, w.sh_down = act(state[p + "mlp.shared.up"]), act(state[p + "mlp.shared.down"])
            self.lw.append(w)

    # ------------------------------------------------------------------ construction
    @classmethod
    def from_state_dict(cls, shape: KezolixShape, sd: Dict[str, Tensor], dtype, device) -> "KezolixForCausalLM":
        want = tensor_shapes(shape)
        optional = lambda k: k.split(".", 1)[-1] in OPTIONAL_LEAVES
        missing = [k for k in want if k not in sd and not optional(k)]
        if missing:
            raise RuntimeError(f"{len(missing)} tensors missing from the checkpoint, e.g. {missing[:3]}")
        for k, shp in want.items():
            if k in sd and tuple(sd[k].shape) != shp:
                raise RuntimeError(f"tensor {k}: shape {tuple(sd[k].shape)} in the checkpoint, {shp} by config.json")
        return cls(shape, dtype, device, {k: sd[k] for k in want if k in sd})

    @staticmethod
    def random_state_dict(shape: KezolixShape, seed: int = 0) -> Dict[str, Tensor]:
        """Random bfloat16 weights of a size that keeps activations O(1): linears N(0, 1/fan_in), norm weights near 1,
        lower bounds in (0, 0.9), depth weights near an average of the levels."""
        g = torch.Generator().manual_seed(seed)
        sd = {}
        for k, shp in tensor_shapes(shape).items():
            leaf = k.split(".", 1)[-1] if k[0] == "l" and k[1].isdigit() else k
            if leaf in ("norm1", "norm1b", "norm2", "norm2b", "mix.norm", "mix.q.norm", "mix.k.norm", "final.norm"):
                t = 1.0 + 0.1 * torch.randn(shp, generator=g)
            elif leaf == "mix.lower":
                t = 0.9 * torch.rand(shp, generator=g)
            elif leaf == "mix.f.b":
                t = torch.randn(shp, generator=g)
            elif leaf == "dwa":
                t = torch.full(shp, 1.0 / shp[0]) + 0.1 * torch.randn(shp, generator=g) / shp[0]
                t[-1] += 0.5
            elif leaf == "mlp.correction":
                t = 0.02 * torch.randn(shp, generator=g)
            elif leaf == "mlp.act":
                t = torch.tensor([0.5, 0.3, 0.2, 0.05]) + 0.1 * torch.randn(shp, generator=g)
            elif k in ("embed", "pos"):
                t = torch.randn(shp, generator=g) * 0.7
            else:
                t = torch.randn(shp, generator=g) / math.sqrt(shp[-1])
            sd[k] = t.to(torch.bfloat16)      # checkpoints hold bfloat16
        return sd

    @classmethod
    def random_init(cls, shape: KezolixShape, dtype, device, seed: int = 0) -> "KezolixForCausalLM":
        return cls(shape, dtype, device, cls.random_state_dict(shape, seed))

    # ------------------------------------------------------------------ what the engine asks
    def cache_spec(self) -> dict:
        """Planes and row size of the paged cache: a key and a value plane per attention layer with keys of its own."""
        sh = self.shape
        return {"n_layers": sh.num_hidden_layers, "n_tokens": 2, "n_heads": sh.num_key_value_heads, "head_size": sh.head_dim}

    def state_spec(self) -> Optional[dict]:
        """What a sequence carries from step to step: the matrix state of every recurrent layer, one row each."""
        sh = self.shape
        if not sh.state_row:
            return None
        return {"rows": len(sh.state_row),
                "width": max(l.mixer.heads * l.mixer.dim * l.mixer.vdim for l in sh.layers if l.mixer.type == "hgrn2")}

    def prepare_decode(self, max_rows: int = 64, keep_row_major: bool = True) -> None:
        """Nothing to prepare: decode steps run on the same weights as portions of prompts."""

    def weight_bytes(self, tokens: int = 1) -> int:
        """Bytes of matrix weights a step of `tokens` tokens streams at most (an expert is read once if any token chose it)."""
        e = torch.empty((), dtype=self.dtype).element_size()
        n = self.head.numel()
        for l, w in zip(self.shape.layers, self.lw):
            n += w.w_in.numel() + w.o.numel()
            f = l.mlp
            if f is None:
                continue
            if f.kind == "dense":
                n += w.up.numel() + w.down.numel()
            else:
                used = min(f.experts, tokens * f.top)
                n += (w.up.numel() + w.down.numel()) * used // f.experts
                n += (w.sh_up.numel() + w.sh_down.numel()) if f.shared_ff else 0
        return n * e

    def embed(self, input_ids: Tensor) -> Tensor:
        return input_ids

    # ------------------------------------------------------------------ forward
    def _attention(self, i: int, h: Tensor, position_ids: Tensor, params, seq: SequenceState) -> Tensor:
        m, w, sh = self.shape.layers[i].mixer, self.lw[i], self.shape
        ap = params.attention_params[sh.cache_plane[i]]
        T, H, G, D, V = h.shape[0], m.heads, m.kv_heads, m.dim, m.vdim
        kc, vc = ap.kv_cache.get_kv_cache()
        proj = torch.matmul(h, w.w_in.t())                           # [T, q | k | v]  (a borrower: q only)
        if m.kv_from is None:
            q = qk_norm_cache(proj, H * D, G * D, G * V, w.q_norm, w.k_norm, sh.norm_eps, G, ap.new_cache_slots, kc, vc)
        else:
            q = qk_norm_cache(proj, H * D, 0, 0, w.q_norm, None, sh.norm_eps, G)
        o = biased_attention(q.view(T, H, D), kc, vc, V, seq.tok_seq, position_ids, ap.q_cu_seq_lens, ap.block_tables,
                             ap.cu_blocks_lens, m.scale, w.slopes, m.mask if m.chunk else "causal", m.chunk or 0,
                             max_q_len=ap.q_max_seq_len, kv_heads=G, max_kv_len=ap.kv_max_seq_len)
        return torch.matmul(o.view(T, H * V), w.o.t())

    def _recurrence(self, i: int, h: Tensor, position_ids: Tensor, params, seq: SequenceState) -> Tensor:
        m, w, sh = self.shape.layers[i].mixer, self.lw[i], self.shape
        HD = m.heads * m.dim
        proj = torch.matmul(h, w.w_in.t())                           # [T, q | f | v]
        o = gated_recurrence(proj[:, :HD], proj[:, HD:2 * HD], proj[:, 2 * HD:], w.f_bias, w.low, w.o_norm, sh.norm_eps, seq,
                             sh.state_row[i], params.attention_params[0].q_cu_seq_lens, position_ids, m.heads, m.dim, m.vdim,
                             max_q_len=params.attention_params[0].q_max_seq_len)
        return torch.matmul(o, w.o.t())

    def _feed_forward(self, i: int, h: Tensor) -> Tensor:
        f, w = self.shape.layers[i].mlp, self.lw[i]
        if f.kind == "dense":
            return torch.matmul(poly_norm(torch.matmul(h, w.up.t()), w.coef, self.shape.norm_eps), w.down.t())
        T = h.shape[0]
        r = torch.matmul(h.float(), w.router.t())                    # float: router logits (| the shared expert's gate)
        weights, experts = route_softmax_topk(r, f.experts, f.top, f.router_scale, w.correction)
        seg, row_of, src = moe_plan(experts, f.experts)
        y = grouped_linear(h, w.up, seg, T * f.top, src=src, act="relu2")
        y = grouped_linear(y, w.down, seg, T * f.top)
        shared = gate = None
        if f.shared_ff:
            shared = torch.matmul(relu_squared(torch.matmul(h, w.sh_up.t())), w.sh_down.t())
            gate = r[:, f.experts:]
        return moe_combine(y, row_of, weights, shared, gate)

    def forward_hidden(self, input_ids: Tensor, position_ids: Tensor, model_params) -> Tensor:
        """The normed output [n_selected, width] of model_params.selected_token_ids (all rows if None).  Every token's keys
        and values go to the cache and every sequence's state slot is brought up to date."""
        sh, dt = self.shape, self.dtype
        if input_ids.dtype not in (torch.int32, torch.int64):
            raise ValueError("Kezolix takes token ids (its embedding is summed with the position table in float)")
        if position_ids.dtype != torch.int32:
            position_ids = position_ids.to(torch.int32)
        input_ids, position_ids = input_ids.contiguous(), position_ids.contiguous()
        seq = model_params.sequence_state
        if seq is None:
            if sh.state_row:
                raise ValueError("Kezolix with recurrent layers needs LanguageModelParameters.sequence_state (the batch's "
                                 "sequences and their state slots)")
            q_cu = model_params.attention_params[0].q_cu_seq_lens
            tok_seq = torch.repeat_interleave(torch.arange(q_cu.numel() - 1, device=q_cu.device), q_cu.diff().long(),
                                              output_size=input_ids.shape[0]).to(torch.int32)
            seq = SequenceState(None, None, tok_seq)
        T, W, L = input_ids.shape[0], sh.hidden_size, len(sh.layers)
        eps, mult = sh.norm_eps, sh.residual_mult
        levels = torch.empty((L + 1, T, W), dtype=torch.float32, device=self.device)
        mid = torch.empty((T, W), dtype=torch.float32, device=self.device)
        nxt = torch.empty((T, W), dtype=torch.float32, device=self.device)
        x = embed_positions(input_ids, position_ids, self.embed_table, self.pos_table, out=levels[0])
        h = depth_norm(x, dt, eps, next_w=self.lw[0].norm1) if L else None
        sel = model_params.selected_token_ids
        rows = sel.to(torch.int32).contiguous() if sel is not None and self.layer_trace is None else None
        for i, (l, w) in enumerate(zip(sh.layers, self.lw)):
            mix = self._attention if l.mixer.type == "attention" else self._recurrence
            y = mix(i, h, position_ids, model_params, seq)
            post = w.norm1b
            if l.mlp is not None:
                h = depth_norm(x, dt, eps, y=y, post_w=post, mult=mult, x_out=mid, next_w=w.norm2)
                y, post, x = self._feed_forward(i, h), w.norm2b, mid
            last = i == L - 1
            # the layer's result joins the levels; their weighted average is the next input, normed for its first sublayer
            h = depth_norm(x, dt, eps, y=y, post_w=post, mult=mult, level_out=levels[i + 1], levels=levels, depth_w=w.dwa,
                           x_out=None if (last and rows is not None) else nxt,
                           next_w=self.final_norm if last else self.lw[i + 1].norm1, rows=rows if last else None)
            x = nxt
            if self.layer_trace is not None:
                self.layer_trace.append(nxt.clone())
        if L == 0:
            h = depth_norm(x, dt, eps, next_w=self.final_norm, rows=rows)
        elif rows is None and sel is not None:
            h = h.index_select(0, sel.to(torch.int64))
        return h

    def forward_logits(self, input_ids: Tensor, position_ids: Tensor, model_params) -> Tensor:
        """float32 logits [n_selected, vocab]."""
        x = self.forward_hidden(input_ids, position_ids, model_params)
        return torch.matmul(x, self.head.t()).float()

    def forward(self, input_ids: Tensor, position_ids: Tensor, model_params) -> Tensor:
        """Greedy token ids of the selected rows, like the framework's other models."""
        return torch.argmax(self.forward_logits(input_ids, position_ids, model_params), dim=-1)

    __call__ = forward


def read_shape(model_path: str) -> KezolixShape:
    with open(os.path.join(model_path, "config.json")) as f:
        return KezolixShape.from_config(json.load(f))
