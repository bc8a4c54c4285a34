"""A plain, slow restatement of the Tetepel design in float64 on the CPU, one function per mechanism, written from the
design's equations (it shares no code with hydrainfer_amd).  Weights are a dict under the checkpoint's tensor names; the
configuration is the dict config.json holds.  Whole sequences only: no cache, no state, no batching — what the engine
must reproduce however it cuts and batches the work."""
import math
from typing import Dict, List, Optional

import torch

F = torch.float64


def grouped_rms_norm(x: torch.Tensor, w: torch.Tensor, groups: int, eps: float) -> torch.Tensor:
    """x [..., n] split into `groups` consecutive parts, each divided by sqrt(mean(part^2) + eps); then times w."""
    parts = x.reshape(*x.shape[:-1], groups, x.shape[-1] // groups)
    rms = torch.sqrt((parts ** 2).mean(dim=-1, keepdim=True) + eps)
    return (parts / rms).reshape(x.shape) * w


def token_shift(h: torch.Tensor, shift: torch.Tensor) -> torch.Tensor:
    """h [n, w] of one sequence: row i moves towards row i - 1 (zeros before the first): h_i + (h_{i-1} - h_i) * shift."""
    prev = torch.zeros_like(h)
    prev[1:] = h[:-1]
    return h + (prev - h) * shift


def streams_read(xs: torch.Tensor, w_in: torch.Tensor) -> torch.Tensor:
    """xs [s, n, w]: u = sum_s w_in[s] xs[s]."""
    return (w_in[:, None, None] * xs).sum(dim=0)


def streams_write(xs: torch.Tensor, y: torch.Tensor, mix: torch.Tensor, w_out: torch.Tensor) -> torch.Tensor:
    """new[t] = sum_s mix[s, t] xs[s] + w_out[t] y, every target from the old streams."""
    new = torch.zeros_like(xs)
    for t in range(xs.shape[0]):
        for s in range(xs.shape[0]):
            new[t] += mix[s, t] * xs[s]
        new[t] += w_out[t] * y
    return new


def result_gate(h: torch.Tensor, w: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    return torch.sigmoid(h @ w.T + b)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def dense_ff(h, w_gate, w_up, w_down):
    return (gelu_tanh(h @ w_gate.T) * (h @ w_up.T)) @ w_down.T


def window_visible(n: int, window: Optional[int]) -> torch.Tensor:
    """[n, n] bool: query i sees key j iff 0 <= i - j (< window)."""
    d = torch.arange(n)[:, None] - torch.arange(n)[None, :]
    ok = d >= 0
    if window:
        ok &= d < window
    return ok


def latent_attention(h: torch.Tensor, W: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    """The mixer on the (shifted) input h [n, w] of one sequence; keys and values are materialised per head."""
    n, H, D, V = h.shape[0], m["heads"], m["dim"], m["vdim"]
    cq = grouped_rms_norm(h @ W[p + "dq"].T, W[p + "dq.norm"], 1, eps)
    q = (cq @ W[p + "uq"].T).reshape(n, H, D)
    c = grouped_rms_norm(h @ W[p + "dkv"].T, W[p + "dkv.norm"], 1, eps)
    k = (c @ W[p + "uk"].T).reshape(n, H, D)
    v = (c @ W[p + "uv"].T).reshape(n, H, V)
    size = (m.get("mask") or {}).get("size")
    visible = window_visible(n, size)
    gate = torch.sigmoid(h @ W[p + "g"].T)                       # [n, H]
    out = torch.zeros(n, H, V, dtype=h.dtype)
    for hd in range(H):
        score = (q[:, hd] @ k[:, hd].T) * m["scale"]
        score = score.masked_fill(~visible, float("-inf"))
        out[:, hd] = torch.softmax(score, dim=-1) @ v[:, hd]
        out[:, hd] *= gate[:, hd:hd + 1]
    return out.reshape(n, H * V) @ W[p + "o"].T


def run_order(cfg: dict) -> List[int]:
    n = len(cfg["layers"])
    loop = cfg.get("loop") or {"start": 0, "stop": 0, "times": 1}
    return (list(range(loop["start"])) + list(range(loop["start"], loop["stop"])) * loop["times"]
            + list(range(loop["stop"], n)))


def forward(cfg: dict, weights: Dict[str, torch.Tensor], tokens: List[int], layer_sums: Optional[list] = None) -> torch.Tensor:
    """Logits [n, vocab] of one sequence."""
    W = {k: v.to(F) for k, v in weights.items()}
    eps, groups, S = cfg["norm"]["eps"], cfg["norm"]["groups"], cfg.get("streams", 1)
    x = W["embed"][torch.tensor(tokens)] * cfg["embedding"]["scale"]
    xs = torch.stack([x] * S)
    for li in run_order(cfg):
        layer, p = cfg["layers"][li], f"l{li}."
        for q in (1, 2):
            if q == 2 and layer.get("mlp") is None:
                continue
            if p + f"hc{q}.in" in W:
                w_in, mix, w_out = W[p + f"hc{q}.in"], W[p + f"hc{q}.mix"], W[p + f"hc{q}.out"]
            else:
                w_in, mix, w_out = torch.ones(1, dtype=F), torch.ones(1, 1, dtype=F), torch.ones(1, dtype=F)
            h = grouped_rms_norm(streams_read(xs, w_in), W[p + f"norm{q}"], groups, eps)
            if q == 1:
                hs = token_shift(h, W[p + "shift"]) if p + "shift" in W else h
                y = latent_attention(hs, W, p + "mix.", layer["mixer"], eps)
            else:
                y = dense_ff(h, W[p + "mlp.gate"], W[p + "mlp.up"], W[p + "mlp.down"])
            if p + f"rg{q}" in W:
                y = y * result_gate(h, W[p + f"rg{q}"], W[p + f"rg{q}.b"])
            xs = streams_write(xs, y, mix, w_out)
        if layer_sums is not None:
            layer_sums.append(xs.sum(dim=0))
    out = grouped_rms_norm(xs.sum(dim=0), W["final.norm"], groups, eps)
    return out @ W["embed"].T


def greedy(cfg, weights, prompt: List[int], n_new: int):
    """(tokens generated greedily, top-1 margin of every step)."""
    toks, out, margins = list(prompt), [], []
    for _ in range(n_new):
        last = forward(cfg, weights, toks)[-1]
        top = torch.topk(last, 2).values
        out.append(int(torch.argmax(last)))
        margins.append(float(top[0] - top[1]))
        toks.append(out[-1])
    return out, margins
