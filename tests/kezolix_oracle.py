"""A plain, slow restatement of the Kezolix design in float64 on the CPU, one function per mechanism, written from the
design's equations (it shares no code with hydrainfer_amd).  Weights are a dict under the checkpoint's tensor names; the
configuration is the dict config.json holds.  Whole sequences only: no cache, no state slots, no batching — what the
engine must reproduce however it cuts and batches the work."""
import math
from typing import Dict, List, Optional

import torch

F = torch.float64


def layer_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """(x - mean) / sqrt(var + eps) * w over the last axis; var is the mean squared deviation; no bias."""
    mu = x.mean(dim=-1, keepdim=True)
    var = ((x - mu) ** 2).mean(dim=-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w


def rms_div(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x ** 2).mean(dim=-1, keepdim=True) + eps)


def head_slopes(n_heads: int) -> torch.Tensor:
    """slope of head h = 2^(-8 (h + 1) / H)."""
    return torch.tensor([2.0 ** (-8.0 * (h + 1) / n_heads) for h in range(n_heads)], dtype=F)


def visible(n: int, chunk: Optional[int], kind: str = "chunk") -> torch.Tensor:
    """[n, n] bool: query i sees key j iff j <= i and, with chunks, both lie in the same chunk counted from 0 (kind
    "window": i - j < size instead)."""
    i, j = torch.arange(n)[:, None], torch.arange(n)[None, :]
    ok = j <= i
    if chunk and kind == "window":
        ok &= i - j < chunk
    elif chunk:
        ok &= (i // chunk) == (j // chunk)
    return ok


def attention_keys_values(h: torch.Tensor, W: Dict[str, torch.Tensor], p: str, m: dict, eps: float):
    """What an attention layer leaves behind for itself and for the layers that borrow from it: keys after their norm
    (one RMS norm over the whole projection) and values."""
    k = rms_div(h @ W[p + "k"].T, eps) * W[p + "k.norm"]
    v = h @ W[p + "v"].T
    return k, v


def attention(h: torch.Tensor, W: Dict[str, torch.Tensor], p: str, m: dict, eps: float, k: torch.Tensor,
              v: torch.Tensor) -> torch.Tensor:
    n, H, D, V = h.shape[0], m["heads"], m["dim"], m["vdim"]
    G = m.get("kv_heads", H)
    q = (rms_div(h @ W[p + "q"].T, eps) * W[p + "q.norm"]).reshape(n, H, D)
    k, v = k.reshape(n, G, D), v.reshape(n, G, V)
    see = visible(n, (m.get("mask") or {}).get("size"), (m.get("mask") or {}).get("kind", "chunk"))
    dist = (torch.arange(n)[:, None] - torch.arange(n)[None, :]).to(F)
    slopes = head_slopes(H)
    out = torch.zeros(n, H, V, dtype=F)
    for hd in range(H):
        g = hd // (H // G)
        score = (q[:, hd] @ k[:, g].T) * m["scale"] - slopes[hd] * dist
        score = score.masked_fill(~see, float("-inf"))
        out[:, hd] = torch.softmax(score, dim=-1) @ v[:, g]
    return out.reshape(n, H * V) @ W[p + "o"].T


def hgrn2(h: torch.Tensor, W: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    """Gated linear recurrence, token by token: S <- diag(f) S + (1 - f) v^T, o = S^T q."""
    n, H, D, V = h.shape[0], m["heads"], m["dim"], m["vdim"]
    q = torch.nn.functional.silu(h @ W[p + "q"].T).reshape(n, H, D)
    v = (h @ W[p + "v"].T).reshape(n, H, V)
    low = W[p + "lower"]
    f = (low + (1.0 - low) * torch.sigmoid(h @ W[p + "f"].T + W[p + "f.b"])).reshape(n, H, D)
    S = torch.zeros(H, D, V, dtype=F)
    out = torch.zeros(n, H, V, dtype=F)
    for t in range(n):
        S = f[t][:, :, None] * S + (1.0 - f[t])[:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hd,hdv->hv", q[t], S)
    out = rms_div(out, eps) * W[p + "norm"]
    return out.reshape(n, H * V) @ W[p + "o"].T


def poly_norm(z: torch.Tensor, coef: torch.Tensor, eps: float) -> torch.Tensor:
    a, b, c, e = coef.tolist()
    return a * rms_div(z, eps) + b * rms_div(z ** 2, eps) + c * rms_div(z ** 3, eps) + e


def dense_ff(h, W, p, eps):
    return poly_norm(h @ W[p + "up"].T, W[p + "act"], eps) @ W[p + "down"].T


def relu_squared_expert(h, W, p):
    return (torch.relu(h @ W[p + "up"].T) ** 2) @ W[p + "down"].T


def route(h: torch.Tensor, W: Dict[str, torch.Tensor], p: str, router: dict):
    """-> (chosen experts [n, top], their weights [n, top])."""
    s = torch.softmax(h @ W[p + "router"].T, dim=-1)
    choice = s + W[p + "correction"] if p + "correction" in W else s
    idx = torch.topk(choice, router["top"], dim=-1).indices
    w = torch.gather(s, 1, idx)
    w = w / (w.sum(dim=-1, keepdim=True) + 1e-20) * router.get("scale", 1.0)
    return idx, w


def moe_ff(h, W, p, mlp):
    idx, w = route(h, W, p, mlp["router"])
    out = torch.zeros(h.shape[0], W[p + "e0.down"].shape[0], dtype=F)
    for t in range(h.shape[0]):
        for k in range(idx.shape[1]):
            out[t] += w[t, k] * relu_squared_expert(h[t:t + 1], W, f"{p}e{int(idx[t, k])}.")[0]
    if mlp.get("shared"):
        gate = torch.sigmoid(h @ W[p + "shared.sg"].T)
        out = out + gate * relu_squared_expert(h, W, p + "shared.")
    return out


def forward(cfg: dict, weights: Dict[str, torch.Tensor], tokens: List[int], layers_out: Optional[list] = None) -> torch.Tensor:
    """Logits [n, vocab] of one whole sequence; layers_out (a list) receives what every layer passes on (after the depth average)."""
    W = {k: v.to(F) for k, v in weights.items()}
    eps, m_res = cfg["norm"]["eps"], cfg.get("residual_mult", 1.0)
    n = len(tokens)
    x = W["embed"][torch.tensor(tokens)] + W["pos"][:n]
    levels = [x]
    kept = {}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        h = layer_norm(x, W[p + "norm1"], eps)
        if layer["type"] == "attention":
            src = m.get("kv_from")
            if src is None:
                kept[i] = attention_keys_values(h, W, p + "mix.", m, eps)
                src = i
            y = attention(h, W, p + "mix.", m, eps, *kept[src])
        elif layer["type"] == "hgrn2":
            y = hgrn2(h, W, p + "mix.", m, eps)
        else:
            raise ValueError(layer["type"])
        x = x + m_res * layer_norm(y, W[p + "norm1b"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            h = layer_norm(x, W[p + "norm2"], eps)
            y = dense_ff(h, W, p + "mlp.", eps) if mlp["kind"] == "dense" else moe_ff(h, W, p + "mlp.", mlp)
            x = x + m_res * layer_norm(y, W[p + "norm2b"], eps)
        levels.append(x)
        if p + "dwa" in W:
            x = sum(W[p + "dwa"][j] * levels[j] for j in range(i + 2))
        if layers_out is not None:
            layers_out.append(x)
    return layer_norm(x, W["final.norm"], eps) @ W["head"].T


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
