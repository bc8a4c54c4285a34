"""GPU: the Kezolix path (kernels of libhydra_mix.so, the model, the engine's scheduler / cache / state-slot managers)
against the float64 restatement in tests/kezolix_oracle.py.  Small made-up configurations and random weights; float32
runs are held to a tight tolerance (a chunk edge that is one token off, a lost state or a stale page moves the logits by
percents), bfloat16 runs to a loose one."""
import json
import math
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import kezolix_oracle as oracle  # noqa: E402

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
TOL32, TOL16 = 2e-4, 6e-2


@pytest.fixture(autouse=True)
def _leave_the_device_rng_alone():
    state = torch.cuda.get_rng_state(DEV) if torch.cuda.is_available() else None
    yield
    if state is not None:
        torch.cuda.set_rng_state(state, DEV)


def _shape(kind: str):
    from hydrainfer_amd.model.kezolix import FeedForwardSpec as F, KezolixLayer as L, KezolixShape, MixerSpec as M
    att = lambda *a, **k: M("attention", *a, **k)
    rec = lambda h, d, v: M("hgrn2", h, d, v)
    moe = lambda ff, e, top, scale, shared: F("moe", ff, e, top, scale, shared)
    if kind == "hybrid":      # attention first, a borrower two layers later, a layer without feed-forward, chunks of 13 and 7
        return KezolixShape(97, 96, [L(att(6, 16, 24, 2, 0.3, 13), F("dense", 72)),
                                     L(rec(3, 16, 40), moe(32, 5, 2, 1.7, 48)),
                                     L(att(6, 16, 24, 2, 0.2, 7, kv_from=0), None),
                                     L(rec(1, 24, 72), moe(64, 9, 3, 0.8, None)),
                                     L(att(2, 32, 8, 1, 0.25, None), F("dense", 40)),
                                     L(att(4, 8, 16, 2, 0.35, 9, mask="window"), None)],      # (a sliding window: the kernel's third mask)
                            max_position_embeddings=256, norm_eps=1e-5, residual_mult=0.4)
    if kind == "odd":         # nothing a multiple of four or of sixteen: every kernel's element-by-element path; top 1
        return KezolixShape(45, 38, [L(rec(3, 6, 10), F("dense", 26)),
                                     L(att(3, 5, 7, 3, 0.45, 5), moe(11, 3, 1, 1.0, 9)),
                                     L(rec(2, 9, 70), None),
                                     L(att(3, 5, 7, 3, 0.5, 11, kv_from=1), moe(6, 7, 7, 2.5, None))],
                            max_position_embeddings=200, norm_eps=1e-4, residual_mult=1.0)
    if kind == "attention":   # no recurrent layer: no state slots; heads == kv heads; more experts than a wave has lanes
        return KezolixShape(130, 128, [L(att(4, 32, 32, 4, 0.18, 16), moe(32, 70, 4, 1.0, 32)),
                                       L(att(8, 16, 64, 2, 0.25, 64), F("dense", 96))],
                            max_position_embeddings=300, norm_eps=1e-6, residual_mult=0.5)
    if kind == "recurrent":   # no attention layer: the cache pool has a plane nobody uses; wide states
        return KezolixShape(61, 64, [L(rec(2, 64, 128), F("dense", 48)),
                                     L(rec(1, 130, 32), moe(32, 4, 2, 1.2, 16)),
                                     L(rec(4, 8, 16), None)],
                            max_position_embeddings=300, norm_eps=1e-5, residual_mult=0.7)
    raise KeyError(kind)


def _weights(shape, seed=0, optional=True):
    from hydrainfer_amd.model.kezolix import tensor_shapes
    g = torch.Generator().manual_seed(seed)
    W = {}
    for k, s in tensor_shapes(shape).items():
        leaf = k.split(".", 1)[-1] if k[0] == "l" and k[1].isdigit() else k
        if not optional and leaf in ("dwa", "mlp.correction"):
            continue
        if "norm" in leaf:
            t = 1.0 + 0.2 * torch.randn(s, generator=g)
        elif leaf == "mix.lower":
            t = torch.rand(s, generator=g)
        elif leaf == "dwa":
            t = 0.5 * torch.randn(s, generator=g) / math.sqrt(s[0])
            t[-1] += 0.8
        elif leaf == "mlp.correction":
            t = 0.3 * torch.randn(s, generator=g)          # large enough to change which experts are chosen
        elif leaf == "mlp.act":
            t = torch.randn(s, generator=g)
        elif leaf.endswith(".b") or k in ("embed", "pos"):
            t = torch.randn(s, generator=g)
        elif leaf == "mlp.router":
            t = 3.0 * torch.randn(s, generator=g) / math.sqrt(s[-1])      # scores apart: no near-ties among the chosen
        else:
            t = 1.5 * torch.randn(s, generator=g) / math.sqrt(s[-1])
        W[k] = t.to(torch.bfloat16).float()       # representable in a bfloat16 checkpoint: both dtypes see the same weights
    return W


def _model(shape, W, dtype):
    from hydrainfer_amd.model.kezolix import KezolixForCausalLM
    from hydrainfer_amd.model.llava import TextLanguageModel
    return TextLanguageModel(KezolixForCausalLM.from_state_dict(shape, W, dtype, DEV))


def _replayer(lm, dtype, max_tokens, max_live=4):
    from hydrainfer_amd.engine.trace import TraceReplayer
    return TraceReplayer(lm, dtype, DEV, max_tokens, max_live_requests=max_live)


def _tokens(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def _run(rp, requests, schedule):
    """schedule: steps of [(request, n_tokens)]; every position's logits are wanted.  Returns {request: [n, vocab]}."""
    at = {r: 0 for r in requests}
    got = {r: [] for r in requests}
    with torch.inference_mode():
        for step in schedule:
            entries, end = [], []
            for r, n in step:
                toks = requests[r][at[r]:at[r] + n]
                entries.append({"id": r, "tokens": toks, "want": list(range(len(toks)))})
                at[r] += n
                if at[r] == len(requests[r]):
                    end.append(r)
            lg = rp.step(entries, end).float().cpu()
            o = 0
            for e in entries:
                got[e["id"]].append(lg[o:o + len(e["tokens"])])
                o += len(e["tokens"])
    return {r: torch.cat(v) for r, v in got.items()}


def _close(got, ref, tol, what=""):
    d = got.double().cpu() - ref
    if tol < 1e-2:
        err = d.abs().max().item() / max(1.0, ref.abs().max().item())
    else:
        err = d.pow(2).mean().sqrt().item() / max(1e-6, ref.pow(2).mean().sqrt().item())
    assert err <= tol, f"{what}: relative error {err:.3e} > {tol}"


def _dev(t, dtype=torch.float32):
    return t.to(device=DEV, dtype=dtype).contiguous()


# ------------------------------------------------------------------------------------------------ mechanisms alone
@pytest.mark.parametrize("W_,pad", [(38, 5), (96, 5), (96, 8), (1024, 8)])
def test_depth_norm_kernel_every_combination(W_, pad):
    """The residual/norm kernel: pre-norm alone, a sublayer's result entering, a level written and averaged, selected rows,
    RMS instead of layer norm.  (pad 8: rows that a lane can move four elements at a time.)"""
    from hydrainfer_amd._C.kernel.depth_ops import depth_norm
    g = torch.Generator().manual_seed(W_)
    T, n_lv = 9, 4
    x, y = torch.randn(T, W_, generator=g) * 3 + 1, torch.randn(T, W_ + pad, generator=g) * 2 - 0.5
    w1, w2 = torch.randn(W_, generator=g), torch.randn(W_, generator=g)
    levels = torch.randn(n_lv, T, W_, generator=g)
    dw = torch.randn(n_lv, generator=g)
    xd, yd = x.double(), y[:, :W_].double()
    for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 1e-2)):
        yq = y.to(dtype)
        yref = yq[:, :W_].double()
        h = depth_norm(_dev(x), dtype, 1e-5, next_w=_dev(w2))
        _close(h, oracle.layer_norm(xd, w2.double(), 1e-5), tol, "pre-norm")
        xo = torch.empty(T, W_, device=DEV)
        h = depth_norm(_dev(x), dtype, 1e-5, y=_dev(yq, dtype)[:, :W_], post_w=_dev(w1), mult=0.3, x_out=xo, next_w=_dev(w2))
        xr = xd + 0.3 * oracle.layer_norm(yref, w1.double(), 1e-5)
        _close(xo, xr, 1e-5, "residual")
        _close(h, oracle.layer_norm(xr, w2.double(), 1e-5), tol, "mid-layer norm")
        lv = _dev(levels)
        rows = torch.tensor([7, 2, 2], dtype=torch.int32, device=DEV)
        for sel in (None, rows):
            lv.copy_(levels)
            xo.zero_()
            h = depth_norm(_dev(x), dtype, 1e-5, y=_dev(yq, dtype)[:, :W_], post_w=_dev(w1), mult=0.3, level_out=lv[2], levels=lv,
                           depth_w=_dev(dw), x_out=xo, next_w=_dev(w2), rows=sel)
            full = levels.double().clone()
            full[2] = xr
            avg = (dw.double()[:, None, None] * full).sum(0)
            pick = slice(None) if sel is None else sel.cpu().long()
            _close(lv[2].cpu()[pick], xr[pick], 1e-5, "level")
            _close(xo[:T if sel is None else 3], avg[pick], 1e-5, "depth average")
            _close(h, oracle.layer_norm(avg, w2.double(), 1e-5)[pick], tol, "next norm")
        h = depth_norm(_dev(x), dtype, 1e-3, next_w=_dev(w2), rms=True)
        _close(h, oracle.rms_div(xd, 1e-3) * w2.double(), tol, "rms form")
    assert yd.shape == (T, W_)


def test_embedding_poly_norm_and_squared_relu_kernels():
    from hydrainfer_amd._C.kernel.depth_ops import embed_positions, poly_norm, relu_squared
    g = torch.Generator().manual_seed(3)
    for W_, n in ((38, 26), (128, 1000)):
        table, pos = torch.randn(50, W_, generator=g), torch.randn(30, W_, generator=g)
        ids, p = torch.randint(0, 50, (17,), generator=g), torch.randint(0, 30, (17,), generator=g)
        for dtype in (torch.float32, torch.bfloat16):
            tq, pq = table.to(dtype), pos.to(dtype)
            x = embed_positions(_dev(ids, torch.int32), _dev(p, torch.int32), _dev(tq, dtype), _dev(pq, dtype))
            assert x.dtype == torch.float32
            _close(x, tq.double()[ids] + pq.double()[p], 1e-6, "embedding + position")
            x = embed_positions(_dev(ids, torch.int64), None, _dev(tq, dtype), None)
            _close(x, tq.double()[ids], 1e-6, "embedding alone")
        z = torch.randn(7, n + 3, generator=g) * 2
        coef = torch.tensor([0.7, -0.4, 0.25, 0.1])
        for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 1e-2)):
            zq = z.to(dtype)
            out = poly_norm(_dev(zq, dtype)[:, :n], _dev(coef), 1e-5)
            _close(out, oracle.poly_norm(zq[:, :n].double(), coef.double(), 1e-5), tol, "PolyNorm")
            out = relu_squared(_dev(zq, dtype)[:, :n])
            _close(out, torch.relu(zq[:, :n].double()) ** 2, tol, "squared ReLU")


@pytest.mark.parametrize("E,top", [(5, 2), (11, 4), (70, 1), (200, 8), (9, 9)])
def test_router_choice_bias_weights_and_ties(E, top):
    from hydrainfer_amd._C.kernel.moe_mix import route_softmax_topk
    g = torch.Generator().manual_seed(E)
    T = 33
    logits = torch.randn(T, E + 1, generator=g) * 2          # one column more: the shared expert's gate rides along
    bias = torch.randn(E, generator=g) * 0.2
    for b in (bias, None):
        w, idx = route_softmax_topk(_dev(logits), E, top, 1.5, None if b is None else _dev(b))
        s = torch.softmax(logits[:, :E].double(), dim=-1)
        choice = s if b is None else s + b.double()
        want = torch.topk(choice, top, dim=-1).indices
        assert torch.equal(idx.cpu().long(), want), "chosen experts (in order of their choice scores)"
        ws = torch.gather(s, 1, want)
        _close(w, ws / (ws.sum(-1, keepdim=True) + 1e-20) * 1.5, 1e-5, "weights come from the scores without the bias")
    # equal scores: the lower expert wins
    w, idx = route_softmax_topk(_dev(torch.zeros(4, E)), E, top, 1.0, None)
    assert torch.equal(idx.cpu(), torch.arange(top, dtype=torch.int32).expand(4, top))


@pytest.mark.parametrize("dims", [(38, 11, 3, 1, 77), (96, 32, 5, 2, 77), (128, 64, 70, 4, 77), (200, 72, 3, 2, 333)])
def test_expert_plan_grouped_products_and_combine(dims):
    """(the last case: hundreds of rows an expert — the large tiles of the bfloat16 product; sizes that are multiples of 8
    but not of 32 or 64)"""
    from hydrainfer_amd._C.kernel.moe_mix import grouped_linear, moe_combine, moe_plan
    W_, ff, E, top, T = dims
    g = torch.Generator().manual_seed(ff)
    h = torch.randn(T, W_, generator=g)
    up, down = torch.randn(E, ff, W_, generator=g) / math.sqrt(W_), torch.randn(E, W_, ff, generator=g) / math.sqrt(ff)
    idx = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(T)]).to(torch.int32)
    if top == 1:
        idx[idx == 1] = 0      # an expert nobody chose
    wts = torch.rand(T, top, generator=g)
    shared, gate = torch.randn(T, W_, generator=g), torch.randn(T, 3, generator=g)
    seg, row_of, src = moe_plan(_dev(idx, torch.int32), E)
    counts = torch.bincount(idx.flatten().long(), minlength=E)
    assert torch.equal(seg.cpu().long(), torch.cat([torch.zeros(1, dtype=torch.long), counts.cumsum(0)]))
    ro, sr = row_of.cpu().long(), src.cpu().long()
    assert sorted(ro.flatten().tolist()) == list(range(T * top))
    for t in range(T):
        for k in range(top):
            e = int(idx[t, k])
            assert seg[e] <= ro[t, k] < seg[e + 1] and sr[ro[t, k]] == t
    for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 2e-2)):
        hq, uq, dq, sq = h.to(dtype), up.to(dtype), down.to(dtype), shared.to(dtype)
        y1 = grouped_linear(_dev(hq, dtype), _dev(uq, dtype), seg, T * top, src=src, act="relu2")
        y2 = grouped_linear(y1, _dev(dq, dtype), seg, T * top)
        out = moe_combine(y2, row_of, _dev(wts), _dev(sq, dtype), _dev(gate)[:, 1:2])
        ref = torch.zeros(T, W_, dtype=torch.float64)
        for t in range(T):
            for k in range(top):
                e = int(idx[t, k])
                a = torch.relu(hq[t].double() @ uq[e].double().T) ** 2
                if dtype == torch.bfloat16:
                    a = a.to(dtype).double()
                ref[t] += wts[t, k].double() * (a @ dq[e].double().T)
        ref += torch.sigmoid(gate[:, 1:2].double()) * sq.double()
        _close(out, ref, tol, f"moe {dtype}")
        out = moe_combine(y2, row_of, _dev(wts))
        _close(out, ref - torch.sigmoid(gate[:, 1:2].double()) * sq.double(), tol, "without a shared expert")


@pytest.mark.parametrize("H,D,V", [(3, 16, 64), (3, 6, 10), (1, 130, 32), (2, 64, 128), (1, 24, 200)])
def test_recurrence_kernel_portions_slots_and_fresh_starts(H, D, V):
    """Whole sequences, then the same cut into portions through state slots that held other sequences before."""
    from hydrainfer_amd._C.kernel.recurrence import gated_recurrence
    from hydrainfer_amd._C.kernel.stream_ops import SequenceState
    g = torch.Generator().manual_seed(D)
    lens = [37, 1, 20]
    eps = 1e-5
    Wd = {"q": torch.eye(H * D), "f": torch.eye(H * D), "f.b": torch.randn(H * D, generator=g),
          "lower": torch.rand(H * D, generator=g), "v": torch.eye(H * V), "norm": torch.randn(V, generator=g), "o": torch.eye(H * V)}
    proj = [torch.randn(n, 2 * H * D + H * V, generator=g) for n in lens]

    def ref_of(p):      # the oracle's mixer on identity projections: h = (q_pre | f_pre | v) picked apart by hand
        n = p.shape[0]
        qp, fp, v = p[:, :H * D].double(), p[:, H * D:2 * H * D].double(), p[:, 2 * H * D:].double()
        q = torch.nn.functional.silu(qp).reshape(n, H, D)
        f = (Wd["lower"].double() + (1 - Wd["lower"].double()) * torch.sigmoid(fp + Wd["f.b"].double())).reshape(n, H, D)
        S = torch.zeros(H, D, V, dtype=torch.float64)
        out = torch.zeros(n, H, V, dtype=torch.float64)
        for t in range(n):
            S = f[t][:, :, None] * S + (1 - f[t])[:, :, None] * v[t].reshape(H, V)[:, None, :]
            out[t] = torch.einsum("hd,hdv->hv", q[t], S)
        return (oracle.rms_div(out, eps) * Wd["norm"].double()).reshape(n, H * V), S

    for dtype, tol in ((torch.float32, 2e-5), (torch.bfloat16, 2e-2)):
        pq = [p.to(dtype) for p in proj]
        refs = [ref_of(p.float()) for p in pq]
        state = torch.full((4, 2, H * D * V + 3), 7.0, device=DEV)        # stale numbers: a fresh start must not read them

        def run(parts, pos0, slots):
            P = _dev(torch.cat(parts), dtype)
            q_cu = torch.tensor([0] + list(torch.tensor([p.shape[0] for p in parts]).cumsum(0)), dtype=torch.int32, device=DEV)
            pos = torch.cat([torch.arange(a, a + p.shape[0]) for a, p in zip(pos0, parts)]).to(torch.int32).to(DEV)
            seq = SequenceState(state, torch.tensor(slots, dtype=torch.int32, device=DEV), None)
            return gated_recurrence(P[:, :H * D], P[:, H * D:2 * H * D], P[:, 2 * H * D:], _dev(Wd["f.b"]), _dev(Wd["lower"]),
                                    _dev(Wd["norm"]), eps, seq, 1, q_cu, pos, H, D, V)

        out = run(pq, [0, 0, 0], [2, 0, 3])
        _close(out, torch.cat([r[0] for r in refs]), tol, "whole sequences")
        for s, (_, S) in zip([2, 0, 3], refs):
            _close(state[s, 1, :H * D * V].view(H, D, V), S, tol, "state left in the slot")
        assert torch.all(state[:, 0] == 7.0) and torch.all(state[1] == 7.0), "only the sequences' own rows are written"
        # portions: 16 + 2 + 19 tokens of the first, the third in 17 + 3, through the slots the whole runs dirtied
        a, c = pq[0], pq[2]
        o1 = run([a[:16], pq[1], c[:17]], [0, 0, 0], [3, 1, 0])
        o2 = run([a[16:18], c[17:]], [16, 17], [3, 0])
        o3 = run([a[18:]], [18], [3])
        got_a = torch.cat([o1[:16], o2[:2], o3])
        got_c = torch.cat([o1[17:], o2[2:]])
        _close(got_a, refs[0][0], tol, "first sequence in three portions")
        # single tokens through the decode step's kernel: the second sequence from a stale slot, then one more token of it
        more = torch.randn(1, 2 * H * D + H * V, generator=g).to(dtype)
        two, _ = ref_of(torch.cat([pq[1], more]).float())
        P = _dev(torch.cat([pq[1], c[:1]]), dtype)
        seq = SequenceState(state, torch.tensor([1, 2], dtype=torch.int32, device=DEV), None)
        step = lambda rows, pos0, sl: gated_recurrence(
            rows[:, :H * D], rows[:, H * D:2 * H * D], rows[:, 2 * H * D:], _dev(Wd["f.b"]), _dev(Wd["lower"]), _dev(Wd["norm"]), eps,
            SequenceState(state, torch.tensor(sl, dtype=torch.int32, device=DEV), None), 1,
            torch.arange(len(sl) + 1, dtype=torch.int32, device=DEV), torch.tensor(pos0, dtype=torch.int32, device=DEV), H, D, V, max_q_len=1)
        o = step(P, [0, 0], [1, 2])
        _close(o[:1], two[:1], tol, "decode step from position 0")
        _close(o[1:], refs[2][0][:1], tol, "decode step, second sequence of the batch")
        o = step(_dev(more, dtype), [1], [1])
        _close(o, two[1:], tol, "decode step from the slot")
        _close(got_c, refs[2][0], tol, "third sequence in two portions")


def _paged(rows_k, rows_v, block_size, G, head_size, seed, dtype):
    """Scatter every sequence's key / value rows over shuffled blocks.  Returns caches, flat block table, cu_block_lens."""
    g = torch.Generator().manual_seed(seed)
    n_blocks = sum((k.shape[0] + block_size - 1) // block_size for k in rows_k) + 3
    order = torch.randperm(n_blocks, generator=g).tolist()
    kc = torch.full((n_blocks, block_size, G, head_size), 9.0, dtype=dtype)       # stale numbers in what no token owns
    vc = torch.full((n_blocks, block_size, G, head_size), -9.0, dtype=dtype)
    table, cu = [], [0]
    for k, v in zip(rows_k, rows_v):
        nb = (k.shape[0] + block_size - 1) // block_size
        mine = [order.pop() for _ in range(nb)]
        for j in range(k.shape[0]):
            kc[mine[j // block_size], j % block_size, :, :k.shape[2]] = k[j].to(dtype)
            vc[mine[j // block_size], j % block_size, :, :v.shape[2]] = v[j].to(dtype)
        table += mine
        cu.append(len(table))
    return kc.to(DEV), vc.to(DEV), torch.tensor(table, dtype=torch.int32, device=DEV), torch.tensor(cu, dtype=torch.int32, device=DEV)


@pytest.mark.parametrize("H,G,D,V,mask,size", [(4, 2, 64, 40, "chunk", 24), (3, 3, 5, 7, "chunk", 5), (6, 1, 16, 130, "causal", 0),
                                              (2, 2, 32, 32, "window", 17), (8, 2, 128, 64, "chunk", 100)])
def test_attention_kernel_edges_far_keys_and_page_borders(H, G, D, V, mask, size):
    """One key made to stand out (query and key scaled so that its score dominates): far back, just inside and just outside
    the chunk or window, at a page border; prompts' rows and single decoded rows in one launch."""
    from hydrainfer_amd._C.kernel.biased_attn import biased_attention
    g = torch.Generator().manual_seed(D + size)
    bs, scale = 16, 0.3
    lens = [150, 33, 1]
    slopes = oracle.head_slopes(H)
    ks = [torch.randn(n, G, D, generator=g) for n in lens]
    vs = [torch.randn(n, G, V, generator=g) for n in lens]
    # queries: the last 40 rows of the first sequence (a portion), all of the second, the one token of the third
    q_pos = [list(range(110, 150)), list(range(33)), [0]]
    qs = [torch.randn(len(p), H, D, generator=g) for p in q_pos]
    # stand-out keys of sequence 0 for the query at position 149: far (3), the first of its chunk / window and the one before
    i = 149
    lo = i // size * size if mask == "chunk" else max(0, i - size + 1) if mask == "window" else 0
    for j in {3, lo, max(lo - 1, 0), 127, 128}:
        ks[0][j] *= 4.0
    qs[0][-1] *= 3.0
    for dtype, tol in ((torch.float32, 2e-5), (torch.bfloat16, 3e-2)):
        kq, vq, qq = [k.to(dtype) for k in ks], [v.to(dtype) for v in vs], [q.to(dtype) for q in qs]
        kc, vc, table, cu = _paged(kq, vq, bs, G, max(D, V), 5, dtype)
        ref = []
        for s in range(len(lens)):
            n = lens[s]
            ii, jj = torch.tensor(q_pos[s])[:, None], torch.arange(n)[None, :]
            see = jj <= ii
            if mask == "chunk":
                see &= (ii // size) == (jj // size)
            if mask == "window":
                see &= ii - jj < size
            out = torch.zeros(len(q_pos[s]), H, V, dtype=torch.float64)
            for h in range(H):
                gk = h // (H // G)
                sc = qq[s][:, h].double() @ kq[s][:, gk].double().T * scale - slopes[h] * (ii - jj).double()
                out[:, h] = torch.softmax(sc.masked_fill(~see, float("-inf")), dim=-1) @ vq[s][:, gk].double()
            ref.append(out)
        q = _dev(torch.cat(qq), dtype)
        pos = torch.tensor(sum(q_pos, []), dtype=torch.int32, device=DEV)
        tok_seq = torch.tensor(sum([[s] * len(p) for s, p in enumerate(q_pos)], []), dtype=torch.int32, device=DEV)
        q_cu = torch.tensor([0, 40, 73, 74], dtype=torch.int32, device=DEV)
        for form, max_kv in (("auto", 0), ("auto", 150), ("tile", 0), ("rows", 0)):      # (with the keys' count known the tile form may split them)
            out = biased_attention(q, kc, vc, V, tok_seq, pos, q_cu, table, cu, scale, _dev(slopes), mask, size, max_q_len=40,
                                   kv_heads=G, max_kv_len=max_kv, form=form)
            _close(out, torch.cat(ref), tol, f"attention {mask} {dtype} {form} {max_kv}")
        out = biased_attention(q, kc, vc, V, tok_seq, pos, q_cu, table, cu, scale, None, mask, size, max_q_len=40)
        assert (out.float().cpu() - torch.cat(ref).float()).abs().max() > 1e-3, "the distance bias changes the result"


@pytest.mark.parametrize("mask,size", [("causal", 0), ("chunk", 300), ("window", 257)])
def test_attention_tile_form_splits_the_keys_of_decode_steps(mask, size):
    """Single decoded tokens of sequences of unequal length: few row tiles, so every tile's keys are dealt to several waves
    and merged; one far key stands out."""
    from hydrainfer_amd._C.kernel.biased_attn import biased_attention
    g = torch.Generator().manual_seed(size)
    H, G, D, V, bs, scale = 8, 2, 64, 96, 16, 0.2
    lens = [700, 33, 1, 512, 301]
    slopes = oracle.head_slopes(H)
    ks = [torch.randn(n, G, D, generator=g).to(torch.bfloat16) for n in lens]
    vs = [torch.randn(n, G, V, generator=g).to(torch.bfloat16) for n in lens]
    qs = torch.randn(len(lens), H, D, generator=g).to(torch.bfloat16)
    ks[0][5] *= 4.0
    kc, vc, table, cu = _paged(ks, vs, bs, G, max(D, V), 6, torch.bfloat16)
    ref = []
    for s, n in enumerate(lens):
        i, jj = n - 1, torch.arange(n)
        see = jj <= i
        if mask == "chunk":
            see &= (jj // size) == (i // size)
        if mask == "window":
            see &= i - jj < size
        out = torch.zeros(H, V, dtype=torch.float64)
        for h in range(H):
            gk = h // (H // G)
            sc = ks[s][:, gk].double() @ qs[s, h].double() * scale - slopes[h] * (i - jj).double()
            out[h] = torch.softmax(sc.masked_fill(~see, float("-inf")), dim=-1) @ vs[s][:, gk].double()
        ref.append(out)
    n = len(lens)
    pos = torch.tensor([x - 1 for x in lens], dtype=torch.int32, device=DEV)
    ids = torch.arange(n, dtype=torch.int32, device=DEV)
    q_cu = torch.arange(n + 1, dtype=torch.int32, device=DEV)
    out = biased_attention(_dev(qs, torch.bfloat16), kc, vc, V, ids, pos, q_cu, table, cu, scale, _dev(slopes), mask, size,
                           max_q_len=1, max_kv_len=max(lens))
    _close(out, torch.stack(ref), 3e-2, f"decode with key splits, {mask}")


def test_query_key_norm_over_all_heads_and_cache_rows():
    from hydrainfer_amd._C.kernel.biased_attn import qk_norm_cache
    g = torch.Generator().manual_seed(1)
    T, H, G, D, V, bs = 21, 3, 3, 5, 7, 16
    proj = torch.randn(T, H * D + G * D + G * V + 2, generator=g)
    qw, kw = torch.randn(H * D, generator=g), torch.randn(G * D, generator=g)
    slots = torch.randperm(4 * bs, generator=g)[:T].to(torch.int32)
    slots[5] = -1
    for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 1e-2)):
        pq = proj.to(dtype)
        kc = torch.zeros(4, bs, G, max(D, V), dtype=dtype, device=DEV)
        vc = torch.zeros_like(kc)
        q = qk_norm_cache(_dev(pq, dtype), H * D, G * D, G * V, _dev(qw), _dev(kw), 1e-5, G, _dev(slots, torch.int32), kc, vc)
        p = pq.double()
        _close(q, oracle.rms_div(p[:, :H * D], 1e-5) * qw.double(), tol, "queries: one norm over all heads")
        kref = (oracle.rms_div(p[:, H * D:H * D + G * D], 1e-5) * kw.double()).reshape(T, G, D)
        vref = p[:, H * D + G * D:H * D + G * D + G * V].reshape(T, G, V)
        kf, vf = kc.view(-1, G, max(D, V)).cpu(), vc.view(-1, G, max(D, V)).cpu()
        for t, s in enumerate(slots.tolist()):
            if s >= 0:
                _close(kf[s, :, :D], kref[t], tol, "cached keys")
                _close(vf[s, :, :V], vref[t], tol, "cached values")
        written = {s for s in slots.tolist() if s >= 0}
        assert all(torch.all(kf[s] == 0) and torch.all(vf[s] == 0) for s in range(4 * bs) if s not in written)
        q2 = qk_norm_cache(_dev(pq, dtype)[:, :H * D], H * D, 0, 0, _dev(qw), None, 1e-5, G)      # a layer that borrows its keys
        assert torch.equal(q2, q)


# ------------------------------------------------------------------------------------------------ the model in the engine
@pytest.mark.parametrize("kind", ["hybrid", "odd", "attention", "recurrent"])
def test_whole_prompts_match_the_oracle_layer_by_layer(kind):
    shape = _shape(kind)
    W = _weights(shape, seed=11)
    toks = _tokens(70, shape.vocab_size, 4)
    passed = []
    ref = oracle.forward(shape.to_config(), W, toks, passed)
    for dtype, tol in ((torch.float32, TOL32), (torch.bfloat16, 0.1 if kind == "odd" else TOL16)):
        lm = _model(shape, W, dtype)
        rp = _replayer(lm, dtype, 128)
        lm.language_model.layer_trace = []
        got = _run(rp, {"a": toks}, [[("a", 70)]])["a"]
        trace, lm.language_model.layer_trace = lm.language_model.layer_trace, None
        assert len(trace) == len(passed) == len(shape.layers)
        for r, (a, b) in enumerate(zip(trace, passed)):
            _close(a.cpu(), b, tol, f"{kind} {dtype}: what layer {r} passes on")
        _close(got, ref, tol, f"{kind} {dtype}: logits")


def test_checkpoint_without_depth_weights_and_choice_bias():
    shape = _shape("hybrid")
    W = _weights(shape, seed=12, optional=False)
    assert "l0.dwa" not in W and "l1.mlp.correction" not in W
    toks = _tokens(40, shape.vocab_size, 5)
    ref = oracle.forward(shape.to_config(), W, toks)
    lm = _model(shape, W, torch.float32)
    got = _run(_replayer(lm, torch.float32, 64), {"a": toks}, [[("a", 17)], [("a", 23)]])["a"]
    _close(got, ref, TOL32, "no depth average / choice bias")


def test_specs_the_engine_reads():
    a, r, h = (_model(_shape(k), _weights(_shape(k)), torch.float32).language_model for k in ("attention", "recurrent", "hybrid"))
    assert a.state_spec() is None and a.cache_spec() == {"n_layers": 2, "n_tokens": 2, "n_heads": 4, "head_size": 64}
    assert r.state_spec() == {"rows": 3, "width": 2 * 64 * 128} and r.cache_spec()["n_layers"] == 1
    assert h.cache_spec() == {"n_layers": 3, "n_tokens": 2, "n_heads": 2, "head_size": 32}      # the borrower has no plane
    assert h.shape.cache_plane == {0: 0, 2: 0, 4: 1, 5: 2} and h.shape.state_row == {1: 0, 3: 1}


@pytest.mark.parametrize("kind", ["hybrid", "odd", "recurrent"])
def test_decoding_token_by_token_and_portions_of_every_size_equal_the_whole_prompt(kind):
    shape = _shape(kind)
    W = _weights(shape, seed=13)
    n = 90
    toks = _tokens(n, shape.vocab_size, 6)
    ref = oracle.forward(shape.to_config(), W, toks)
    lm = _model(shape, W, torch.float32)
    rp = _replayer(lm, torch.float32, 96)
    # from the very first token on, one token a step: the first tokens of a sequence, every chunk and page edge
    got = _run(rp, {"a": toks}, [[("a", 1)] for _ in range(n)])["a"]
    _close(got, ref, TOL32, "decoded from the first token")
    # portions down to two tokens, cut inside pages and chunks; then a long run of single tokens
    cuts = [2, 3, 2, 9, 16, 1, 15, 2, 7]
    cuts += [1] * (n - sum(cuts))
    got = _run(rp, {"b": toks}, [[("b", c)] for c in cuts])["b"]
    _close(got, ref, TOL32, "portions")
    got = _run(rp, {"c": toks}, [[("c", 33)], [("c", 31)], [("c", 26)]])["c"]
    _close(got, ref, TOL32, "three portions")


def test_mixed_batches_reused_pages_and_slots():
    """Five unequal requests through a pool for two and a half of them and three state slots: portions beside single
    tokens in one batch, requests that sit steps out, pages and slots handed on to later requests."""
    shape = _shape("hybrid")
    W = _weights(shape, seed=14)
    lens = {"a": 70, "b": 23, "c": 41, "d": 1, "e": 64}
    reqs = {r: _tokens(n, shape.vocab_size, 20 + i) for i, (r, n) in enumerate(lens.items())}
    ref = {r: oracle.forward(shape.to_config(), W, t) for r, t in reqs.items()}
    schedule = [[("a", 30), ("b", 2)], [("b", 1), ("a", 1)], [("a", 17), ("b", 20), ("c", 3)], [("c", 1)],
                [("a", 22), ("c", 30)],                                  # a ends: its pages and slot go back
                [("d", 1), ("c", 2)],                                    # d takes a's slot, ends at once
                [("e", 2), ("c", 1)], [("e", 31), ("c", 1)], [("c", 1), ("e", 1)], [("e", 30), ("c", 2)]]
    for dtype, tol in ((torch.float32, TOL32), (torch.bfloat16, TOL16)):
        lm = _model(shape, W, dtype)
        rp = _replayer(lm, dtype, 80 + 32 + 48, max_live=3)
        kv, sm = rp.node.kv_cache_block_manager, rp.node.batch_scheduler.context.state_manager
        free0 = len(kv.shared_cache.to_be_evicted)       # blocks no request holds
        assert free0 == kv.n_blocks
        got = _run(rp, reqs, schedule)
        for r in reqs:
            _close(got[r], ref[r], tol, f"request {r} in mixed batches ({dtype})")
        assert len(kv.shared_cache.to_be_evicted) == free0 and sm.get_num_available_slots() == 3
        assert sm.n_allocated_total == 5
        # and again on the used pool: every page and slot now has had an owner before
        got = _run(rp, {"a": reqs["a"], "e": reqs["e"]}, [[("a", 35), ("e", 64)], [("a", 35)]])
        _close(got["a"], ref["a"], tol, "second use of the pool")
        _close(got["e"], ref["e"], tol, "second use of the pool")


def test_long_decoding_across_chunks():
    shape = _shape("hybrid")
    W = _weights(shape, seed=15)
    toks = _tokens(10 + 150, shape.vocab_size, 8)
    ref = oracle.forward(shape.to_config(), W, toks)
    lm = _model(shape, W, torch.float32)
    got = _run(_replayer(lm, torch.float32, 160), {"a": toks}, [[("a", 10)]] + [[("a", 1)] for _ in range(150)])["a"]
    _close(got, ref, TOL32, "150 decoded tokens")


def test_greedy_generation_through_the_offline_engine():
    """The framework's own entry point: requests in, the scheduler batches prompts (chunked under a small token budget)
    and decode steps, greedy tokens out.  Compared with the oracle wherever its top-1 margin is not a near-tie."""
    from hydrainfer_amd.engine.offline import OfflineInferenceEngine, OfflineRequest
    shape = _shape("hybrid")
    W = _weights(shape, seed=16)
    lm = _model(shape, W, torch.float32)
    eng = OfflineInferenceEngine(lm, None, torch.float32, device=DEV, max_running_requests=3, token_budgets=24,
                                 max_context=96, warm_up=False)
    prompts = [_tokens(n, shape.vocab_size, 30 + i) for i, n in enumerate((37, 5, 18, 50, 1))]
    n_new = 12
    outs = eng.generate([OfflineRequest(token_ids=p, max_tokens=n_new) for p in prompts])
    for p, o in zip(prompts, outs):
        want, margins = oracle.greedy(shape.to_config(), W, p, n_new)
        assert len(o.output_token_ids) == n_new
        for i, (a, b, m) in enumerate(zip(o.output_token_ids, want, margins)):
            if m < 1e-3:
                break            # a near-tie: either token is right, what follows depends on it
            assert a == b, f"prompt of {len(p)}: token {i} is {a}, the oracle says {b} (margin {m:.3g})"
    kv, sm = eng.node.kv_cache_block_manager, eng.node.batch_scheduler.context.state_manager
    assert sm.get_num_available_slots() == 3 and sm.n_allocated_total == 5
    assert len(kv.shared_cache.to_be_evicted) == kv.n_blocks


def test_registry_and_trace_run_command_line(tmp_path):
    """A checkpoint directory through the registry, and bin/trace_run as a user starts it: steps on standard input,
    `done <step>` lines and .f32 files out."""
    import subprocess
    import numpy as np
    import safetensors.torch
    from hydrainfer_amd.model.registry import architecture_of, load_model
    shape = _shape("odd")
    W = _weights(shape, seed=18)
    model_dir, out_dir = tmp_path / "model", tmp_path / "out"
    model_dir.mkdir()
    (model_dir / "config.json").write_text(json.dumps(shape.to_config()))
    safetensors.torch.save_file({k: v.to(torch.bfloat16) for k, v in W.items()}, str(model_dir / "model.safetensors"))
    assert architecture_of(str(model_dir)) == "Kezolix"
    lm, vision = load_model(str(model_dir), torch.float32, DEV)
    assert vision is None and lm.language_model.shape.to_config() == shape.to_config()
    a, b = _tokens(21, shape.vocab_size, 40), _tokens(9, shape.vocab_size, 41)
    ra, rb = oracle.forward(shape.to_config(), W, a), oracle.forward(shape.to_config(), W, b)
    _close(_run(_replayer(lm, torch.float32, 32), {"a": a}, [[("a", 21)]])["a"], ra, TOL32, "loaded checkpoint")
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:17], "want": [0, 16]}], "end": []},
             {"step": 1, "entries": [{"id": "b", "tokens": b[:8], "want": []}, {"id": "a", "tokens": a[17:18], "want": [0]}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": a[18:], "want": [2]}, {"id": "b", "tokens": b[8:], "want": [0]}], "end": ["a", "b"]}]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", str(model_dir), "--dtype", "float32", "--out", str(out_dir),
                        "--max-tokens", "64"], input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True,
                       timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    read = lambda n: torch.from_numpy(np.fromfile(str(out_dir / f"{n}.f32"), dtype="<f4")).view(-1, shape.vocab_size)
    _close(read(0), ra[[0, 16]], TOL32, "step 0")
    _close(read(1), ra[[17]], TOL32, "step 1")
    _close(read(2), torch.cat([ra[[20]], rb[[8]]]), TOL32, "step 2")


def test_chat_endpoint_serves_a_checkpoint_directory(tmp_path):
    """`python -m hydrainfer_amd.entrypoint --checkpoint DIR` in parts: registry -> node -> front end -> HTTP endpoint.  The
    streams carry the tokens the offline engine generates for the same token ids."""
    import asyncio
    from types import SimpleNamespace
    import safetensors.torch
    from hydrainfer_amd.engine.offline import OfflineInferenceEngine, OfflineRequest
    from hydrainfer_amd.entrypoint.__main__ import build_checkpoint_server
    from hydrainfer_amd.entrypoint.api_protocol import parse_chat_completion_request as parse
    from tests.test_api_server import _client_stream, _payload
    shape = _shape("hybrid")
    W = _weights(shape, seed=19)
    (tmp_path / "config.json").write_text(json.dumps(shape.to_config()))
    safetensors.torch.save_file({k: v.to(torch.bfloat16) for k, v in W.items()}, str(tmp_path / "model.safetensors"))
    args = SimpleNamespace(checkpoint=str(tmp_path), max_running=4, max_tokens=128, tokenizer=None, host="127.0.0.1", port=0, dtype="fp32")
    server, front = build_checkpoint_server(args, torch.float32, torch.device(DEV))
    jobs = [("what a fine day it is today", 6), ("one two three four five six seven eight nine ten eleven twelve", 9), ("hello", 4)]

    async def go():
        await server.start()
        front.start()
        try:
            return await asyncio.gather(*[_client_stream(f"http://127.0.0.1:{server.port}/v1", _payload(t, None, n)) for t, n in jobs])
        finally:
            front.stop()
            await server.close()
    got = asyncio.run(go())
    assert front.error is None and front.n_admitted == len(jobs)
    eng = OfflineInferenceEngine.from_checkpoint(str(tmp_path), torch.float32, DEV, max_running_requests=4, max_context=128, warm_up=False)
    for (text, n_events, done), (prompt, n) in zip(got, jobs):
        assert done and n_events == n + 1 and len(text.split()) == n
        ids = server._token_request(parse(_payload(prompt, None, n))).token_ids
        want = eng.generate([OfflineRequest(token_ids=ids, max_tokens=n)])[0].output_token_ids
        assert text == "".join(server.tokenizer.decode(t) for t in want)
