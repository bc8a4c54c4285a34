"""GPU: the Tetepel path (kernels of libhydra_mix.so, the model, the engine's scheduler / cache / state-slot managers)
against the float64 restatement in tests/tetepel_oracle.py.  Small made-up configurations and random weights; float32
runs are held to a tight tolerance (a window that is one token off, a lost state row or a stale page moves the logits
by percents), bfloat16 runs to a loose one."""
import math
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import tetepel_oracle as oracle  # noqa: E402

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(autouse=True)
def _leave_the_device_rng_alone():
    """Cache pools are filled from the device's default generator; tests that come after this file keep drawing the
    numbers they drew before it existed."""
    state = torch.cuda.get_rng_state(DEV) if torch.cuda.is_available() else None
    yield
    if state is not None:
        torch.cuda.set_rng_state(state, DEV)


def _shape(kind: str):
    from hydrainfer_amd.model.tetepel import LatentAttentionSpec as A, TetepelLayer as L, TetepelShape
    if kind == "looped":        # three streams, grouped norm, a looped span, windows that differ, a layer without feed-forward
        return TetepelShape(97, 96, [L("latent_attention", A(3, 16, 8, 40, 24, 0.25, 11), 72),
                                     L("latent_attention", A(2, 8, 24, 72, 16, 0.4, 24), None),
                                     L("latent_attention", A(4, 8, 8, 24, 8, 0.3, 7), 40)],
                            loop_start=1, loop_stop=3, loop_times=2, norm_eps=1e-5, norm_groups=3, streams=3, embedding_scale=3.0)
    if kind == "plain":         # one stream, one norm group, no loop, no window on one layer, one head, window 1
        return TetepelShape(61, 40, [L("latent_attention", A(1, 12, 20, 16, 8, 0.4, None), 24),
                                     L("latent_attention", A(5, 4, 4, 136, 32, 0.5, 1), 16)],
                            norm_eps=1e-6, norm_groups=1, streams=1, embedding_scale=1.0)
    if kind == "wide":          # latents wider than 64 / 128 / 256 columns, five streams, whole model looped
        return TetepelShape(130, 128, [L("latent_attention", A(2, 32, 16, 320, 48, 0.2, 33), 64)],
                            loop_start=0, loop_stop=1, loop_times=3, norm_eps=1e-6, norm_groups=8, streams=5, embedding_scale=0.5)
    if kind == "odd":           # nothing a multiple of four: every kernel's element-by-element path, the row-form attention
        return TetepelShape(45, 38, [L("latent_attention", A(3, 6, 10, 20, 10, 0.35, 5), 26),
                                     L("latent_attention", A(2, 5, 3, 9, 7, 0.6, None), 13)],
                            loop_start=0, loop_stop=2, loop_times=2, norm_eps=1e-4, norm_groups=2, streams=2, embedding_scale=1.5)
    raise KeyError(kind)


def _weights(shape, seed=0, optional=True):
    from hydrainfer_amd.model.tetepel import tensor_shapes
    g = torch.Generator().manual_seed(seed)
    W = {}
    for k, s in tensor_shapes(shape).items():
        leaf = k.split(".", 1)[-1]
        if not optional and (leaf.startswith(("shift", "rg")) or (shape.streams == 1 and leaf.startswith("hc"))):
            continue
        if "norm" in leaf:
            t = 1.0 + 0.2 * torch.randn(s, generator=g)
        elif leaf == "shift":
            t = torch.rand(s, generator=g)
        elif leaf.startswith("hc"):
            t = 0.6 * torch.randn(s, generator=g) + (0.5 if leaf.endswith(("in", "out")) else 0.0)
        elif leaf.endswith(".b"):
            t = torch.randn(s, generator=g)
        else:
            t = 1.5 * torch.randn(s, generator=g) / math.sqrt(s[-1])
        W[k] = t.to(torch.bfloat16).float()       # representable in a bfloat16 checkpoint: both dtypes see the same weights
    return W


def _model(shape, W, dtype):
    from hydrainfer_amd.model.llava import TextLanguageModel
    from hydrainfer_amd.model.tetepel import TetepelForCausalLM
    return TextLanguageModel(TetepelForCausalLM.from_state_dict(shape, W, dtype, DEV))


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
    """float32 runs (tol < 1e-2): the largest difference against the largest value.  bfloat16 runs: root mean square of
    the difference against that of the values (single elements of a 16-bit run may be off by more than the average)."""
    d = got.double() - ref
    if tol < 1e-2:
        err = d.abs().max().item() / max(1.0, ref.abs().max().item())
    else:
        err = d.pow(2).mean().sqrt().item() / max(1e-6, ref.pow(2).mean().sqrt().item())
    assert err <= tol, f"{what}: relative error {err:.3e} > {tol}"


TOL32, TOL16 = 2e-4, 5e-2


# ------------------------------------------------------------------------------------------------ mechanisms alone
def test_stream_embed_norm_update_and_gelu_kernels():
    from hydrainfer_amd._C.kernel import stream_ops as so
    g = torch.Generator().manual_seed(1)
    for S, W_, groups in ((1, 40, 1), (3, 96, 4), (5, 136, 8), (8, 48, 3), (4, 1024, 2), (2, 512, 1), (16, 768, 3), (3, 46, 2)):
        T = 9
        table = torch.randn(30, W_, generator=g)
        ids = torch.randint(0, 30, (T,), generator=g)
        x = so.stream_embed(ids.to(DEV).to(torch.int32), table.to(DEV), 1.7, S)
        assert torch.equal(x.cpu(), (table[ids] * 1.7)[:, None, :].expand(T, S, W_))
        x = torch.randn(T, S, W_, generator=g)
        w_in, nw = torch.randn(S, generator=g), torch.randn(W_, generator=g)
        ref = oracle.grouped_rms_norm(oracle.streams_read(x.double().transpose(0, 1), w_in.double()), nw.double(), groups, 1e-5)
        h = so.stream_norm(x.to(DEV), w_in.to(DEV), nw.to(DEV), groups, 1e-5, torch.float32)
        _close(h.cpu(), ref, 1e-5, "stream_norm")
        rows = torch.tensor([7, 0, 3], dtype=torch.int32)
        h = so.stream_norm(x.to(DEV), w_in.to(DEV), nw.to(DEV), groups, 1e-5, torch.float32, rows=rows.to(DEV))
        _close(h.cpu(), ref[rows.long()], 1e-5, "stream_norm rows")
        y, gp, gb = torch.randn(T, W_, generator=g), torch.randn(T, W_ + 8, generator=g), torch.randn(W_, generator=g)
        mix, w_out = torch.randn(S, S, generator=g), torch.randn(S, generator=g)
        xd = x.to(DEV).clone()
        so.stream_update(xd, y.to(DEV), mix.to(DEV), w_out.to(DEV), gp.to(DEV)[:, :W_], gb.to(DEV))
        ref = oracle.streams_write(x.double().transpose(0, 1), y.double() * torch.sigmoid(gp[:, :W_].double() + gb.double()),
                                   mix.double(), w_out.double()).transpose(0, 1)
        _close(xd.cpu(), ref, 1e-5, "stream_update gated")
        # the update and the next sublayer's read side as one launch
        xd = x.to(DEV).clone()
        in2, nw2 = torch.randn(S, generator=g), torch.randn(W_, generator=g)
        h2 = so.stream_update_norm(xd, y.to(DEV), mix.to(DEV), w_out.to(DEV), gp.to(DEV)[:, :W_], gb.to(DEV), in2.to(DEV), nw2.to(DEV),
                                   groups, 1e-5)
        _close(xd.cpu(), ref, 1e-5, "stream_update_norm: streams")
        _close(h2.cpu(), oracle.grouped_rms_norm(oracle.streams_read(ref.transpose(0, 1), in2.double()), nw2.double(), groups, 1e-5),
               1e-5, "stream_update_norm: h")
        xd = x.to(DEV).clone()
        so.stream_update(xd, y.to(DEV), mix.to(DEV), w_out.to(DEV))
        _close(xd.cpu(), oracle.streams_write(x.double().transpose(0, 1), y.double(), mix.double(), w_out.double()).transpose(0, 1),
               1e-5, "stream_update")
    a, b = torch.randn(5, 70, generator=g) * 3, torch.randn(5, 70, generator=g)
    both = torch.cat([a, b], dim=1).to(DEV)
    _close(so.gelu_tanh_and_mul(both[:, :70], both[:, 70:]).cpu(), oracle.gelu_tanh(a.double()) * b.double(), 1e-5, "gelu")
    out16 = so.gelu_tanh_and_mul(both[:, :70].bfloat16(), both[:, 70:].bfloat16())
    _close(out16.float().cpu(), oracle.gelu_tanh(a.bfloat16().double()) * b.bfloat16().double(), 2e-2, "gelu bf16")


@pytest.mark.parametrize("W_,groups", [(48, 4), (768, 3), (50, 5)])
def test_token_shift_carries_the_previous_row_through_the_state_slot(W_, groups):
    """Two sequences in one batch, cut into portions (one of a single token, one of two): the shifted rows equal the
    shift of the whole sequences, the slot of a reused sequence number starts from zeros at position 0."""
    from hydrainfer_amd._C.kernel import stream_ops as so
    g = torch.Generator().manual_seed(2)
    S = 2
    lens = {0: 9, 1: 6}
    xs = {b: torch.randn(n, S, W_, generator=g) for b, n in lens.items()}
    w_in, nw, sh = torch.randn(S, generator=g), torch.randn(W_, generator=g), torch.rand(W_, generator=g)
    ref = {b: oracle.token_shift(oracle.grouped_rms_norm(oracle.streams_read(x.double().transpose(0, 1), w_in.double()),
                                                         nw.double(), groups, 1e-6), sh.double()) for b, x in xs.items()}
    state = torch.full((3, 2, W_), 7.0, device=DEV)        # stale rows of earlier owners: never read at position 0
    slots = {0: 2, 1: 0}
    at = {0: 0, 1: 0}
    for cut in ({0: 1, 1: 2}, {0: 5, 1: 1}, {1: 3}, {0: 2}, {0: 1}):
        seqs = sorted(cut)
        x = torch.cat([xs[b][at[b]:at[b] + cut[b]] for b in seqs])
        pos = torch.cat([torch.arange(at[b], at[b] + cut[b]) for b in seqs]).to(torch.int32)
        tok_seq = torch.cat([torch.full((cut[b],), i) for i, b in enumerate(seqs)]).to(torch.int32)
        q_cu = torch.tensor([0] + list(torch.tensor([cut[b] for b in seqs]).cumsum(0)), dtype=torch.int32)
        seq = so.SequenceState(state, torch.tensor([slots[b] for b in seqs], dtype=torch.int32, device=DEV), tok_seq.to(DEV))
        h, hs = so.stream_norm(x.to(DEV), w_in.to(DEV), nw.to(DEV), groups, 1e-6, torch.float32, shift_w=sh.to(DEV), seq=seq,
                               state_row=1, q_cu=q_cu.to(DEV), positions=pos.to(DEV))
        want = torch.cat([ref[b][at[b]:at[b] + cut[b]] for b in seqs])
        _close(hs.cpu(), want, 1e-5, f"shifted rows of portions {cut}")
        for b in seqs:
            at[b] += cut[b]
    assert torch.all(state[:, 0] == 7.0) and torch.all(state[1] == 7.0)      # other rows and slots untouched


def _paged(c_rows, block_size, row_width, seed, dtype=torch.float32):
    """Scatter per-sequence latent rows into a shuffled paged cache; returns (cache, flat block table, cu_block_lens)."""
    g = torch.Generator().manual_seed(seed)
    n_blocks = sum((len(c) + block_size - 1) // block_size for c in c_rows) + 3
    perm = torch.randperm(n_blocks, generator=g).tolist()
    cache = torch.randn(n_blocks, block_size, 1, row_width, generator=g) * 50      # garbage wherever nothing was written
    table, cu = [], [0]
    for c in c_rows:
        nb = (len(c) + block_size - 1) // block_size
        blocks, perm = perm[:nb], perm[nb:]
        for j in range(len(c)):
            cache[blocks[j // block_size], j % block_size, 0, :c.shape[1]] = c[j]
        table += blocks
        cu.append(len(table))
    return cache.to(dtype).to(DEV), torch.tensor(table, dtype=torch.int32, device=DEV), torch.tensor(cu, dtype=torch.int32, device=DEV)


@pytest.mark.parametrize("R,H,window", [(40, 3, 17), (128, 8, 100), (320, 2, None), (64, 1, 1), (72, 5, 16), (48, 2, 9), (104, 4, 40),
                                            (80, 3, None), (200, 2, 64), (8, 16, 5), (112, 1, 300), (328, 3, 29), (512, 2, None)])
def test_latent_attention_kernel_window_edges_page_borders_and_far_keys(R, H, window):
    """One key is made to stand out (the query is a multiple of its row): just inside the window, just outside it, on
    both sides of a page border, and the sequence's first key hundreds of positions back."""
    from hydrainfer_amd._C.kernel.latent_attn import latent_attention
    g = torch.Generator().manual_seed(R + H)
    n_ctx = [300, 45]
    c_rows = [torch.randn(n, R, generator=g) for n in n_ctx]
    cache, table, cu_blocks = _paged(c_rows, 16, R + 8, seed=5)
    w = window or 10 ** 9
    queries = []          # (sequence, position, key that stands out)
    for pos in (299, 200, 31, 16, 15, 0):
        for target in (pos - w + 1, pos - w, pos - w + 2, 0, 15, 16, pos - 1, pos):
            if 0 <= target <= pos:
                queries.append((0, pos, target))
    queries += [(1, 44, 44 - w + 1 if 44 - w + 1 >= 0 else 0), (1, 44, max(0, 44 - w)), (1, 0, 0)]
    T = len(queries)
    q = torch.randn(T, H, R, generator=g) * 0.3
    for t, (b, pos, target) in enumerate(queries):
        q[t, t % H] += 9.0 * c_rows[b][target] / c_rows[b][target].norm() ** 2 * math.sqrt(R)
    scale = 1.0 / math.sqrt(R)
    gate = torch.randn(T, H + 2, generator=g)
    def reference(dtype):      # from the operands as the kernel sees them (rounded to its dtype)
        ref = torch.zeros(T, H, R, dtype=torch.float64)
        qr, gr = q.to(dtype).double(), gate.to(dtype).double()
        for t, (b, pos, target) in enumerate(queries):
            lo = max(0, pos - w + 1)
            keys = c_rows[b][lo:pos + 1].to(dtype).double()
            for h in range(H):
                p = torch.softmax(keys @ qr[t, h] * scale, dim=0)
                ref[t, h] = (p[:, None] * keys).sum(0) * torch.sigmoid(gr[t, h])
        return ref
    tok_seq = torch.tensor([b for b, _, _ in queries], dtype=torch.int32)
    positions = torch.tensor([p for _, p, _ in queries], dtype=torch.int32)
    # the rows of a batch lie sequence by sequence
    order = sorted(range(T), key=lambda t: queries[t][0])
    q_cu = torch.tensor([0, sum(1 for b, _, _ in queries if b == 0), T], dtype=torch.int32)
    idx = torch.tensor(order)
    for dtype, tol in ((torch.float32, 2e-5), (torch.bfloat16, 1e-2)):
        ref = reference(dtype)
        ch = cache.to(dtype)
        qd = q[idx].to(dtype).to(DEV)
        out = latent_attention(qd, ch, tok_seq[idx].to(DEV), positions[idx].to(DEV), q_cu.to(DEV), table, cu_blocks, scale,
                               window, int(q_cu.diff().max()), gate_pre=gate[idx].to(dtype).to(DEV), max_kv_len=max(n_ctx))
        _close(out.float().cpu(), ref[idx], tol, f"latent attention {dtype}")
        # without key splits (no bound on the keys given): wide latents then take the group form, four waves a chunk
        whole = latent_attention(qd, ch, tok_seq[idx].to(DEV), positions[idx].to(DEV), q_cu.to(DEV), table, cu_blocks, scale,
                                 window, int(q_cu.diff().max()), gate_pre=gate[idx].to(dtype).to(DEV))
        _close(whole.float().cpu(), ref[idx], tol, f"latent attention {dtype}, no key splits")
        # strided query / result layouts (heads outermost), as the model hands them over
        qh = qd.transpose(0, 1).contiguous()
        oh = torch.empty_like(qh)
        latent_attention(qh.transpose(0, 1), ch, tok_seq[idx].to(DEV), positions[idx].to(DEV), q_cu.to(DEV), table, cu_blocks,
                         scale, window, int(q_cu.diff().max()), gate_pre=gate[idx].to(dtype).to(DEV), out=oh.transpose(0, 1), max_kv_len=max(n_ctx))
        assert torch.equal(oh.transpose(0, 1), out)
        if dtype == torch.bfloat16:      # the row form of the same kernel (what float32 runs on) agrees with the tile form
            from hydrainfer_amd import _lib
            _lib.mix_lib().hxm_set_option(b"attn_tile_form", 0)
            try:
                rows = latent_attention(qd, ch, tok_seq[idx].to(DEV), positions[idx].to(DEV), q_cu.to(DEV), table, cu_blocks,
                                        scale, window, int(q_cu.diff().max()), gate_pre=gate[idx].to(dtype).to(DEV), max_kv_len=max(n_ctx))
            finally:
                _lib.mix_lib().hxm_set_option(b"attn_tile_form", 1)
            _close(rows.float().cpu(), ref[idx], tol, "latent attention, row form in bfloat16")


def test_latent_norm_cache_kernel_writes_the_rows_it_is_told_to():
    from hydrainfer_amd._C.kernel.latent_attn import latent_norm_cache
    g = torch.Generator().manual_seed(3)
    T, qr, R, extra = 7, 24, 40, 3
    proj = torch.randn(T, qr + R + extra, generator=g) * 2
    qw, kw = torch.randn(qr, generator=g), torch.randn(R, generator=g)
    cache = torch.zeros(6, 16, 1, R + 8, device=DEV)
    slots = torch.tensor([95, 0, 15, 16, -1, 31, 47], dtype=torch.int32)
    cq = latent_norm_cache(proj.to(DEV), 0, qr, qr, R, qw.to(DEV), kw.to(DEV), 1e-6, slots.to(DEV), cache)
    _close(cq.cpu(), oracle.grouped_rms_norm(proj[:, :qr].double(), qw.double(), 1, 1e-6), 1e-5, "query latent")
    c = oracle.grouped_rms_norm(proj[:, qr:qr + R].double(), kw.double(), 1, 1e-6)
    flat = cache.view(-1, R + 8).cpu()
    for t, s in enumerate(slots.tolist()):
        if s >= 0:
            _close(flat[s, :R], c[t], 1e-5, "cached latent")
    written = {s for s in slots.tolist() if s >= 0}
    assert all(torch.all(flat[s] == 0) for s in range(flat.shape[0]) if s not in written)
    assert torch.all(flat[:, R:] == 0)


# ------------------------------------------------------------------------------------------------ the model in the engine
@pytest.mark.parametrize("kind", ["looped", "plain", "wide", "odd"])
def test_whole_prompts_match_the_oracle_layer_by_layer(kind):
    shape = _shape(kind)
    W = _weights(shape, seed=11)
    toks = _tokens(70, shape.vocab_size, 4)
    sums = []
    ref = oracle.forward(shape.to_config(), W, toks, sums)
    # (bfloat16 rounding averages out over fewer terms in 9-column latents and 19-element norm groups)
    for dtype, tol in ((torch.float32, TOL32), (torch.bfloat16, 8e-2 if kind == "odd" else TOL16)):
        lm = _model(shape, W, dtype)
        rp = _replayer(lm, dtype, 128)
        lm.language_model.layer_trace = []
        got = _run(rp, {"a": toks}, [[("a", 70)]])["a"]
        trace, lm.language_model.layer_trace = lm.language_model.layer_trace, None
        assert len(trace) == len(sums) == shape.num_hidden_layers
        for r, (a, b) in enumerate(zip(trace, sums)):
            _close(a.cpu(), b, tol, f"{kind} {dtype}: sum of the streams after layer run {r}")
        _close(got, ref, tol, f"{kind} {dtype}: logits")


def test_checkpoint_without_shift_gates_and_stream_weights():
    shape = _shape("plain")
    W = _weights(shape, seed=12, optional=False)
    assert "l0.shift" not in W and "l0.rg1" not in W and "l0.hc1.in" not in W
    toks = _tokens(40, shape.vocab_size, 5)
    ref = oracle.forward(shape.to_config(), W, toks)
    lm = _model(shape, W, torch.float32)
    assert lm.language_model.state_spec() is None
    got = _run(_replayer(lm, torch.float32, 64), {"a": toks}, [[("a", 17)], [("a", 23)]])["a"]
    _close(got, ref, TOL32, "no shift / gates / stream weights")


@pytest.mark.parametrize("kind", ["looped", "wide", "odd"])
def test_decoding_token_by_token_and_portions_of_every_size_equal_the_whole_prompt(kind):
    shape = _shape(kind)
    W = _weights(shape, seed=13)
    n = 90
    toks = _tokens(n, shape.vocab_size, 6)
    ref = oracle.forward(shape.to_config(), W, toks)
    lm = _model(shape, W, torch.float32)
    rp = _replayer(lm, torch.float32, 96)
    # from the very first token on, one token a step: the first tokens of a sequence, every window and page edge
    got = _run(rp, {"a": toks}, [[("a", 1)] for _ in range(n)])["a"]
    _close(got, ref, TOL32, "decoded from the first token")
    # portions down to two tokens, cut inside pages and windows; then a long run of single tokens
    cuts = [2, 3, 2, 9, 16, 1, 15, 2, 7]
    cuts += [1] * (n - sum(cuts))
    got = _run(rp, {"b": toks}, [[("b", c)] for c in cuts])["b"]
    _close(got, ref, TOL32, "portions")
    got = _run(rp, {"c": toks}, [[("c", 33)], [("c", 31)], [("c", 26)]])["c"]
    _close(got, ref, TOL32, "three portions")


def test_mixed_batches_reused_pages_and_slots():
    """Five unequal requests through a pool for two and a half of them and three state slots: portions beside single
    tokens in one batch, requests that sit steps out, pages and slots handed on to later requests."""
    shape = _shape("looped")
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


def test_long_decoding_past_the_window():
    shape = _shape("looped")
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
    shape = _shape("looped")
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


def test_registry_loads_a_checkpoint_directory(tmp_path):
    import json
    import safetensors.torch
    from hydrainfer_amd.model.registry import architecture_of, load_model
    shape = _shape("plain")
    W = _weights(shape, seed=17)
    (tmp_path / "config.json").write_text(json.dumps(shape.to_config()))
    safetensors.torch.save_file({k: v.to(torch.bfloat16) for k, v in W.items()}, str(tmp_path / "model.safetensors"))
    assert architecture_of(str(tmp_path)) == "Tetepel"
    lm, vision = load_model(str(tmp_path), torch.float32, DEV)
    assert vision is None and lm.language_model.shape.run_order == shape.run_order
    toks = _tokens(20, shape.vocab_size, 9)
    got = _run(_replayer(lm, torch.float32, 32), {"a": toks}, [[("a", 20)]])["a"]
    _close(got, oracle.forward(shape.to_config(), W, toks), TOL32, "loaded checkpoint")


def test_trace_run_command_line(tmp_path):
    """bin/trace_run as a user starts it: steps on standard input, `done <step>` lines and .f32 files out."""
    import json
    import subprocess
    import numpy as np
    import safetensors.torch
    shape = _shape("looped")
    W = _weights(shape, seed=18)
    model_dir, out_dir = tmp_path / "model", tmp_path / "out"
    model_dir.mkdir()
    (model_dir / "config.json").write_text(json.dumps(shape.to_config()))
    safetensors.torch.save_file({k: v.to(torch.bfloat16) for k, v in W.items()}, str(model_dir / "model.safetensors"))
    a, b = _tokens(21, shape.vocab_size, 40), _tokens(9, shape.vocab_size, 41)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:17], "want": [0, 16]}], "end": []},
             {"step": 1, "entries": [{"id": "b", "tokens": b[:8], "want": []}, {"id": "a", "tokens": a[17:18], "want": [0]}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": a[18:], "want": [2]}, {"id": "b", "tokens": b[8:], "want": [0]}], "end": ["a", "b"]}]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", str(model_dir), "--dtype", "float32", "--out", str(out_dir),
                        "--max-tokens", "64"], input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True,
                       timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    ra, rb = oracle.forward(shape.to_config(), W, a), oracle.forward(shape.to_config(), W, b)
    read = lambda n: torch.from_numpy(np.fromfile(str(out_dir / f"{n}.f32"), dtype="<f4")).view(-1, shape.vocab_size)
    _close(read(0), ra[[0, 16]], TOL32, "step 0")
    _close(read(1), ra[[17]], TOL32, "step 1")
    _close(read(2), torch.cat([ra[[20]], rb[[8]]]), TOL32, "step 2")


@pytest.mark.parametrize("lens", [(1500, 700, 100), (3000, 1201, 50, 1)])
def test_token_shift_in_long_batches(lens):
    """Thousands of rows in one launch: a workgroup then takes several consecutive rows and hands h from one to the next;
    sequence borders fall inside such runs."""
    from hydrainfer_amd._C.kernel import stream_ops as so
    g = torch.Generator().manual_seed(7)
    S, W_, groups = 3, 56, 7
    xs = [torch.randn(n, S, W_, generator=g) for n in lens]
    w_in, nw, sh = torch.randn(S, generator=g), torch.randn(W_, generator=g), torch.rand(W_, generator=g)
    norm = lambda x: oracle.grouped_rms_norm(oracle.streams_read(x.double().transpose(0, 1), w_in.double()), nw.double(), groups, 1e-6)
    ref = torch.cat([oracle.token_shift(norm(x), sh.double()) for x in xs])
    state = torch.zeros((len(lens), 1, W_), device=DEV)
    q_cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    pos = torch.cat([torch.arange(n) for n in lens]).to(torch.int32)
    tok_seq = torch.cat([torch.full((n,), i) for i, n in enumerate(lens)]).to(torch.int32)
    seq = so.SequenceState(state, torch.arange(len(lens), dtype=torch.int32, device=DEV), tok_seq.to(DEV))
    h, hs = so.stream_norm(torch.cat(xs).to(DEV), w_in.to(DEV), nw.to(DEV), groups, 1e-6, torch.float32, shift_w=sh.to(DEV), seq=seq,
                           q_cu=q_cu.to(DEV), positions=pos.to(DEV))
    _close(hs.cpu(), ref, 1e-5, "shifted rows")
    _close(h.cpu(), torch.cat([norm(x) for x in xs]), 1e-5, "plain rows")
    _close(state[:, 0].cpu(), torch.stack([norm(x)[-1] for x in xs]), 1e-5, "state rows: the h of every sequence's last token")


def test_chat_endpoint_serves_a_checkpoint_directory(tmp_path):
    """`python -m hydrainfer_amd.entrypoint --checkpoint DIR` in parts: registry -> node -> front end -> HTTP endpoint.  The
    streams carry the tokens the offline engine generates for the same token ids."""
    import asyncio
    import json
    from types import SimpleNamespace
    import safetensors.torch
    from hydrainfer_amd.engine.offline import OfflineInferenceEngine, OfflineRequest
    from hydrainfer_amd.entrypoint.__main__ import build_checkpoint_server
    from tests.test_api_server import _client_stream, _payload
    shape = _shape("looped")
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
    from hydrainfer_amd.entrypoint.api_protocol import parse_chat_completion_request as parse
    eng = OfflineInferenceEngine.from_checkpoint(str(tmp_path), torch.float32, DEV, max_running_requests=4, max_context=128, warm_up=False)
    for (text, n_events, done), (prompt, n) in zip(got, jobs):
        assert done and n_events == n + 1 and len(text.split()) == n
        ids = server._token_request(parse(_payload(prompt, None, n))).token_ids
        want = eng.generate([OfflineRequest(token_ids=ids, max_tokens=n)])[0].output_token_ids
        assert text == "".join(server.tokenizer.decode(t) for t in want)
