"""CPU: the host side of the Kezolix integration — configuration reading, cache planes and state rows, tensor names, the
model registry, the mix library's exports — and the float64 restatement's own mechanisms on cases worked out by hand."""
import json

import pytest
import torch

import tests.kezolix_oracle as oracle
from hydrainfer_amd.model.kezolix import KezolixForCausalLM, KezolixShape, tensor_shapes


def _config(**over):
    att = {"heads": 6, "kv_heads": 2, "dim": 8, "vdim": 12, "scale": 0.25, "mask": {"size": 9}}
    rec = {"heads": 3, "dim": 4, "vdim": 10}
    moe = {"kind": "moe", "expert": {"ff": 16}, "router": {"experts": 5, "top": 2, "scale": 1.25}, "shared": {"ff": 24}}
    cfg = {"architecture": "Kezolix", "vocab": 33, "width": 24, "max_positions": 77, "norm": {"eps": 1e-4}, "residual_mult": 0.6,
           "layers": [{"type": "hgrn2", "mixer": dict(rec), "mlp": {"kind": "dense", "ff": 40}},
                      {"type": "attention", "mixer": dict(att), "mlp": dict(moe)},
                      {"type": "attention", "mixer": dict(att, mask=None, kv_heads=6), "mlp": None},
                      {"type": "hgrn2", "mixer": dict(rec, heads=1), "mlp": dict(moe, shared=None)},
                      {"type": "attention", "mixer": dict(att, kv_from=1, mask={"size": 4}), "mlp": {"kind": "dense", "ff": 8}}]}
    cfg.update(over)
    return cfg


def test_shape_from_config_planes_rows_and_names():
    sh = KezolixShape.from_config(_config())
    assert sh.cache_plane == {1: 0, 2: 1, 4: 0} and sh.state_row == {0: 0, 3: 1} and sh.num_hidden_layers == 2
    assert sh.head_dim == 12 and sh.num_key_value_heads == 6 and sh.num_attention_heads == 6
    assert sh.max_position_embeddings == 77 and sh.norm_eps == 1e-4 and sh.residual_mult == 0.6
    assert sh.layers[2].mixer.chunk is None and sh.layers[4].mixer.chunk == 4 and sh.layers[2].mlp is None
    assert sh.layers[3].mlp.shared_ff is None and sh.layers[1].mlp.shared_ff == 24 and sh.layers[1].mlp.router_scale == 1.25
    assert KezolixShape.from_config(sh.to_config()).to_config() == sh.to_config()
    w = _config()
    w["layers"][2]["mixer"]["mask"] = {"kind": "window", "size": 6}
    ws = KezolixShape.from_config(w)
    assert (ws.layers[2].mixer.mask, ws.layers[2].mixer.chunk) == ("window", 6) and ws.to_config()["layers"][2]["mixer"]["mask"] == {"kind": "window", "size": 6}
    names = tensor_shapes(sh)
    assert names["l1.mix.k"] == (16, 24) and names["l1.mix.k.norm"] == (16,) and names["l1.mix.q.norm"] == (48,)
    assert "l4.mix.k" not in names and "l4.mix.v" not in names and names["l4.mix.o"] == (24, 72)
    assert names["l0.mix.lower"] == (12,) and names["l0.mix.norm"] == (10,) and names["l3.dwa"] == (5,)
    assert names["l1.mlp.e4.down"] == (24, 16) and names["l1.mlp.shared.sg"] == (1, 24) and "l3.mlp.shared.up" not in names
    assert "l2.norm2" not in names and names["pos"] == (77, 24) and names["head"] == (33, 24)
    sd = KezolixForCausalLM.random_state_dict(sh, seed=1)
    assert set(sd) == set(names) and all(tuple(sd[k].shape) == v for k, v in names.items())


def test_configurations_that_cannot_be():
    with pytest.raises(ValueError):
        KezolixShape.from_config(_config(architecture="Other"))
    bad = _config()
    bad["layers"][4]["mixer"]["kv_from"] = 0              # a recurrent layer has no keys to lend
    with pytest.raises(ValueError):
        KezolixShape.from_config(bad)
    bad = _config()
    bad["layers"][4]["mixer"]["dim"] = 16                 # a borrower's keys have the lender's shape
    with pytest.raises(ValueError):
        KezolixShape.from_config(bad)
    bad = _config()
    bad["layers"][1]["mixer"]["kv_from"] = 2              # only earlier layers lend
    with pytest.raises(ValueError):
        KezolixShape.from_config(bad)
    bad = _config()
    bad["layers"][0]["type"] = "other"
    with pytest.raises(ValueError):
        KezolixShape.from_config(bad)


def test_registry_names_the_architecture(tmp_path):
    from hydrainfer_amd.model.registry import architecture_of, registered
    (tmp_path / "config.json").write_text(json.dumps(_config()))
    assert architecture_of(str(tmp_path)) == "Kezolix" and "Kezolix" in registered()


def test_mix_library_header_and_binding_agree():
    import os
    import re
    from hydrainfer_amd import _lib
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    header = open(os.path.join(root, "include", "hydra_mix.h")).read()
    declared = set(re.findall(r"^(?:int|int64_t) (hxm_\w+)\(", header, flags=re.M))
    assert declared == set(_lib._MIX_SIGNATURES)
    assert int(re.search(r"#define HXM_ABI_VERSION (\d+)", header).group(1)) == _lib.HXM_ABI_VERSION


# ------------------------------------------------------------------------------------------------ the restatement itself
def test_oracle_mask_slopes_and_norms_by_hand():
    see = oracle.visible(7, 3)
    assert see[5].tolist() == [False, False, False, True, True, True, False]
    assert see[3].tolist() == [False, False, False, True, False, False, False]
    assert oracle.visible(4, None)[3].tolist() == [True] * 4
    assert torch.allclose(oracle.head_slopes(4), torch.tensor([0.25, 0.0625, 0.015625, 0.00390625], dtype=torch.float64))
    x = torch.tensor([[1.0, 3.0]], dtype=torch.float64)
    assert torch.allclose(oracle.layer_norm(x, torch.tensor([2.0, 1.0], dtype=torch.float64), 0.0), torch.tensor([[-2.0, 1.0]], dtype=torch.float64))
    assert torch.allclose(oracle.rms_div(x, 0.0), x / 5.0 ** 0.5)


def test_oracle_router_weights_come_from_the_unbiased_scores():
    W = {"r.router": torch.eye(3, dtype=torch.float64), "r.correction": torch.tensor([0.0, 0.0, 10.0], dtype=torch.float64)}
    h = torch.tensor([[2.0, 1.0, 0.0]], dtype=torch.float64)
    idx, w = oracle.route(h, W, "r.", {"top": 2, "scale": 3.0})
    s = torch.softmax(h, dim=-1)[0]
    assert idx.tolist() == [[2, 0]]                       # the bias lifts expert 2 to the front
    assert torch.allclose(w[0], torch.stack([s[2], s[0]]) / (s[2] + s[0]) * 3.0)


def test_oracle_recurrence_one_channel_by_hand():
    # one head, one key channel, one value channel, identity projections: S_t = f S_(t-1) + (1 - f) v_t, o = silu(q) S
    W = {"m.q": torch.tensor([[1.0, 0.0, 0.0]]), "m.f": torch.tensor([[0.0, 1.0, 0.0]]), "m.v": torch.tensor([[0.0, 0.0, 1.0]]),
         "m.f.b": torch.zeros(1), "m.lower": torch.tensor([0.5]), "m.norm": torch.ones(1), "m.o": torch.ones(1, 1)}
    W = {k: v.double() for k, v in W.items()}
    h = torch.tensor([[1.0, 0.0, 2.0], [1.0, 0.0, -4.0]], dtype=torch.float64)
    out = oracle.hgrn2(h, W, "m.", {"heads": 1, "dim": 1, "vdim": 1}, 0.0)
    f = 0.5 + 0.5 * 0.5                                   # sigmoid(0) = 0.5
    s1 = (1 - f) * 2.0
    s2 = f * s1 + (1 - f) * -4.0
    assert out[:, 0].tolist() == [1.0, -1.0] and s1 > 0 > s2      # one value channel: the norm leaves the sign
