"""CPU: the host side of the Tetepel integration — configuration reading, the layer-run order of looped spans, state
slots, requests that wait for their next tokens, logit rows through a chunked fill, the model registry."""
import json

import pytest
import torch

from hydrainfer_amd.engine.isa import AwaitTokens, EmptyInstruction, InstructionListBuilder, TextFill
from hydrainfer_amd.engine.rcb import RequestControlBlock, SamplingParameters
from hydrainfer_amd.engine.scheduler import BatchScheduler, BatchSchedulerConfig, BatchSchedulerContext
from hydrainfer_amd.memory.state_slots import StateSlotManager
from hydrainfer_amd.memory.token_cache_manger import BlockTableManager
from hydrainfer_amd.model.tetepel import TetepelShape, tensor_shapes


def _config(**over):
    mixer = {"heads": 2, "dim": 8, "vdim": 4, "kv_rank": 16, "q_rank": 8, "scale": 0.5, "mask": {"size": 7}}
    cfg = {"architecture": "Tetepel", "vocab": 33, "width": 24, "streams": 2, "embedding": {"scale": 3.0},
           "norm": {"eps": 1e-5, "groups": 3},
           "layers": [{"type": "latent_attention", "mixer": dict(mixer), "mlp": {"kind": "dense", "ff": 40}},
                      {"type": "latent_attention", "mixer": dict(mixer, heads=3, kv_rank=40, mask=None), "mlp": None},
                      {"type": "latent_attention", "mixer": dict(mixer, vdim=12), "mlp": {"kind": "dense", "ff": 8}}],
           "loop": {"start": 1, "stop": 3, "times": 3}}
    cfg.update(over)
    return cfg


def test_shape_from_config_and_run_order():
    sh = TetepelShape.from_config(_config())
    assert sh.run_order == [0, 1, 2, 1, 2, 1, 2] and sh.num_hidden_layers == 7
    assert sh.head_dim == 40 and sh.num_key_value_heads == 1 and sh.num_attention_heads == 3
    assert sh.layers[1].mixer.window is None and sh.layers[0].mixer.window == 7 and sh.layers[1].ff is None
    assert TetepelShape.from_config(sh.to_config()).run_order == sh.run_order
    assert TetepelShape.from_config(_config(loop=None)).run_order == [0, 1, 2]
    assert TetepelShape.from_config(_config(loop={"start": 0, "stop": 3, "times": 2})).run_order == [0, 1, 2, 0, 1, 2]
    names = tensor_shapes(sh)
    assert names["l1.mix.uk"] == (3 * 8, 40) and names["l2.mix.uv"] == (2 * 12, 16) and "l1.mlp.gate" not in names
    assert names["l0.hc2.mix"] == (2, 2) and names["l0.rg1.b"] == (24,)
    with pytest.raises(ValueError):
        TetepelShape.from_config(_config(architecture="Other"))
    with pytest.raises(ValueError):
        TetepelShape.from_config(_config(loop={"start": 2, "stop": 1, "times": 2}))
    with pytest.raises(ValueError):
        TetepelShape.from_config(_config(norm={"eps": 1e-5, "groups": 5}))


def test_state_slots_are_handed_out_again():
    sm = StateSlotManager(3, rows=2, width=8, device="cpu")
    a, b, c = sm.allocate(), sm.allocate(), sm.allocate()
    assert sorted((a, b, c)) == [0, 1, 2] and sm.allocate() == -1
    sm.free(b)
    assert sm.get_num_available_slots() == 1 and sm.allocate() == b
    with pytest.raises(ValueError):
        sm.free(7)
    sm.free(a)
    with pytest.raises(ValueError):
        sm.free(a)
    assert sm.state.shape == (3, 2, 8) and sm.state.dtype == torch.float32


def _request(tokens, first=0):
    rcb = RequestControlBlock()
    rcb.sampling_params = SamplingParameters(max_tokens=1 << 30)
    ids = list(range(first, first + len(tokens)))
    b = InstructionListBuilder()
    b.append(TextFill(list(tokens), ids, list(ids), False, None, None))
    b.append(AwaitTokens())
    rcb.instructions = b.build_instruction_list()
    return rcb


def test_scheduler_parks_requests_that_wait_for_tokens_and_owns_their_slots():
    kv = BlockTableManager(n_blocks=6, block_size=16)
    sm = StateSlotManager(2, rows=1, width=4, device="cpu")
    sched = BatchScheduler(BatchSchedulerConfig(max_running_requests=4, token_budgets=1 << 20, chunked_prefill=False),
                           BatchSchedulerContext(kv, None, sm))
    r1, r2, r3 = _request([1] * 20), _request([2] * 3), _request([3] * 5)
    for r in (r1, r2, r3):
        sched.schedule_new(r)
    batch = sched.step()
    assert [r for r, _ in batch] == [r1, r2]                       # two slots: the third request waits for one
    assert {r1.state_slot, r2.state_slot} == {0, 1} and r3.state_slot is None
    assert len(r1.virtual_kv_cache.block_table) == 2
    batch.step()
    for r in (r1, r2):
        assert isinstance(r.current_instruction(), AwaitTokens)
        sched.schedule_running(r)
    assert len(sched.step()) == 0                                   # everyone is parked (r3 still without a slot)
    # r1's client sends one more token, r2's says that nothing more comes
    r1.instructions.extend(TextFill([9], [20], [20], False, None, None))
    r1.instructions.extend(AwaitTokens())
    r2.instructions.tail.prev.closed = True
    batch = sched.step()
    kinds = {id(r): type(i) for r, i in batch}
    assert kinds[id(r1)] is TextFill and kinds[id(r2)] is EmptyInstruction and id(r3) not in kinds
    assert [i.token_ids for r, i in batch if r is r1] == [[9]]


def test_logit_rows_follow_their_tokens_through_a_chunked_fill():
    f = TextFill(list(range(10)), list(range(10)), list(range(10)), False, None, None)
    f.logit_rows = [0, 3, 4, 9]
    b = InstructionListBuilder()
    b.append(f)
    b.build_instruction_list()
    f.chunk_prefill(4)
    assert f.logit_rows == [0, 3] and f.next.logit_rows == [0, 5] and f.next.token_ids == list(range(4, 10))


def test_registry_names_the_architecture(tmp_path):
    from hydrainfer_amd.model.registry import architecture_of, load_model, registered
    (tmp_path / "config.json").write_text(json.dumps(_config()))
    assert architecture_of(str(tmp_path)) == "Tetepel" and "Tetepel" in registered()
    assert "LlavaForConditionalGeneration" in registered()
    (tmp_path / "config.json").write_text(json.dumps({"architectures": ["Nope"]}))
    with pytest.raises(ValueError):
        load_model(str(tmp_path), torch.float32, "cpu")


def test_mix_library_exports_what_its_header_declares():
    """include/hydra_mix.h, the ctypes table and the built library name the same entry points (no GPU needed to open it)."""
    import ctypes
    import os
    import re
    from hydrainfer_amd import _lib
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    declared = set(re.findall(r"^(?:int|int64_t|const char\*)\s+(hxm_\w+)\(", open(os.path.join(root, "include", "hydra_mix.h")).read(), re.M))
    assert declared == set(_lib._MIX_SIGNATURES), declared ^ set(_lib._MIX_SIGNATURES)
    if not os.path.exists(_lib.MIX_LIB_PATH):
        pytest.skip("libhydra_mix.so is not built")
    handle = ctypes.CDLL(_lib.MIX_LIB_PATH)
    for name in declared:
        assert hasattr(handle, name), name
    assert handle.hxm_abi_version() == _lib.HXM_ABI_VERSION
