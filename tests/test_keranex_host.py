"""Keranex on the host: its configuration, and the engine's side of it - registry, loading, cache groups and slot
state, batching, the scheduler - with the torch double standing in for the HIP kernels, against the plain
implementation.  The HIP kernels meet the same cases in `test_keranex_gpu.py`."""

import copy
import json
import os

import pytest
import torch

import keranex_cases as K
from ampere_kv_engine_amd.config import ConfigError, KeranexConfig, load_config
from ampere_kv_engine_amd.config.specs import RunEntry
from ampere_kv_engine_amd.engine.model import expected_tensors
from plain import keranex_plain as plain
from torch_kernels import TorchKernels


@pytest.fixture(scope="module", params=list(K.KERANEX))
def case(request, tmp_path_factory):
    return K.make_case(request.param, str(tmp_path_factory.mktemp(f"keranex_{request.param}")))


@pytest.fixture(scope="module")
def engine(case):
    return K.make_engine(case, "float32", "cpu", kernels=TorchKernels())


@pytest.mark.parametrize("cutting", K.CUTTINGS, ids=lambda f: f.__name__)
def test_cutting(engine, case, cutting):
    cutting(engine, case)


def test_the_configuration_names_every_part_and_tensor(tmp_path):
    raw = copy.deepcopy(K.KERANEX_A)
    folder = str(tmp_path)
    with open(os.path.join(folder, "config.json"), "w") as handle:
        json.dump(raw, handle)
    config = load_config(folder)                     # found through the key "architecture"
    assert isinstance(config, KeranexConfig) and config.to_dict() == raw
    spec = config.to_model_spec()
    assert [layer.mixer.kind for layer in spec.layers] == ["selective_scan", "latent_attention", "latent_attention", "selective_scan"]
    assert [layer.feed_forward.kind for layer in spec.layers] == ["none", "routed_experts", "routed_experts", "routed_experts"]
    # the third layer reads the second's records and writes none; the owner keeps them for the wider of the two windows
    assert spec.run_order == (RunEntry(0, 0), RunEntry(1, 1), RunEntry(2, 1, writes_cache=False), RunEntry(3, 3))
    assert spec.layers[1].mixer["window"] == 5 and spec.layers[1].mixer["cache_window"] == 9
    assert spec.layers[2].mixer["window"] == 9 and not spec.layers[2].mixer["own_latent"]
    names = {t.name: tuple(t.shape) for t in expected_tensors(spec)}
    assert names["bigram"] == (38, 96) and names["embed"] == (211, 96) and names["head"] == (211, 96)
    assert "l0.norm2" not in names and "l0.mlp.router" not in names and names["l0.norm1b"] == (96,)
    assert names["l1.mix.dkv"] == (48, 96) and names["l1.mix.uq"] == (3 * 24, 24) and names["l1.mix.uv"] == (72, 40)
    assert "l2.mix.dkv" not in names and "l2.mix.dkv.norm" not in names and names["l2.mix.uk"] == (40, 40)
    assert names["l3.mix.x"] == (8 + 32, 64) and names["l3.mix.conv"] == (64, 4) and names["l3.mix.A_log"] == (64, 16)
    assert names["l3.mlp.e3.down"] == (96, 16) and names["l2.mlp.router"] == (4, 96)
    # without the pair table the embedding is the plain one
    del raw["embedding"]
    assert KeranexConfig.from_dict(raw).to_model_spec().embedding.kind == "embedding"


@pytest.mark.parametrize("change,message", [
    (lambda raw: raw["layers"][1].update(type="attention"), "type"),
    (lambda raw: raw["layers"][2]["mixer"].update(kv_from=3), "keeps no latent"),
    (lambda raw: raw["layers"][2]["mixer"].update(kv_rank=48), "kv_rank differs"),
    (lambda raw: raw["layers"][1]["mixer"]["rot"].update(dims=7), "rot.dims"),
    (lambda raw: raw["layers"][1]["mlp"]["router"].update(experts=7), "experts"),
    (lambda raw: raw["layers"][3]["mlp"]["router"].update(top=3), "experts"),
    (lambda raw: raw["layers"][0]["mixer"].pop("state"), "state"),
    (lambda raw: raw.pop("width"), "width"),
])
def test_configurations_the_design_does_not_allow_are_refused(change, message):
    raw = copy.deepcopy(K.KERANEX_A)
    change(raw)
    with pytest.raises(ConfigError, match=message):
        KeranexConfig.from_dict(raw)


def test_cache_groups_slot_state_and_the_word_of_the_token_fed_last(case, engine):
    from ampere_kv_engine_amd.cache.slots import WORD_FED_TOKEN
    from ampere_kv_engine_amd.engine import StepEntry
    layers = case["raw"]["layers"]
    for index, layer in enumerate(layers):
        view = engine.cache.layer_cache.get(index)
        if layer["type"] == "mamba1":
            m = layer["mixer"]
            assert view.state.shape == (4, m["inner"] * m["state"] + (m["conv"] - 1) * m["inner"])
        elif layer["mixer"].get("kv_from") is None:
            assert view.v is None and view.k.shape[1:] == (1, case["page_size"], layer["mixer"]["kv_rank"] + layer["mixer"]["rot_dim"])
        else:
            assert view is None          # a reader has no cache of its own
    seq = engine.open("w")
    ids = case["requests"]["a"][:11]
    engine.step([StepEntry(seq, ids[:6], [])])
    assert int(engine.cache.arrays.words[seq.slot, WORD_FED_TOKEN]) == ids[5]
    # a windowed group gives pages back while the request lives
    engine.step([StepEntry(seq, case["requests"]["d"], [])])
    engine.step([StepEntry(seq, ids[6:7], [])])        # (what a window has passed is given back when tokens register)
    for table, group in zip(seq.tables, engine.cache.groups):
        assert table.num_held <= (group.need.window + case["page_size"] - 1) // case["page_size"] + 1
    slot = seq.slot
    engine.close(seq)
    seq = engine.open("again")           # the slot comes round again: nothing of its predecessor is left
    assert seq.slot == slot and int(engine.cache.arrays.words[slot, WORD_FED_TOKEN]) == -1
    for index, layer in enumerate(layers):
        if layer["type"] == "mamba1":
            assert not engine.cache.layer_cache[index].state[slot].any()
    engine.close(seq)


# ---- the plain implementation's own mechanisms, where a sentence of the design can be checked by hand -----------------

def test_plain_pair_rows_window_and_routing():
    assert plain.bigram_rows([4, 9, 9], buckets=7, mul_prev=3, mul_cur=5) == [7, (12 + 45) % 7, (27 + 45) % 7]
    # groups of two: scores .05 .30 | .25 .20 | .11 .09 -> the groups' bests .30, .25, .11; two groups kept, top 3
    logits = torch.log(torch.tensor([[0.05, 0.30, 0.25, 0.20, 0.11, 0.09]]))
    chosen, weights = plain.route(torch.eye(1), logits.T.contiguous(), experts=6, top=3, groups=3, keep=2)
    assert chosen.tolist() == [[1, 2, 3]]
    torch.testing.assert_close(weights, torch.tensor([[0.30, 0.25, 0.20]]))
    chosen, _ = plain.route(torch.eye(1), logits.T.contiguous(), experts=6, top=2, groups=3, keep=1)
    assert chosen.tolist() == [[1, 0]]       # only the best group's experts, although others score higher than 0.05
    x = torch.arange(8.0).view(1, 1, 8)
    turned = plain.rotate_first_dims(x, torch.tensor([3]), dims=4, base=100.0)
    assert torch.equal(turned[..., 4:], x[..., 4:])
    a0, a1 = 3.0, 3.0 * 100.0 ** -0.5
    torch.testing.assert_close(turned[0, 0, :4], torch.tensor([
        0 * torch.cos(torch.tensor(a0)) - 2 * torch.sin(torch.tensor(a0)), 1 * torch.cos(torch.tensor(a1)) - 3 * torch.sin(torch.tensor(a1)),
        2 * torch.cos(torch.tensor(a0)) + 0 * torch.sin(torch.tensor(a0)), 3 * torch.cos(torch.tensor(a1)) + 1 * torch.sin(torch.tensor(a1))]))
