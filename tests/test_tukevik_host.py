"""Tukevik on the host: its configuration, and the engine's side of it - registry, loading, a cache layer with pages and
a state, chunks whose pages are given back, batching, the scheduler - with the torch double standing in for the HIP
kernels, against the plain implementation.  The HIP kernels meet the same cases in `test_tukevik_gpu.py`."""

import copy
import json
import math
import os

import pytest
import torch

import schedules
import tukevik_cases as T
from ampere_kv_engine_amd.cache.pages import BlockTable, PageAllocator
from ampere_kv_engine_amd.config import ConfigError, TukevikConfig, load_config
from ampere_kv_engine_amd.engine.model import expected_tensors
from conftest import random_ids
from plain import tukevik_plain as plain
from torch_kernels import TorchKernels


@pytest.fixture(scope="module", params=["A", "B"])       # (the third configuration, of served sizes, meets the GPU alone)
def case(request, tmp_path_factory):
    return T.make_case(request.param, str(tmp_path_factory.mktemp(f"tukevik_{request.param}")))


@pytest.fixture(scope="module")
def engine(case):
    return T.make_engine(case, "float32", "cpu", kernels=TorchKernels())


@pytest.mark.parametrize("cutting", T.CUTTINGS, ids=lambda f: f.__name__)
def test_cutting(engine, case, cutting):
    if cutting is T.case_long_decoding:
        cutting(engine, case, tokens=90)         # (the double steps through recurrences token by token on the host)
    else:
        cutting(engine, case)


@pytest.mark.parametrize("mechanism", T.MECHANISMS)
def test_one_mechanism_alone(mechanism, tmp_path):
    case = T.make_case(mechanism, str(tmp_path), T.alone(mechanism))
    engine = T.make_engine(case, "float32", "cpu", kernels=TorchKernels())
    T.case_whole(engine, case)
    T.case_portions_down_to_two_tokens(engine, case)
    T.case_mixed_with_pages_and_slots_used_again(engine, case)


def test_the_configuration_names_every_part_and_tensor(tmp_path):
    raw = copy.deepcopy(T.TUKEVIK_A)
    folder = str(tmp_path)
    with open(os.path.join(folder, "config.json"), "w") as handle:
        json.dump(raw, handle)
    config = load_config(folder)                     # found through the key "architecture"
    assert isinstance(config, TukevikConfig) and config.to_dict() == raw
    spec = config.to_model_spec()
    assert [layer.mixer.kind for layer in spec.layers] == ["rglru", "parallel", "parallel", "rglru"]
    assert [layer.feed_forward.kind for layer in spec.layers] == ["none", "routed_experts", "swiglu", "routed_experts"]
    assert all(layer.block.kind == "scaled_prenorm" and layer.block["residual_scale"] == 0.7 for layer in spec.layers)
    (left, left_scale), (right, right_scale) = spec.layers[1].mixer["branches"]
    assert (left.kind, left_scale, right.kind, right_scale) == ("gated_attention", 1.3, "retention", 0.6)
    assert left["chunk"] == 13 and left["softcap"] == 6.0 and left["sink"] and left["head_gate"] and right["rotary_dims"] == 8
    assert spec.head["tied_to"] == "embed"
    names = {t.name: tuple(t.shape) for t in expected_tensors(spec) if not t.optional}
    assert names["embed"] == (211, 96) and "head" not in names and names["final.norm"] == (96,)
    assert "l0.norm2" not in names and names["l0.mix.conv"] == (80, 4) and names["l0.mix.ra"] == (5, 16, 16)
    assert names["l0.mix.ri.b"] == (5, 16) and names["l0.mix.lam"] == (80,) and names["l0.mix.y.b"] == (80,)
    assert names["l1.mix.left.q"] == (144, 96) and names["l1.mix.left.k.b"] == (48,) and names["l1.mix.left.v"] == (32, 96)
    assert names["l1.mix.left.g"] == (6, 96) and "l1.mix.left.g.b" not in names and names["l1.mix.left.o"] == (96, 96)
    assert names["l1.mix.right.k"] == (48, 96) and names["l1.mix.right.g"] == (72, 96) and names["l1.mix.right.o"] == (96, 72)
    assert names["l1.mlp.e5.gate"] == (20, 96) and names["l1.mlp.router.b"] == (6,) and names["l1.mlp.shared.sg"] == (1, 96)
    assert names["l1.mlp.shared.down"] == (96, 28) and names["l2.mlp.down"] == (96, 72)
    assert "l3.mlp.shared.sg" not in names and names["l3.mlp.e3.down"] == (96, 16)


@pytest.mark.parametrize("change,message", [
    (lambda raw: raw["layers"][1].update(type="attention"), "type"),
    (lambda raw: raw["layers"][1]["mixer"]["left"].update(kv_heads=4), "kv_heads"),
    (lambda raw: raw["layers"][1]["mixer"]["right"].update(decay=[0.9]), "decay"),
    (lambda raw: raw["layers"][1]["mixer"]["right"]["rot"].update(dims=7), "rot.dims"),
    (lambda raw: raw["layers"][0]["mixer"].update(blocks=3), "blocks"),
    (lambda raw: raw["layers"][3]["mlp"]["router"].update(top=5), "experts"),
    (lambda raw: raw["layers"][2]["mlp"].update(kind="glu"), "kind"),
    (lambda raw: raw["layers"][1]["mixer"].pop("left_scale"), "left_scale"),
    (lambda raw: raw.pop("residual_mult"), "residual_mult"),
])
def test_configurations_the_design_does_not_allow_are_refused(change, message):
    raw = copy.deepcopy(T.TUKEVIK_A)
    change(raw)
    with pytest.raises(ConfigError, match=message):
        TukevikConfig.from_dict(raw)


def test_a_layer_with_pages_and_a_state_and_chunks_that_give_pages_back(case, engine):
    from ampere_kv_engine_amd.engine import StepEntry
    layers = case["raw"]["layers"]
    page = case["page_size"]
    for index, layer in enumerate(layers):
        view = engine.cache.layer_cache[index]
        m = layer["mixer"]
        if layer["type"] == "rglru":
            assert view.k is None and view.state.shape == (4, m["width"] * m["conv"])
        else:
            left, right = m["left"], m["right"]
            assert view.k.shape[1:] == (left["kv_heads"], page, left["dim"]) and view.v.shape[1:] == (left["kv_heads"], left["vdim"], page)
            assert view.state.shape == (4, right["heads"] * right["dim"] * right["vdim"])
    seq = engine.open("w")
    engine.step([StepEntry(seq, case["requests"]["d"], [])])
    engine.step([StepEntry(seq, case["requests"]["a"][:1], [])])    # (what a chunk has left behind is given back when tokens register)
    for table, group in zip(seq.tables, engine.cache.groups):
        assert table.num_held <= (group.need.chunk + page - 1) // page + 1
    slot = seq.slot
    engine.close(seq)
    seq = engine.open("again")           # the slot comes round again: nothing of its predecessor is left
    assert seq.slot == slot
    for index in range(len(layers)):
        assert not engine.cache.layer_cache[index].state[slot].any()
    engine.close(seq)


def test_block_table_with_chunks():
    pool = PageAllocator(16)
    table = BlockTable(pool, page_size=4, chunk=10)
    table.append_tokens(9)                      # positions 0..8: chunk 0
    assert table.num_held == 3
    table.append_tokens(3)                      # 9..11: position 10 opens chunk 1, whose first page also holds 8 and 9
    assert table.num_held == 3
    table.append_tokens(1)                      # the next position, 12, is of chunk 1 (from 10): pages 0 and 1 are passed
    assert table.num_held == 2 and table.pages[:2] == (-1, -1)
    table.append_tokens(9)                      # positions 13..21; 21 is of chunk 2 - but what is given back is decided
    assert table.num_held == 4                  # when tokens register: the portion's first position, 13, still reads from 10 on
    table.append_tokens(1)                      # the next position, 22, is of chunk 2 (from 20): page 5 holds 20..23
    assert table.num_held == 1 and pool.num_free == 15
    table.release()
    assert pool.num_free == 16


# ---- the plain implementation's own mechanisms, where a sentence of the design can be checked by hand -----------------

def test_plain_mechanisms_by_hand():
    assert plain.chunk_mask(5, 3).int().tolist() == [[1, 0, 0, 0, 0], [1, 1, 0, 0, 0], [1, 1, 1, 0, 0], [0, 0, 0, 1, 0], [0, 0, 0, 1, 1]]
    p = plain.sink_softmax(torch.tensor([[0.0, math.log(2.0), 5.0]]), torch.tensor([[True, True, False]]))
    torch.testing.assert_close(p, torch.tensor([[0.25, 0.5, 0.0]]))
    chosen, weights = plain.route(torch.eye(2), torch.tensor([[1.0, 0.0], [3.0, 0.0], [2.0, 0.0]]), torch.tensor([0.0, 0.0, 1.5]), 2)
    assert chosen[0].tolist() == [2, 1]        # logits 1, 3, 3.5 for the first token
    torch.testing.assert_close(weights[0], torch.softmax(torch.tensor([3.5, 3.0]), 0))
    out = plain.causal_conv(torch.tensor([[1.0], [2.0], [4.0]]), torch.tensor([[100.0, 10.0, 1.0]]), torch.tensor([0.5]))
    assert out[:, 0].tolist() == [1.5, 12.5, 124.5]
    u = torch.ones(3, 2)
    S = plain.rglru_scan(u, torch.full((3, 2), 0.5), torch.ones(3, 2), torch.zeros(2))
    a = math.exp(-8 * 0.5 * math.log(2.0))
    torch.testing.assert_close(S[1], torch.full((2,), a * math.sqrt(1 - a * a) + math.sqrt(1 - a * a)))
    turned = plain.rotate_first_dims(torch.arange(6.0).view(1, 1, 6), torch.tensor([2]), dims=4, base=100.0)
    assert torch.equal(turned[..., 4:], torch.tensor([[[4.0, 5.0]]]))
    torch.testing.assert_close(turned[0, 0, 0], torch.tensor(0 * math.cos(2.0) - 2 * math.sin(2.0)))
    torch.testing.assert_close(turned[0, 0, 3], torch.tensor(3 * math.cos(0.2) + 1 * math.sin(0.2)))


def test_a_far_key_at_the_chunks_edges_decides_the_output():
    """The plain attention with inputs made so that one key stands out: the first position of a chunk is seen by the
    chunk's last query and by no query of the next chunk."""
    n, size = 24, 8
    m = dict(heads=1, kv_heads=1, dim=4, vdim=2, mask=dict(size=size), scale=4.0, softcap=50.0)
    h = torch.zeros(n, 3)
    h[:, 0] = 1.0                      # every token: the same query direction
    h[8, 1] = 1.0                      # position 8, a chunk's first: a key along the queries, a value of its own
    w = {"q": torch.tensor([[1.0, 0, 0], [0, 0, 0], [0, 0, 0], [0, 0, 0]]), "q.b": torch.zeros(4),
         "k": torch.tensor([[0, 1.0, 0], [0.3, 0, 0], [0, 0, 0], [0, 0, 0]]), "k.b": torch.zeros(4),
         "v": torch.tensor([[0, 1.0, 0], [1.0, 0, 0]]), "v.b": torch.zeros(2), "g": torch.full((1, 3), 5.0),
         "o": torch.eye(2)}
    out = plain.chunked_attention(h, w, m, 1e-6)
    assert out[15, 0] > 0.9 and out[9, 0] > 0.9           # seen from the chunk's own last position, and from nearby
    assert out[16, 0].abs() < 1e-6 and out[7, 0].abs() < 1e-6      # not from the next chunk, nor from before
