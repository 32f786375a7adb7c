"""Shared by the Tukevik tests on the GPU and, with the torch double of the kernel set, on the host: small
configurations whose sizes differ from each other in every respect, model folders with random weights made sharp
enough that a fault shows, the expectation from the plain implementation, and the check of a schedule."""

import json
import os

import torch
from safetensors.torch import load_file, save_file

import keranex_cases as K
import schedules
from conftest import random_ids
from plain import tukevik_plain as plain

LEFT = lambda heads, kv, dim, vdim, chunk, scale, softcap: dict(heads=heads, kv_heads=kv, dim=dim, vdim=vdim,
                                                                mask=dict(size=chunk), scale=scale, softcap=softcap)
RIGHT = lambda heads, dim, vdim, decay, dims, base: dict(heads=heads, dim=dim, vdim=vdim, decay=decay, rot=dict(dims=dims, base=base))
PARALLEL = lambda left, right, ls, rs: dict(left=left, right=right, left_scale=ls, right_scale=rs)
RGLRU = lambda width, blocks, conv: dict(width=width, blocks=blocks, conv=conv)
MOE = lambda experts, top, ff, shared: dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, top=top),
                                            **({"shared": dict(ff=shared)} if shared else {}))
DENSE = lambda ff: dict(kind="dense", ff=ff)

# A recurrent layer first and without a feed-forward; grouped heads (three query heads a key head), keys and values of
# different widths on both sides, a rotation over a part of the head, chunks that are no multiple of a page, a
# convolution of one tap, one block, routing without a shared expert and with one expert a token, widths that are no
# multiple of 16.
TUKEVIK_A = dict(
    architecture="Tukevik", vocab=211, width=96, norm=dict(eps=1e-6), residual_mult=0.7,
    layers=[
        dict(type="rglru", mixer=RGLRU(80, 5, 4), mlp=None),
        dict(type="parallel", mlp=MOE(6, 3, 20, 28),
             mixer=PARALLEL(LEFT(6, 2, 24, 16, 13, 0.9, 6.0), RIGHT(3, 16, 24, [0.9, 0.97, 0.995], 8, 100.0), 1.3, 0.6)),
        dict(type="parallel", mlp=DENSE(72),
             mixer=PARALLEL(LEFT(3, 3, 16, 40, 7, 1.1, 4.0), RIGHT(1, 24, 8, [0.98], 24, 10000.0), 0.5, 1.5)),
        dict(type="rglru", mixer=RGLRU(64, 1, 1), mlp=MOE(4, 1, 16, None)),
    ])
# One key head for all, a chunk of exactly two pages and a chunk of a single position (a query sees itself and the sink),
# every expert chosen, a multiplier of one, a rotation over the whole head, a convolution of two taps.
TUKEVIK_B = dict(
    architecture="Tukevik", vocab=130, width=64, norm=dict(eps=1e-5), residual_mult=1.0,
    layers=[
        dict(type="parallel", mlp=MOE(2, 2, 32, 8),
             mixer=PARALLEL(LEFT(4, 1, 32, 32, 16, 0.6, 50.0), RIGHT(1, 32, 16, [0.96875], 32, 1e6), 1.0, 1.0)),
        dict(type="rglru", mixer=RGLRU(128, 4, 2), mlp=DENSE(40)),
        dict(type="parallel", mlp=None,
             mixer=PARALLEL(LEFT(2, 2, 8, 8, 1, 0.8, 3.0), RIGHT(4, 8, 8, [0.5, 0.9, 0.99, 1.0], 4, 50.0), 0.8, 1.1)),
        dict(type="rglru", mixer=RGLRU(48, 3, 3), mlp=MOE(5, 2, 24, 40)),
    ])
# Sizes in multiples of 64 - what a served model has - with a chunk longer than most requests and one of three pages.
TUKEVIK_C = dict(
    architecture="Tukevik", vocab=300, width=128, norm=dict(eps=1e-5), residual_mult=0.6,
    layers=[
        dict(type="parallel", mlp=DENSE(192),
             mixer=PARALLEL(LEFT(8, 2, 64, 64, 48, 0.7, 25.0), RIGHT(2, 64, 64, [0.96875, 0.998], 32, 1e4), 0.9, 1.2)),
        dict(type="rglru", mixer=RGLRU(256, 4, 4), mlp=MOE(8, 2, 64, 64)),
        dict(type="parallel", mlp=MOE(4, 2, 128, None),
             mixer=PARALLEL(LEFT(4, 4, 128, 64, 200, 0.5, 20.0), RIGHT(2, 128, 64, [0.99, 0.999], 128, 1e4), 1.0, 1.0)),
    ])
TUKEVIK = {"A": (TUKEVIK_A, 21, 4), "B": (TUKEVIK_B, 22, 8), "C": (TUKEVIK_C, 23, 16)}        # config, weight seed, page size

LENGTHS, PROMPTS, POOL_TOKENS = K.LENGTHS, K.PROMPTS, K.POOL_TOKENS
# float32: a few hundred float32 operations and recurrences over a hundred tokens.  bfloat16: as served, against the plain
# float32 logits; a router's close call that rounding turns the other way replaces an expert at that one position.
LIMITS = {"float32": dict(max=2e-4, rms=2e-4), "bfloat16": dict(max=0.08, rms=0.1)}
BEYOND = {"float32": 0.0, "bfloat16": 0.1}


def sharpen(folder: str, raw: dict, seed: int = 0) -> None:
    """Random tensors of N(0, 0.02) hide faults: a recurrence whose decay is exp(-8 * 0.5 * softplus(0)) forgets its state
    within a token, a convolution with weights of 0.02 passes almost nothing of the earlier inputs, gates stay at one
    half and routers' logits hardly differ.  `lam` is drawn so that decays lie between 0.6 and 0.999, the convolutions,
    the gates' matrices and the routers are scaled up."""
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    generator = torch.Generator().manual_seed(1000 + seed)
    scaled = lambda name, factor: (tensors[name].float() * factor).to(torch.bfloat16)
    for index, layer in enumerate(raw["layers"]):
        p = f"l{index}.mix."
        if layer["type"] == "rglru":
            width = layer["mixer"]["width"]
            tensors[p + "lam"] = (-6.0 + 4.0 * torch.rand(width, generator=generator)).to(torch.bfloat16)
            for name, factor in (("conv", 25.0), ("ra", 40.0), ("ri", 40.0), ("x", 3.0), ("y", 3.0)):
                tensors[p + name] = scaled(p + name, factor)
        else:
            for name in ("left.g", "right.g", "right.q", "right.k", "right.v"):
                tensors[p + name] = scaled(p + name, 4.0)
            for name in ("left.q.b", "left.k.b", "left.v.b"):
                tensors[p + name] = scaled(p + name, 10.0)
        mlp = layer.get("mlp")
        if mlp is not None and mlp["kind"] == "moe":
            tensors[f"l{index}.mlp.router"] = scaled(f"l{index}.mlp.router", 20.0)
            tensors[f"l{index}.mlp.router.b"] = scaled(f"l{index}.mlp.router.b", 20.0)
            if mlp.get("shared"):
                tensors[f"l{index}.mlp.shared.sg"] = scaled(f"l{index}.mlp.shared.sg", 20.0)
    save_file(tensors, path, metadata={"format": "pt"})


def make_folder(folder: str, raw: dict, seed: int) -> str:
    from ampere_kv_engine_amd.config import TukevikConfig
    from ampere_kv_engine_amd.weights import write_random_model
    write_random_model(folder, TukevikConfig.from_dict(raw), seed)
    sharpen(folder, raw, seed)
    return folder


def plain_logits(folder: str, ids: list[int]) -> torch.Tensor:
    with open(os.path.join(folder, "config.json")) as handle:
        raw = json.load(handle)
    return plain.forward(raw, load_file(os.path.join(folder, "model.safetensors")), ids)


def plain_greedy(folder: str, prompt: list[int], new_tokens: int) -> list[int]:
    ids, out = list(prompt), []
    for _ in range(new_tokens):
        out.append(int(plain_logits(folder, ids)[-1].argmax()))
        ids.append(out[-1])
    return out


def make_case(name: str, folder: str, config=None) -> dict:
    raw, seed, page_size = config if config is not None else TUKEVIK[name]
    make_folder(folder, raw, seed)
    requests = {r: random_ids(raw["vocab"], n, seed=300 + i) for i, (r, n) in enumerate(LENGTHS.items())}
    expected = {r: plain_logits(folder, ids) for r, ids in requests.items()}
    return dict(name=name, folder=folder, page_size=page_size, requests=requests, expected=expected, raw=raw)


make_engine = K.make_engine


def errors(got, want, dtype):
    saved = K.LIMITS, K.BEYOND
    K.LIMITS, K.BEYOND = LIMITS, BEYOND
    try:
        return K.errors(got, want, dtype)
    finally:
        K.LIMITS, K.BEYOND = saved


def assert_close(got, want, dtype: str, what: str = ""):
    position, by_max, by_rms = errors(got, want, dtype)
    if position is not None:
        raise AssertionError(f"{what}: first wrong position {position} of {want.reshape(-1, want.shape[-1]).shape[0]}; "
                             f"worst max error {by_max:.2f} x its limit, worst rms error {by_rms:.2f} x its limit ({dtype})")
    return max(by_max, by_rms)


def check(engine, case, schedule):
    got, pages = schedules.run(engine, case["requests"], schedule)
    dtype = engine.config.dtype
    worst = 0.0
    for name, want in case["expected"].items():
        worst = max(worst, assert_close(got[name], want, dtype, f"{case['name']}/{dtype} request {name}"))
    assert engine.cache.num_free_pages == [engine.config.num_pages] * len(engine.cache.groups), "pages were lost"
    assert engine.cache.slots.num_free == engine.config.max_seqs, "slots were lost"
    print(f"[tukevik {case['name']} {dtype}] worst error {worst:.2f} of its limit")
    return pages


# ---- the cuttings ------------------------------------------------------------------------------------------------

def case_whole(engine, case):
    check(engine, case, schedules.whole(case["requests"]))


def case_prefill_then_token_by_token(engine, case):
    check(engine, case, schedules.last_one_by_one(case["requests"], 32))


def case_token_by_token_from_the_first(engine, case):
    requests = {k: case["requests"][k][:40] for k in ("a", "b")}
    sub = dict(case, requests=requests, expected={k: case["expected"][k][:40] for k in requests})
    check(engine, sub, schedules.last_one_by_one(requests, 40))


def case_portions_down_to_two_tokens(engine, case):
    check(engine, case, schedules.portions(case["requests"]))
    check(engine, case, schedules.portions(case["requests"], sizes=(2, 2, 3, 1, 2, 17, 2, 1, 1, 6)))


def case_mixed_with_pages_and_slots_used_again(engine, case):
    schedule = schedules.mixed(case["requests"], PROMPTS, case["page_size"], engine.config.num_pages, seed=5, max_live=3)
    assert any(any(c == 1 for _, c in entries) and any(c > 1 for _, c in entries) for entries, _ in schedule)
    pages = check(engine, case, schedule)
    names = list(pages)
    if engine.cache.groups:          # (a model of recurrent layers alone keeps no pages)
        assert any(pages[a] & pages[b] for i, a in enumerate(names) for b in names[i + 1:]), "no page was used again"
    for seed in (21, 22):
        check(engine, case, schedules.mixed(case["requests"], PROMPTS, case["page_size"], engine.config.num_pages, seed=seed))


def case_first_tokens(engine, case):
    requests = {"x": case["requests"]["a"][:1], "y": case["requests"]["c"][:3], "z": case["requests"]["d"][:2]}
    sub = dict(case, requests=requests, expected={k: case["expected"][n][:len(v)] for (k, v), n in zip(requests.items(), "acd")})
    check(engine, sub, schedules.whole(requests))
    check(engine, sub, schedules.last_one_by_one(requests, 32))
    check(engine, sub, [([("x", 1), ("y", 2), ("z", 1)], ["x"]), ([("y", 1), ("z", 1)], ["y", "z"])])


def case_long_decoding(engine, case, tokens: int = 230):
    """Every chunk's edge passes under decoded tokens many times, the pages of chunks that were left are given back and
    taken again while the request lives, and the states carry two hundred steps."""
    ids = random_ids(case["raw"]["vocab"], tokens, seed=77)
    sub = dict(case, requests={"long": ids}, expected={"long": plain_logits(case["folder"], ids)})
    check(engine, sub, schedules.last_one_by_one({"long": ids}, tokens - 10))


def case_greedy_generation(engine, case):
    """Through the framework's own entry points: single-request generation, and the scheduler with several requests."""
    from ampere_kv_engine_amd.engine.generate import generate_tokens
    from ampere_kv_engine_amd.engine.scheduler import Scheduler
    prompts = {name: case["requests"][name][:length] for name, length in (("a", 21), ("b", 9), ("c", 2))}
    want = {name: plain_greedy(case["folder"], ids, 10) for name, ids in prompts.items()}
    for name, ids in prompts.items():
        assert generate_tokens(engine, ids, max_new_tokens=10, ignore_eos=True, prefill_chunk_size=8) == want[name], name
    scheduler = Scheduler(engine, prefill_chunk_size=7)
    submitted = {name: scheduler.submit(name, ids, 10, ignore_eos=True) for name, ids in prompts.items()}
    scheduler.run_until_idle()
    for name, request in submitted.items():
        assert request.output_ids == want[name], f"scheduler, request {name}"
    assert engine.cache.slots.num_free == engine.config.max_seqs


CUTTINGS = [case_whole, case_prefill_then_token_by_token, case_token_by_token_from_the_first,
            case_portions_down_to_two_tokens, case_mixed_with_pages_and_slots_used_again, case_first_tokens,
            case_long_decoding, case_greedy_generation]


# ---- one mechanism alone: a model of one layer in which nothing else contributes --------------------------------------

def alone(mechanism: str) -> tuple:
    """(config, weight seed, page size) of a one-layer model in which one mechanism alone shapes the logits."""
    left, right = LEFT(4, 2, 16, 24, 11, 0.9, 5.0), RIGHT(2, 16, 12, [0.9, 0.99], 8, 1000.0)
    layers = {
        "chunked attention": dict(type="parallel", mixer=PARALLEL(left, right, 1.0, 0.0), mlp=None),
        "retention": dict(type="parallel", mixer=PARALLEL(left, right, 0.0, 1.0), mlp=None),
        "recurrent unit": dict(type="rglru", mixer=RGLRU(72, 3, 3), mlp=None),
        "dense feed-forward": dict(type="rglru", mixer=RGLRU(8, 1, 1), mlp=DENSE(56)),
        "routed feed-forward": dict(type="rglru", mixer=RGLRU(8, 1, 1), mlp=MOE(7, 3, 12, 20)),
    }
    raw = dict(architecture="Tukevik", vocab=150, width=48, norm=dict(eps=1e-6), residual_mult=1.0, layers=[layers[mechanism]])
    return raw, 31 + sorted(layers).index(mechanism), 4


MECHANISMS = ("chunked attention", "retention", "recurrent unit", "dense feed-forward", "routed feed-forward")
