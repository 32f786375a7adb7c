"""Shared by the Keranex tests on the GPU and, with the torch double of the kernel set, on the host: small
configurations whose sizes differ from each other in every respect, model folders with random weights made sharp
enough that a fault shows, the expectation from the plain implementation, and the check of a schedule."""

import json
import os

import torch
from safetensors.torch import load_file, save_file

import schedules
from conftest import random_ids
from plain import keranex_plain as plain

MOE = lambda experts, top, groups, keep, ff: dict(kind="moe", expert=dict(ff=ff), router=dict(
    experts=experts, top=top, groups=dict(count=groups, keep=keep)))
LATENT = lambda heads, dim, rot, vdim, kv, q, window, scale, base, **more: dict(
    heads=heads, dim=dim, rot_dim=rot, vdim=vdim, kv_rank=kv, q_rank=q, mask=dict(size=window), scale=scale,
    rot=dict(base=base, dims=rot), **more)
SCAN = lambda inner, state, dt_rank, conv: dict(inner=inner, state=state, dt_rank=dt_rank, conv=conv)

# A scan first and without a feed-forward; odd head counts; a reader whose window is wider than its cache's owner's;
# groups of one expert, one group, top 1; latents that are no multiple of 64, 16 or 8 wide; a state that is no power of two.
KERANEX_A = dict(
    architecture="Keranex", vocab=211, width=96, norm=dict(eps=1e-6),
    embedding=dict(bigram=dict(buckets=37, mul_prev=5, mul_cur=3)),
    layers=[
        dict(type="mamba1", mixer=SCAN(80, 5, 3, 3), mlp=None),
        dict(type="latent_attention", mixer=LATENT(3, 16, 8, 24, 40, 24, 5, 0.2, 100.0), mlp=MOE(6, 3, 3, 2, 20)),
        dict(type="latent_attention", mixer=LATENT(5, 8, 8, 16, 40, 16, 9, 0.3, 100.0, kv_from=1), mlp=MOE(4, 1, 1, 1, 24)),
        dict(type="mamba1", mixer=SCAN(64, 16, 8, 4), mlp=MOE(4, 2, 4, 2, 16)),
    ])
# Twelve heads (two blocks of the attention kernel), a window of one page and more, a window of a single token, a
# convolution of two taps, every expert chosen, one bucket.
KERANEX_B = dict(
    architecture="Keranex", vocab=130, width=64, norm=dict(eps=1e-5),
    embedding=dict(bigram=dict(buckets=1, mul_prev=1, mul_cur=1)),
    layers=[
        dict(type="latent_attention", mixer=LATENT(12, 32, 16, 32, 72, 40, 19, 0.15, 10000.0), mlp=MOE(2, 2, 2, 2, 32)),
        dict(type="mamba1", mixer=SCAN(128, 20, 4, 2), mlp=MOE(8, 2, 2, 1, 8)),
        dict(type="latent_attention", mixer=LATENT(2, 16, 4, 8, 24, 8, 1, 0.25, 50.0), mlp=None),
        dict(type="latent_attention", mixer=LATENT(4, 16, 16, 16, 72, 32, 19, 0.25, 10000.0, kv_from=0), mlp=MOE(3, 1, 3, 1, 40)),
    ])
# Heads in multiples of 16 and latents of 128: the sizes at which, in bfloat16, the attention runs on the matrix cores
# and the layer keeps its latents a second time - for the reader of 32 heads too, whose window is the narrower one.
KERANEX_C = dict(
    architecture="Keranex", vocab=300, width=128, norm=dict(eps=1e-5),
    embedding=dict(bigram=dict(buckets=64, mul_prev=7, mul_cur=9)),
    layers=[
        dict(type="latent_attention", mixer=LATENT(16, 32, 32, 32, 128, 64, 36, 0.12, 10000.0), mlp=MOE(4, 2, 2, 1, 32)),
        dict(type="mamba1", mixer=SCAN(128, 8, 8, 4), mlp=None),
        dict(type="latent_attention", mixer=LATENT(32, 16, 32, 16, 128, 48, 24, 0.15, 10000.0, kv_from=0), mlp=MOE(4, 2, 2, 1, 32)),
    ])
KERANEX = {"A": (KERANEX_A, 11, 4), "B": (KERANEX_B, 12, 8), "C": (KERANEX_C, 13, 16)}        # config, weight seed, page size

LENGTHS = {"a": 70, "b": 45, "e": 33, "d": 96, "c": 61, "f": 27}
PROMPTS = {"a": 40, "b": 45, "c": 30, "d": 20, "e": 1, "f": 20}
POOL_TOKENS = 256

# |engine - plain| as a fraction of the largest |logit| ("max") and, per position, of the largest root mean square
# ("rms").  float32: a few hundred float32 operations, amplified by softmaxes made sharp; no position may lie beyond.
# bfloat16: positions lie within 0.04 of the plain float32 logits (median 0.007) - except where the rounding of an
# activation turns a router's close call the other way, which replaces an expert and moves that one position by 0.1 to
# 0.7 (the torch double, which rounds where the kernels round, shows the same: up to 4 of a request's 45 positions): a
# tenth of a request's positions may lie beyond the limit.  What a cutting, a page or a slot could break is held to the float32 limits by the same cases in float32; a
# window that is one token off moves the median position by 0.07 to 0.4.
LIMITS = {"float32": dict(max=1e-4, rms=1e-4), "bfloat16": dict(max=0.06, rms=0.08)}
BEYOND = {"float32": 0.0, "bfloat16": 0.1}       # the share of a request's positions that may lie beyond the limits


def sharpen(folder: str, raw: dict) -> None:
    """Random matrices of N(0, 0.02) give nearly flat softmaxes, in which one key more or less hardly shows.  The
    queries' and keys' up-projections are scaled until scores are a few units apart, and the routers until the
    experts' scores differ."""
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    for index, layer in enumerate(raw["layers"]):
        if layer["type"] == "latent_attention":
            for name in ("uq", "uk"):
                tensors[f"l{index}.mix.{name}"] = (tensors[f"l{index}.mix.{name}"].float() * 8.0).to(torch.bfloat16)
        if layer.get("mlp") is not None:
            tensors[f"l{index}.mlp.router"] = (tensors[f"l{index}.mlp.router"].float() * 20.0).to(torch.bfloat16)
    save_file(tensors, path, metadata={"format": "pt"})


def make_folder(folder: str, raw: dict, seed: int) -> str:
    from ampere_kv_engine_amd.config import KeranexConfig
    from ampere_kv_engine_amd.weights import write_random_model
    write_random_model(folder, KeranexConfig.from_dict(raw), seed)
    sharpen(folder, raw)
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


def make_case(name: str, folder: str) -> dict:
    raw, seed, page_size = KERANEX[name]
    make_folder(folder, raw, seed)
    requests = {r: random_ids(raw["vocab"], n, seed=200 + i) for i, (r, n) in enumerate(LENGTHS.items())}
    expected = {r: plain_logits(folder, ids) for r, ids in requests.items()}
    return dict(name=name, folder=folder, page_size=page_size, requests=requests, expected=expected, raw=raw)


def make_engine(case, dtype, device, kernels=None, num_pages=None, **options):
    from ampere_kv_engine_amd.config import EngineConfig
    from ampere_kv_engine_amd.engine import Engine
    page = case["page_size"]
    config = EngineConfig(dtype=dtype, page_size=page, num_pages=num_pages or POOL_TOKENS // page, max_seqs=4,
                          max_batched_tokens=256, max_seq_len=512, device=device, **options)
    return Engine.from_folder(case["folder"], config, kernels=kernels)


def errors(got: torch.Tensor, want: torch.Tensor, dtype: str):
    got, want = got.reshape(-1, got.shape[-1]).float(), want.reshape(-1, want.shape[-1]).float()
    assert got.shape == want.shape, f"{tuple(got.shape)} logits, {tuple(want.shape)} expected"
    assert not torch.isnan(got).any(), "NaN logits"
    top = max(float(want.abs().max()), 0.25)
    rms = max(float(want.pow(2).mean(dim=1).sqrt().max()), 0.05)
    error = got - want
    by_max = error.abs().max(dim=1).values / (LIMITS[dtype]["max"] * top)
    by_rms = error.pow(2).mean(dim=1).sqrt() / (LIMITS[dtype]["rms"] * rms)
    beyond = ((by_max > 1) | (by_rms > 1)).nonzero()
    allowed = int(BEYOND[dtype] * got.shape[0] + 0.999) if BEYOND[dtype] else 0
    if len(beyond) <= allowed:      # (isolated close calls: the worst is then that of the positions within the limits)
        within = (by_max <= 1) & (by_rms <= 1)
        return None, float(by_max[within].max()) if within.any() else 0.0, float(by_rms[within].max()) if within.any() else 0.0
    return int(beyond[0]), float(by_max.max()), float(by_rms.max())


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
    print(f"[keranex {case['name']} {dtype}] worst error {worst:.2f} of its limit")
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
    assert any(pages[a] & pages[b] for i, a in enumerate(names) for b in names[i + 1:]), "no page was used again"
    for seed in (21, 22):
        check(engine, case, schedules.mixed(case["requests"], PROMPTS, case["page_size"], engine.config.num_pages, seed=seed))


def case_first_tokens(engine, case):
    requests = {"x": case["requests"]["a"][:1], "y": case["requests"]["c"][:3], "z": case["requests"]["d"][:2]}
    sub = dict(case, requests=requests, expected={k: case["expected"][n][:len(v)] for (k, v), n in zip(requests.items(), "acd")})
    check(engine, sub, schedules.whole(requests))
    check(engine, sub, schedules.last_one_by_one(requests, 32))
    check(engine, sub, [([("x", 1), ("y", 2), ("z", 1)], ["x"]), ([("y", 1), ("z", 1)], ["y", "z"])])


def case_long_decoding(engine, case):
    """Every window passes over decoded tokens many times, pages are given back and taken again while the request lives."""
    ids = random_ids(case["raw"]["vocab"], 230, seed=77)
    sub = dict(case, requests={"long": ids}, expected={"long": plain_logits(case["folder"], ids)})
    check(engine, sub, schedules.last_one_by_one({"long": ids}, 220))


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
