"""Keranex on the GPU: every kernel of its own against the plain implementation's function of the same mechanism, and
the engine with the HIP kernels through the cuttings of `keranex_cases` - float32 against tight limits, bfloat16 as
it is served."""

import json
import os
import subprocess
import sys
from types import SimpleNamespace

import pytest
import torch

import keranex_cases as K
import schedules
from conftest import ROOT, random_ids
from plain import keranex_plain as plain

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def hip():
    from ampere_kv_engine_amd.kernels.hip import HipKernels
    return HipKernels("cuda:0")


@pytest.fixture(scope="module", params=list(K.KERANEX))
def case(request, tmp_path_factory):
    return K.make_case(request.param, str(tmp_path_factory.mktemp(f"keranex_{request.param}")))


@pytest.fixture(scope="module", params=["float32", "bfloat16"])
def engine(request, case):
    return K.make_engine(case, request.param, "cuda:0")


@pytest.mark.parametrize("cutting", K.CUTTINGS, ids=lambda f: f.__name__)
def test_cutting(engine, case, cutting):
    if cutting is K.case_greedy_generation and engine.config.dtype != "float32":
        pytest.skip("greedy tokens are compared with the plain float32 implementation's")
    cutting(engine, case)
    assert engine.kernels.parts_library_path.endswith("libakv_parts.so")


def test_steps_are_recorded_and_replayed(case):
    """Decode steps come again and again: the second is recorded, the later ones are replays; all agree with the plain
    implementation, and an engine that records nothing gives the same bits."""
    ids = case["requests"]["d"]
    want = case["expected"]["d"]
    outs = {}
    for graphs in (True, False):
        engine = K.make_engine(case, "float32", "cuda:0", decode_graphs=graphs)
        got, _ = schedules.run(engine, {"d": ids}, schedules.last_one_by_one({"d": ids}, 60))
        K.assert_close(got["d"], want, "float32", f"graphs {graphs}")
        outs[graphs] = got["d"]
        if graphs:
            assert any(g is not None for g in engine._graphs.values()), "nothing was recorded"
    assert torch.equal(outs[True], outs[False])


def test_trace_replay_of_a_random_model(case, tmp_path):
    """bin/trace_run on a configuration file and a seed: the mixed cutting, every position against the plain model."""
    from ampere_kv_engine_amd.config import KeranexConfig
    from ampere_kv_engine_amd.weights import write_random_model
    config_path = tmp_path / "config.json"
    config_path.write_text(json.dumps(case["raw"]))
    folder = write_random_model(str(tmp_path / "model"), KeranexConfig.from_dict(case["raw"]), 9)
    requests = {name: case["requests"][name] for name in ("a", "b", "e")}
    schedule = schedules.mixed(requests, K.PROMPTS, 16, 64, seed=3)
    out = tmp_path / "out"
    lines = "\n".join(json.dumps(r) for r in schedules.to_trace(requests, schedule)) + "\n"
    done = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--random-config", str(config_path),
                           "--weights-seed", "9", "--dtype", "float32", "--out", str(out), "--max-tokens", "1024"],
                          input=lines, capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr[-2000:]
    assert [l for l in done.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(len(schedule))]
    fed = {name: 0 for name in requests}
    import numpy as np
    for number, (entries, _) in enumerate(schedule):
        got = torch.from_numpy(np.fromfile(out / f"{number}.f32", dtype="<f4").reshape(-1, case["raw"]["vocab"]).copy())
        row = 0
        for name, count in entries:
            want = K.plain_logits(folder, requests[name][:fed[name] + count])[fed[name]:]
            K.assert_close(got[row:row + count], want, "float32", f"step {number} request {name}")
            fed[name] += count
            row += count


def random_configuration(seed: int) -> dict:
    """Sizes, constants and the order of layers drawn from a seed: widths that are multiples of 8 only, odd head counts,
    windows of any size, several readers of one layer's records, a second owner, layers without feed-forward."""
    import random
    rng = random.Random(seed)
    width = rng.choice((72, 96, 136, 192))
    layers, owners = [], []
    for index in range(rng.choice((3, 4, 5, 6))):
        mlp = None
        if rng.random() < 0.8:
            groups = rng.choice((1, 2, 3))
            size = rng.choice((1, 2, 4))
            keep = rng.randint(1, groups)
            mlp = K.MOE(groups * size, rng.randint(1, keep * size), groups, keep, rng.choice((8, 24, 40)))
        if index > 0 and rng.random() < 0.35:
            layers.append(dict(type="mamba1", mlp=mlp, mixer=K.SCAN(rng.choice((48, 104, 160)), rng.choice((3, 8, 12, 33)),
                                                                    rng.choice((2, 5, 8, 16)), rng.choice((2, 3, 4, 5)))))
            continue
        heads, dim, vdim = rng.choice((1, 2, 6, 7, 16)), rng.choice((8, 24, 32)), rng.choice((8, 24, 40))
        q_rank, window = rng.choice((16, 24, 56)), rng.choice((2, 3, 17, 31, 64, 100))
        if owners and rng.random() < 0.5:
            source = rng.choice(owners)
            kv, rot, base = (layers[source]["mixer"][k] for k in ("kv_rank", "rot_dim", "rot"))
            mixer = K.LATENT(heads, dim, rot, vdim, kv, q_rank, window, rng.uniform(0.1, 0.3), base["base"], kv_from=source)
        else:
            kv, rot = rng.choice(((128, 32), (48, 16), (88, 8), (40, 24)))
            mixer = K.LATENT(heads, dim, rot, vdim, kv, q_rank, window, rng.uniform(0.1, 0.3), rng.choice((100.0, 10000.0, 5e5)))
            owners.append(index)
        layers.append(dict(type="latent_attention", mixer=mixer, mlp=mlp))
    return dict(architecture="Keranex", vocab=rng.choice((97, 260, 1000)), width=width, norm=dict(eps=rng.choice((1e-5, 1e-6))),
                embedding=dict(bigram=dict(buckets=rng.choice((2, 61, 509)), mul_prev=rng.choice((1, 31, 1009)),
                                           mul_cur=rng.choice((1, 7, 131)))), layers=layers)


@pytest.mark.parametrize("seed", [1, 2, 3, 4, 5, 6])
def test_configurations_drawn_at_random(seed, tmp_path):
    raw = random_configuration(seed)
    folder = K.make_folder(str(tmp_path / "model"), raw, seed)
    requests = {"p": random_ids(raw["vocab"], 150, seed=seed), "q": random_ids(raw["vocab"], 41, seed=seed + 50)}
    case = dict(name=f"random{seed}", folder=folder, page_size=16, requests=requests, raw=raw,
                expected={name: K.plain_logits(folder, ids) for name, ids in requests.items()})
    for dtype in ("float32", "bfloat16"):
        engine = K.make_engine(case, dtype, "cuda:0", num_pages=24)
        K.check(engine, case, schedules.whole(requests))
        K.check(engine, case, schedules.portions(requests, sizes=(9, 2, 30, 1, 1, 17, 2, 64)))
        K.check(engine, case, schedules.mixed(requests, {"p": 100, "q": 20}, 16, 24, seed=seed))


def test_the_command_line_generates_with_a_keranex_model(case, tmp_path):
    """`python -m ampere_kv_engine_amd.runner` on a configuration file and a seed: one request, and several through the
    scheduler, greedy; the tokens of the plain implementation.  `--mode check` holds the serving arithmetic against
    the engine's 32-bit path."""
    import re
    from ampere_kv_engine_amd.config import KeranexConfig
    from ampere_kv_engine_amd.weights import write_random_model
    config_path = tmp_path / "config.json"
    config_path.write_text(json.dumps(case["raw"]))
    folder = write_random_model(str(tmp_path / "model"), KeranexConfig.from_dict(case["raw"]), 5)
    prompts = [case["requests"]["a"][:19], case["requests"]["b"][:6], case["requests"]["c"][:31]]
    want = [K.plain_greedy(folder, ids, 6) for ids in prompts]
    base = [sys.executable, "-m", "ampere_kv_engine_amd.runner", "--random-config", str(config_path), "--weights-seed", "5",
            "--max-new-tokens", "6", "--ignore-eos"]
    run = lambda more: subprocess.run(base + more, capture_output=True, text=True, timeout=600, cwd=ROOT)
    one = run(["--mode", "generate", "--dtype", "float32", "--prompt-ids", " ".join(map(str, prompts[0])), "--prefill-chunk", "8"])
    assert one.returncode == 0, one.stderr[-2000:]
    assert json.loads(re.search(r"generated_token_ids = (\[.*\])", one.stdout).group(1)) == want[0]
    prompts_file = tmp_path / "prompts.txt"
    prompts_file.write_text("\n".join(" ".join(map(str, ids)) for ids in prompts) + "\n")
    many = run(["--mode", "generate", "--dtype", "float32", "--prompts-file", str(prompts_file), "--max-seqs", "2",
                "--prefill-chunk", "5"])
    assert many.returncode == 0, many.stderr[-2000:]
    got = [json.loads(line)["generated_token_ids"] for line in many.stdout.splitlines() if line.startswith("{")]
    assert got == want, many.stdout
    check = run(["--mode", "check", "--prompt-len", "40"])
    assert check.returncode == 0, check.stdout[-1500:] + check.stderr[-1500:]


# ---- the kernels, one mechanism at a time ----------------------------------------------------------------------------

def rand(*shape, seed=0, scale=1.0, dtype=torch.float32):
    return (torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale).to(dtype)


def tol(dtype):
    return dict(rtol=2e-5, atol=2e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)


def step_of(portions, slots=None, device="cuda"):
    """A step's arrays for `portions` = [(history, new tokens)] per request."""
    q_start = [0]
    for _, n in portions:
        q_start.append(q_start[-1] + n)
    slots = list(range(len(portions))) if slots is None else slots
    t = lambda values: torch.tensor(values, dtype=torch.int32, device=device)
    return SimpleNamespace(
        num_seqs=len(portions), num_tokens=q_start[-1], host_q_start=q_start, host_seq_slots=slots,
        host_seq_lens=[h + n for h, n in portions], max_seq_len=max(h + n for h, n in portions),
        q_start=t(q_start), seq_slots=t(slots),
        positions=torch.cat([torch.arange(h, h + n) for h, n in portions]).int().to(device),
        seq_of_token=torch.cat([torch.full((n,), r) for r, (_, n) in enumerate(portions)]).int().to(device))


@pytest.mark.parametrize("dtype", DTYPES)
def test_pair_embedding_across_steps(hip, dtype):
    from ampere_kv_engine_amd.cache.slots import SLOT_WORDS, WORD_FED_TOKEN, WORD_LAST_TOKEN
    vocab, hidden, buckets = 50, 24, 7
    table, pairs = rand(vocab, hidden, seed=1, dtype=dtype), rand(buckets + 1, hidden, seed=2, dtype=dtype)
    a, b = random_ids(vocab, 9, 3), random_ids(vocab, 6, 4)
    want_a = plain.embed(a, table.float(), pairs.float(), dict(buckets=buckets, mul_prev=11, mul_cur=13))
    want_b = plain.embed(b, table.float(), pairs.float(), dict(buckets=buckets, mul_prev=11, mul_cur=13))
    words = torch.full((4, SLOT_WORDS), -1, dtype=torch.int32, device="cuda")
    got_a, got_b = [], []
    # a in portions of 4, 1, 4 (slot 2); b in 1, 5 (slot 0), its second portion beside a's single token
    for pa, pb in (((0, 4), None), ((4, 1), (0, 1)), ((5, 4), (1, 5))):
        portions, ids, slots = [], [], []
        for (portion, tokens, slot) in ((pa, a, 2), (pb, b, 0)):
            if portion is not None:
                portions.append(portion)
                ids += tokens[portion[0]:portion[0] + portion[1]]
                slots.append(slot)
        ctx = step_of(portions, slots)
        ctx.slot_words = words
        out = torch.empty(len(ids), hidden, device="cuda")
        hip.embed_pairs(torch.tensor(ids, dtype=torch.int32, device="cuda"), table.cuda(), pairs.cuda(), buckets, 11, 13, out, ctx)
        got_a.append(out[:pa[1]].cpu())
        if pb is not None:
            got_b.append(out[pa[1]:].cpu())
    torch.testing.assert_close(torch.cat(got_a), want_a, rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(torch.cat(got_b), want_b, rtol=1e-6, atol=1e-6)
    assert int(words[2, WORD_FED_TOKEN]) == a[-1] and int(words[0, WORD_FED_TOKEN]) == b[-1]
    # a single token that the sampler left in the slot (-1 as the id) pairs with the token fed before it
    words[2, WORD_LAST_TOKEN] = 17
    ctx = step_of([(9, 1)], [2])
    ctx.slot_words = words
    out = torch.empty(1, hidden, device="cuda")
    hip.embed_pairs(torch.tensor([-1], dtype=torch.int32, device="cuda"), table.cuda(), pairs.cuda(), buckets, 11, 13, out, ctx)
    want = plain.embed(a + [17], table.float(), pairs.float(), dict(buckets=buckets, mul_prev=11, mul_cur=13))[-1:]
    torch.testing.assert_close(out.cpu(), want, rtol=1e-6, atol=1e-6)
    assert int(words[2, WORD_FED_TOKEN]) == 17


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden", [24, 257, 1024, 4100])
def test_norm_after_add_and_norm_before(hip, dtype, hidden):
    stream, delta = rand(5, hidden, seed=1), rand(5, hidden, seed=2, scale=3.0, dtype=dtype)
    post, pre = 1 + rand(hidden, seed=3, scale=0.1), 1 + rand(hidden, seed=4, scale=0.1)
    new = stream + plain.rms_norm(delta.float(), post, 1e-5)
    want = plain.rms_norm(new, pre, 1e-6)
    s, out = stream.cuda(), torch.empty(5, hidden, dtype=dtype, device="cuda")
    hip.norm_add_norm(s, delta.cuda(), post.cuda(), 1e-5, pre.cuda(), 1e-6, out)
    torch.testing.assert_close(s.cpu(), new, rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(out.cpu().float(), want, **tol(dtype))
    s = stream.cuda()                                         # each half alone
    hip.norm_add_norm(s, delta.cuda(), post.cuda(), 1e-5, None, 0.0, None)
    torch.testing.assert_close(s.cpu(), new, rtol=1e-6, atol=1e-6)
    hip.norm_add_norm(s, None, None, 0.0, pre.cuda(), 1e-6, out)
    torch.testing.assert_close(out.cpu().float(), want, **tol(dtype))
    torch.testing.assert_close(s.cpu(), new, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("q_rank,kv_rank,rot,rot_dims,page", [(24, 40, 8, 8, 4), (96, 192, 64, 64, 16), (16, 72, 12, 6, 8)])
def test_latent_encode_and_rotated_queries(hip, dtype, q_rank, kv_rank, rot, rot_dims, page):
    tokens, heads, dim, base = 11, 3, 16, 100.0
    down = rand(tokens, q_rank + kv_rank + rot, seed=1, dtype=dtype)
    wq, wkv = 1 + rand(q_rank, seed=2, scale=0.1), 1 + rand(kv_rank, seed=3, scale=0.1)
    positions = torch.tensor([0, 1, 2, 3, 40, 41, 7, 300, 5, 6, 1000], dtype=torch.int32)
    inv_freq = (1.0 / (base ** (torch.arange(0, rot_dims, 2).float() / rot_dims))).cuda()
    table = torch.empty(1024, rot_dims // 2, 2, device="cuda")
    hip.rope_table(inv_freq, table)
    pages = torch.full((8, 1, page, kv_rank + rot), float("nan"), dtype=dtype, device="cuda")
    slot_map = torch.randperm(8 * page, generator=torch.Generator().manual_seed(5))[:tokens].int()
    cq = torch.empty(tokens, q_rank, dtype=dtype, device="cuda")
    hip.latent_encode(down.cuda(), q_rank, kv_rank, rot, rot_dims, wq.cuda(), wkv.cuda(), 1e-5, table, positions.cuda(),
                      slot_map.cuda(), cq, pages)
    d = down.float()
    torch.testing.assert_close(cq.cpu().float(), plain.rms_norm(d[:, :q_rank], wq, 1e-5), **tol(dtype))
    records = pages.view(-1, kv_rank + rot)[slot_map.long().cuda()].cpu().float()
    torch.testing.assert_close(records[:, :kv_rank], plain.rms_norm(d[:, q_rank:q_rank + kv_rank], wkv, 1e-5), **tol(dtype))
    turned = plain.rotate_first_dims(d[:, None, q_rank + kv_rank:], positions, rot_dims, base)[:, 0]
    torch.testing.assert_close(records[:, kv_rank:], turned, **(tol(dtype) if dtype == torch.bfloat16 else dict(rtol=1e-4, atol=2e-4)))
    assert torch.isnan(pages.view(-1, kv_rank + rot).float()).all(dim=1).sum() == 8 * page - tokens   # no other slot was touched
    # a layer that reads another's records norms its query latent only
    hip.latent_encode(down[:, :q_rank].contiguous().cuda(), q_rank, kv_rank, rot, rot_dims, wq.cuda(), None, 1e-5, None,
                      positions.cuda(), None, cq, None)
    torch.testing.assert_close(cq.cpu().float(), plain.rms_norm(d[:, :q_rank], wq, 1e-5), **tol(dtype))
    q = rand(tokens, heads * (dim + rot), seed=6, dtype=dtype)
    q_abs = torch.zeros(tokens, heads, kv_rank + rot, device="cuda")
    hip.rotate_queries(q.cuda(), heads, dim, rot, rot_dims, table, positions.cuda(), q_abs, kv_rank)
    want = plain.rotate_first_dims(q.float().view(tokens, heads, dim + rot)[..., dim:], positions, rot_dims, base)
    torch.testing.assert_close(q_abs[..., kv_rank:].cpu(), want, rtol=1e-4, atol=2e-4)
    assert not q_abs[..., :kv_rank].any()


@pytest.mark.parametrize("x_dtype,w_dtype,y_dtype", [(torch.float32,) * 3, (torch.bfloat16, torch.bfloat16, torch.float32),
                                                     (torch.float32, torch.bfloat16, torch.bfloat16)])
@pytest.mark.parametrize("tokens,heads,ins,outs", [(1, 3, 16, 40), (9, 5, 40, 24), (33, 2, 128, 300), (8, 12, 64, 72)])
def test_products_per_head(hip, x_dtype, w_dtype, y_dtype, tokens, heads, ins, outs):
    x = rand(tokens, heads, ins + 5, seed=1, dtype=x_dtype)
    w = rand(heads, ins, outs, seed=2, dtype=w_dtype)
    y = torch.full((tokens, heads, outs + 3), 7.0, dtype=y_dtype, device="cuda")
    hip.heads_linear(x.cuda(), ins + 5, w.cuda(), y, outs + 3)
    want = torch.einsum("thi,hio->tho", x[..., :ins].float(), w.float())
    torch.testing.assert_close(y[..., :outs].cpu().float(), want, **tol(y_dtype))
    assert (y[..., outs:] == 7.0).all()
    one = torch.empty(1, heads, outs + 3, dtype=y_dtype, device="cuda")        # a token's sums do not depend on its batch:
    hip.heads_linear(x[tokens - 1:].contiguous().cuda(), ins + 5, w.cuda(), one, outs + 3)
    if x_dtype == w_dtype == y_dtype == torch.float32:                         # in float32 not by a bit
        assert torch.equal(one[..., :outs], y[tokens - 1:, :, :outs])
    else:
        torch.testing.assert_close(one[..., :outs].float(), y[tokens - 1:, :, :outs].float(), **tol(y_dtype))


def records_case(dtype, kv_rank, rot, page, portions, window, seed):
    """Records of every request in pages handed out in a scrambled order; pages that a window has passed are gone
    (-1 in the table) and unwritten slots hold NaN."""
    g = torch.Generator().manual_seed(seed)
    width = kv_rank + rot
    lengths = [h + n for h, n in portions]
    pages_of = [(l + page - 1) // page for l in lengths]
    num_pages = sum(pages_of) + 2
    order = torch.randperm(num_pages, generator=g).tolist()
    pages = torch.full((num_pages, 1, page, width), float("nan"), dtype=dtype)
    table = torch.full((len(portions), max(pages_of) + 1), -1, dtype=torch.int32)
    records, cursor = [], 0
    for r, length in enumerate(lengths):
        rec = torch.randn(length, width, generator=g).to(dtype)
        records.append(rec)
        lowest = 0 if window is None else max(0, portions[r][0] - window + 1)
        for p in range(pages_of[r]):
            at = order[cursor]
            cursor += 1
            if (p + 1) * page <= lowest:
                continue
            table[r, p] = at
            lo, hi = p * page, min((p + 1) * page, length)
            pages[at, 0, :hi - lo] = rec[lo:hi]
    return pages, table, records


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_rank,rot,page", [(3, 40, 8, 4), (8, 192, 64, 16), (12, 72, 16, 8), (2, 300, 64, 16), (1, 520, 64, 32)])
@pytest.mark.parametrize("portions,window", [([(0, 1)], 5), ([(0, 70)], 19), ([(64, 1), (17, 1), (0, 1)], 16),
                                             ([(5, 7), (63, 2), (130, 1), (0, 70)], 40), ([(200, 3), (0, 9)], None)])
def test_latent_attention_over_records(hip, dtype, heads, kv_rank, rot, page, portions, window):
    pages, table, records = records_case(dtype, kv_rank, rot, page, portions, window, 31)
    ctx = step_of(portions)
    meta = SimpleNamespace(block_table=table.cuda(), width=table.shape[1], window=window, rows=None)
    q_abs = rand(ctx.num_tokens, heads, kv_rank + rot, seed=32, scale=0.4)
    out = torch.empty(ctx.num_tokens, heads, kv_rank, device="cuda")
    hip.latent_attend(q_abs.cuda(), pages.cuda(), ctx, meta, heads, kv_rank, 0.3, window, out)
    for r, (history, count) in enumerate(portions):
        first = ctx.host_q_start[r]
        want = plain.attend_records(q_abs[first:first + count], records[r].float(), list(range(history, history + count)),
                                    window, 0.3, kv_rank)
        torch.testing.assert_close(out[first:first + count].cpu(), want, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("heads,kv_rank,rot,page", [(16, 128, 32, 16), (32, 512, 64, 16), (16, 256, 32, 8), (48, 128, 64, 32)])
@pytest.mark.parametrize("portions,window", [([(0, 1)], 5), ([(0, 70)], 19), ([(64, 1), (17, 1), (0, 1)], 16), ([(31, 2)], 32),
                                             ([(5, 7), (63, 2), (130, 1), (0, 70)], 40), ([(200, 3), (0, 9)], None),
                                             ([(500, 40)], 300), ([(1500, 1), (40, 1), (700, 1)], 1024),
                                             ([(2100, 1), (3, 2)], None), ([(300, 128)], 200), ([(0, 256)], 64),
                                             ([(37, 100)], None), ([(1000, 68)], 1)])
def test_latent_attention_on_the_matrix_cores(hip, heads, kv_rank, rot, page, portions, window):
    """bfloat16 queries and records; the latents a second time with the keys contiguous.  Against the plain function on
    the same rounded operands."""
    assert hip.latent_on_matrix_cores(heads, kv_rank, kv_rank + rot, page, torch.bfloat16)
    pages, table, records = records_case(torch.bfloat16, kv_rank, rot, page, portions, window, 51)
    turned = pages[:, :, :, :kv_rank].transpose(2, 3).contiguous()
    ctx = step_of(portions)
    meta = SimpleNamespace(block_table=table.cuda(), width=table.shape[1], window=window, rows=None)
    q_abs = rand(ctx.num_tokens, heads, kv_rank + rot, seed=52, scale=0.4, dtype=torch.bfloat16)
    out = torch.empty(ctx.num_tokens, heads, kv_rank, dtype=torch.bfloat16, device="cuda")
    hip.latent_attend(q_abs.cuda(), pages.cuda(), ctx, meta, heads, kv_rank, 0.2, window, out, latents_t=turned.cuda())
    for r, (history, count) in enumerate(portions):
        first = ctx.host_q_start[r]
        want = plain.attend_records(q_abs[first:first + count].float(), records[r].float(),
                                    list(range(history, history + count)), window, 0.2, kv_rank)
        torch.testing.assert_close(out[first:first + count].cpu().float(), want, rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("window,page", [(16, 16), (17, 16), (40, 16), (5, 4), (64, 8), (1, 4)])
@pytest.mark.parametrize("history", [0, 3, 63, 64, 200])
def test_one_key_stands_out_just_inside_and_just_outside_the_window(hip, window, page, history):
    """Among keys that hardly matter one is made to dominate: the oldest key a query may see must carry the result,
    and the key one older must leave no trace - for a prompt's tokens and for single ones, at page borders too."""
    heads, kv_rank, rot = 2, 24, 8
    for count in (1, 9):
        pages, table, records = records_case(torch.float32, kv_rank, rot, page, [(history, count)], window, 40 + history)
        ctx = step_of([(history, count)])
        meta = SimpleNamespace(block_table=table.cuda(), width=table.shape[1], window=window, rows=None)
        rec = records[0]
        for offset, seen in ((window - 1, True), (window, False)):
            pos = history + count - 1
            at = pos - offset
            if at < 0:
                continue
            q_abs = rand(count, heads, kv_rank + rot, seed=7, scale=0.1)
            q_abs[-1] = rec[at] * 9.0 / float(rec[at].norm())          # the last query points at that one key
            boosted = rec.clone()
            boosted[at] = rec[at] * 6.0
            flat = pages.clone()
            if table[0, at // page] >= 0:
                flat[table[0, at // page], 0, at % page] = boosted[at]
            out = torch.empty(count, heads, kv_rank, device="cuda")
            hip.latent_attend(q_abs.cuda(), flat.cuda(), ctx, meta, heads, kv_rank, 1.0, window, out)
            want = plain.attend_records(q_abs, boosted, list(range(history, history + count)), window, 1.0, kv_rank)
            torch.testing.assert_close(out.cpu(), want, rtol=1e-4, atol=1e-4)
            dominated = torch.allclose(out[-1, 0].cpu(), boosted[at, :kv_rank], rtol=1e-2, atol=1e-2)
            assert dominated == seen, (offset, seen)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("inner,state,taps", [(80, 5, 3), (320, 20, 4), (64, 16, 2), (130, 70, 5), (64, 1, 1)])
def test_convolution_and_scan_carry_their_state(hip, dtype, inner, state, taps):
    """A request in portions - several, two, one token - beside another one, in slots that are not the rows' numbers:
    every portion continues where the slot's state was left."""
    n = 23
    width = inner * state + (taps - 1) * inner
    kept = torch.zeros(4, width, device="cuda")
    kept[1] = 5.0                                             # a slot nobody uses stays as it is
    weights = dict(conv=rand(inner, taps, seed=1, scale=0.5, dtype=dtype), bias=rand(inner, seed=2, scale=0.1, dtype=dtype),
                   a=-torch.exp(rand(inner, state, seed=3, scale=0.3)), d=1 + rand(inner, seed=4, scale=0.1))
    runs = {"p": dict(slot=3, xz=rand(n, 2 * inner, seed=5, dtype=dtype), dt=rand(n, inner, seed=6),
                      bc=rand(n, 2 * state, seed=7), cuts=[0, 7, 9, 10, 11, 18, 23]),
            "q": dict(slot=0, xz=rand(n, 2 * inner, seed=8, dtype=dtype), dt=rand(n, inner, seed=9),
                      bc=rand(n, 2 * state, seed=10), cuts=[0, 1, 2, 12, 14, 15, 23])}
    got = {name: [] for name in runs}
    for turn in range(6):
        portions, slots, pieces = [], [], []
        for name, run in runs.items():
            lo, hi = run["cuts"][turn], run["cuts"][turn + 1]
            portions.append((lo, hi - lo))
            slots.append(run["slot"])
            pieces.append((name, lo, hi))
        ctx = step_of(portions, slots)
        xz = torch.cat([runs[name]["xz"][lo:hi] for name, lo, hi in pieces]).cuda()
        dt = torch.cat([runs[name]["dt"][lo:hi] for name, lo, hi in pieces]).cuda()
        bc = torch.cat([runs[name]["bc"][lo:hi] for name, lo, hi in pieces]).cuda()
        conv = torch.empty(ctx.num_tokens, inner, dtype=dtype, device="cuda")
        hip.conv_silu(xz, inner, weights["conv"].cuda(), weights["bias"].cuda(), kept, state, ctx, conv)
        y = torch.empty(ctx.num_tokens, inner, dtype=dtype, device="cuda")
        hip.selective_scan(conv, dt, bc, xz, weights["a"].cuda(), weights["d"].cuda(), kept, taps, ctx, y)
        row = 0
        for name, lo, hi in pieces:
            got[name].append((conv[row:row + hi - lo].cpu().float(), y[row:row + hi - lo].cpu().float()))
            row += hi - lo
    for name, run in runs.items():
        x, z = run["xz"][:, :inner].float(), run["xz"][:, inner:].float()
        padded = torch.cat((torch.zeros(taps - 1, inner), x))
        conv = torch.stack([(padded[t:t + taps] * weights["conv"].float().T).sum(0) for t in range(n)]) + weights["bias"].float()
        conv = plain.silu(conv)
        torch.testing.assert_close(torch.cat([c for c, _ in got[name]]), conv, **tol(dtype))
        conv = conv.to(dtype).float()                         # the scan reads what the convolution stored
        step = plain.softplus(run["dt"])
        S, ys = torch.zeros(inner, state), []
        for t in range(n):
            S = torch.exp(step[t][:, None] * weights["a"]) * S + (step[t] * conv[t])[:, None] * run["bc"][t, None, :state]
            ys.append((S @ run["bc"][t, state:] + weights["d"] * conv[t]) * plain.silu(z[t]))
        torch.testing.assert_close(torch.cat([y for _, y in got[name]]), torch.stack(ys), **tol(dtype))
        torch.testing.assert_close(kept[run["slot"], :inner * state].cpu().view(inner, state), S, rtol=1e-4, atol=1e-5)
        torch.testing.assert_close(kept[run["slot"], inner * state:].cpu().view(taps - 1, inner), x[n - (taps - 1):])
    assert (kept[1] == 5.0).all() and not kept[2].any()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("experts,top,groups,keep", [(10, 2, 2, 1), (6, 3, 3, 2), (4, 1, 1, 1), (8, 8, 4, 4), (64, 6, 8, 3), (5, 2, 5, 3)])
def test_router_and_gated_activation(hip, dtype, experts, top, groups, keep):
    tokens, hidden, ff = 37, 96, 24
    x = rand(tokens, hidden, seed=1, dtype=dtype)
    router = rand(experts, hidden, seed=2, scale=0.3)
    gates = torch.empty(tokens, experts, device="cuda")
    hip.route((x.float() @ router.T).cuda(), gates, top, groups, keep)
    chosen, weights = plain.route(x.float(), router, experts, top, groups, keep)
    want = torch.zeros(tokens, experts).scatter_(1, chosen, weights)
    torch.testing.assert_close(gates.cpu(), want, rtol=1e-5, atol=1e-6)
    assert ((gates != 0).sum(1) == top).all()
    up = rand(tokens, experts * ff, seed=3, dtype=dtype)
    act = torch.empty_like(up, device="cuda")
    hip.gate_relu_squared(up.cuda(), gates, act)
    want_act = (torch.relu(up.float()).view(tokens, experts, ff) ** 2 * want[:, :, None]).view(tokens, -1)
    torch.testing.assert_close(act.cpu().float(), want_act, **tol(dtype))
    assert not act.view(tokens, experts, ff)[(gates == 0)].any()
