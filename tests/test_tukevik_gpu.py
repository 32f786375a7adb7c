"""Tukevik on the GPU: every kernel of its own against the plain implementation's function of the same mechanism, and
the engine with the HIP kernels through the cuttings of `tukevik_cases` - float32 against tight limits, bfloat16 as
it is served."""

import json
import math
import os
import random
import subprocess
import sys
from types import SimpleNamespace

import pytest
import torch

import schedules
import tukevik_cases as T
from conftest import ROOT, random_ids
from plain import tukevik_plain as plain

pytestmark = pytest.mark.gpu
DEVICE = "cuda:0"


@pytest.fixture(scope="module")
def hip():
    from ampere_kv_engine_amd.kernels.hip import HipKernels
    return HipKernels(DEVICE)


@pytest.fixture(scope="module", params=list(T.TUKEVIK))
def case(request, tmp_path_factory):
    return T.make_case(request.param, str(tmp_path_factory.mktemp(f"tukevik_{request.param}")))


@pytest.fixture(scope="module", params=["float32", "bfloat16"])
def engine(request, case):
    return T.make_engine(case, request.param, DEVICE)


@pytest.mark.filterwarnings("ignore:a bfloat16 matrix")
@pytest.mark.parametrize("cutting", T.CUTTINGS, ids=lambda f: f.__name__)
def test_cutting(engine, case, cutting):
    if cutting is T.case_greedy_generation and engine.config.dtype != "float32":
        pytest.skip("greedy tokens are compared with the plain float32 implementation's")
    cutting(engine, case)
    assert engine.kernels.parts_library_path.endswith("libakv_parts.so")


@pytest.mark.filterwarnings("ignore:a bfloat16 matrix")
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mechanism", T.MECHANISMS)
def test_one_mechanism_alone(mechanism, dtype, tmp_path):
    case = T.make_case(mechanism, str(tmp_path), T.alone(mechanism))
    engine = T.make_engine(case, dtype, DEVICE)
    T.case_whole(engine, case)
    T.case_prefill_then_token_by_token(engine, case)
    T.case_portions_down_to_two_tokens(engine, case)
    T.case_mixed_with_pages_and_slots_used_again(engine, case)


def test_steps_are_recorded_and_replayed(case):
    """Decode steps come again and again: the second is recorded, the later ones are replays; all agree with the plain
    implementation, and an engine that records nothing gives the same bits."""
    ids = case["requests"]["d"]
    want = case["expected"]["d"]
    outs = {}
    for graphs in (True, False):
        engine = T.make_engine(case, "float32", DEVICE, decode_graphs=graphs)
        got, _ = schedules.run(engine, {"d": ids}, schedules.last_one_by_one({"d": ids}, 60))
        T.assert_close(got["d"], want, "float32", f"graphs {graphs}")
        outs[graphs] = got["d"]
        if graphs:
            assert any(g is not None for g in engine._graphs.values()), "nothing was recorded"
    assert torch.equal(outs[True], outs[False])


def test_portions_whose_shape_comes_again_are_recorded(tmp_path):
    """Portions of 32 tokens, again and again, beside a request's single tokens - retention over chunks with a state of
    128 x 128 (its kernels ask for more than 64 KB of LDS), the matrix-core attention, the scan cut into runs: the
    recorded steps give the bits of an engine that records nothing, in both arithmetics."""
    raw = dict(architecture="Tukevik", vocab=200, width=64, norm=dict(eps=1e-6), residual_mult=0.9, layers=[
        dict(type="parallel", mlp=T.DENSE(64),
             mixer=T.PARALLEL(T.LEFT(4, 2, 64, 64, 50, 0.8, 10.0), T.RIGHT(1, 128, 128, [0.99], 64, 1e4), 1.0, 1.0)),
        dict(type="rglru", mixer=T.RGLRU(96, 2, 3), mlp=T.MOE(4, 2, 16, 16))])
    case = T.make_case("recorded portions", str(tmp_path), (raw, 41, 16))
    from ampere_kv_engine_amd.engine import StepEntry
    ids, single = case["requests"]["d"], case["requests"]["b"]
    for dtype in ("float32", "bfloat16"):
        outs = {}
        for graphs in (True, False):
            engine = T.make_engine(case, dtype, DEVICE, decode_graphs=graphs)
            d, b = engine.open("d"), engine.open("b")
            rows = []
            for step in range(3):          # a step is recorded when its shape comes again; each asks for two rows
                logits = engine.step([StepEntry(d, ids[32 * step:32 * step + 32], [31]), StepEntry(b, single[step:step + 1], [0])])
                rows.append(logits.float().cpu())
            engine.close(d), engine.close(b)
            got = torch.cat(rows)
            want = torch.stack([row for step in range(3) for row in (case["expected"]["d"][32 * step + 31], case["expected"]["b"][step])])
            T.assert_close(got, want, dtype, f"{dtype}, graphs {graphs}")
            outs[graphs] = got
            if graphs:
                assert any(g is not None for g in engine._graphs.values()), "nothing was recorded"
        assert torch.equal(outs[True], outs[False])


def test_trace_replay_of_a_random_model(case, tmp_path):
    """bin/trace_run on a configuration file and a seed: the mixed cutting, every position against the plain model."""
    from ampere_kv_engine_amd.config import TukevikConfig
    from ampere_kv_engine_amd.weights import write_random_model
    import numpy as np
    config_path = tmp_path / "config.json"
    config_path.write_text(json.dumps(case["raw"]))
    folder = write_random_model(str(tmp_path / "model"), TukevikConfig.from_dict(case["raw"]), 9)
    requests = {name: case["requests"][name] for name in ("a", "b", "e")}
    schedule = schedules.mixed(requests, T.PROMPTS, 16, 64, seed=3)
    out = tmp_path / "out"
    lines = "\n".join(json.dumps(r) for r in schedules.to_trace(requests, schedule)) + "\n"
    done = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--random-config", str(config_path),
                           "--weights-seed", "9", "--dtype", "float32", "--out", str(out), "--max-tokens", "1024"],
                          input=lines, capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr[-2000:]
    assert [l for l in done.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(len(schedule))]
    fed = {name: 0 for name in requests}
    for number, (entries, _) in enumerate(schedule):
        got = torch.from_numpy(np.fromfile(out / f"{number}.f32", dtype="<f4").reshape(-1, case["raw"]["vocab"]).copy())
        row = 0
        for name, count in entries:
            want = T.plain_logits(folder, requests[name][:fed[name] + count])[fed[name]:]
            T.assert_close(got[row:row + count], want, "float32", f"step {number} request {name}")
            fed[name] += count
            row += count


def test_the_command_line_generates_with_a_tukevik_model(case, tmp_path):
    """`python -m ampere_kv_engine_amd.runner` on a configuration file and a seed: one request, and several through the
    scheduler, greedy; the tokens of the plain implementation.  `--mode check` holds the serving arithmetic against
    the engine's 32-bit path."""
    import re
    from ampere_kv_engine_amd.config import TukevikConfig
    from ampere_kv_engine_amd.weights import write_random_model
    config_path = tmp_path / "config.json"
    config_path.write_text(json.dumps(case["raw"]))
    folder = write_random_model(str(tmp_path / "model"), TukevikConfig.from_dict(case["raw"]), 5)
    prompts = [case["requests"]["a"][:19], case["requests"]["b"][:6], case["requests"]["c"][:31]]
    want = [T.plain_greedy(folder, ids, 6) for ids in prompts]
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


def random_configuration(seed: int) -> tuple:
    """Sizes, constants and the order of layers drawn from a seed: any head counts and groupings, keys and values of
    different widths (some no multiple of 8), chunks from one position to longer than a request, any number of blocks
    and taps, layers without a feed-forward, routing with and without a shared expert."""
    rng = random.Random(seed)
    layers = []
    for _ in range(rng.choice((2, 3, 4, 5))):
        mlp = rng.choice((None, "dense", "moe", "moe"))
        if mlp == "dense":
            mlp = T.DENSE(rng.choice((40, 64, 100, 136)))
        elif mlp == "moe":
            experts = rng.choice((1, 2, 3, 5, 8, 17))
            mlp = T.MOE(experts, rng.randint(1, experts), rng.choice((8, 12, 32)), rng.choice((None, 8, 20, 48)))
        if rng.random() < 0.45:
            blocks = rng.choice((1, 2, 3, 4, 8))
            layers.append(dict(type="rglru", mlp=mlp, mixer=T.RGLRU(blocks * rng.choice((4, 8, 20, 32)), blocks, rng.choice((1, 2, 3, 4, 5)))))
            continue
        kv, group = rng.choice((1, 2, 3)), rng.choice((1, 2, 4, 5))
        left = T.LEFT(kv * group, kv, rng.choice((8, 12, 32, 64, 80)), rng.choice((4, 8, 24, 64, 72)),
                      rng.choice((1, 2, 5, 16, 31, 64, 100, 500)), rng.uniform(0.3, 1.2), rng.choice((2.0, 10.0, 30.0)))
        heads, dim = rng.choice((1, 2, 3, 5)), rng.choice((8, 12, 32, 64))
        right = T.RIGHT(heads, dim, rng.choice((4, 8, 24, 40)), [rng.choice((0.5, 0.9, 0.99, 0.999, 1.0)) for _ in range(heads)],
                        rng.choice([d for d in (2, 4, 8, 12, 32, 64) if d <= dim]), rng.choice((100.0, 1e4, 1e6)))
        layers.append(dict(type="parallel", mlp=mlp, mixer=T.PARALLEL(left, right, rng.uniform(0.3, 1.5), rng.uniform(0.3, 1.5))))
    raw = dict(architecture="Tukevik", vocab=rng.choice((97, 260, 1000)), width=rng.choice((40, 72, 96, 136, 192)),
               norm=dict(eps=rng.choice((1e-5, 1e-6))), residual_mult=rng.choice((0.3, 0.5, 1.0, 1.4)), layers=layers)
    return raw, seed, rng.choice((4, 8, 16, 32))


@pytest.mark.filterwarnings("ignore:a bfloat16 matrix")
@pytest.mark.parametrize("seed", range(500, 508))
def test_a_random_configuration_through_the_cuttings(seed, tmp_path):
    config = random_configuration(seed)
    print(f"seed {seed}: {config[0]}, pages of {config[2]}", flush=True)
    case = T.make_case(f"random {seed}", str(tmp_path), config)
    for dtype in ("float32", "bfloat16"):
        engine = T.make_engine(case, dtype, DEVICE)
        T.case_whole(engine, case)
        T.case_portions_down_to_two_tokens(engine, case)
        T.case_prefill_then_token_by_token(engine, case)
        T.case_mixed_with_pages_and_slots_used_again(engine, case)


# ---- the kernels one by one, against the plain functions ----------------------------------------------------------------

def _ctx(lengths_before, counts, device=DEVICE):
    """What the kernels read of a step: requests that hold `lengths_before` tokens and bring `counts` more."""
    q_start, positions, seq_of_token = [0], [], []
    for r, (before, count) in enumerate(zip(lengths_before, counts)):
        q_start.append(q_start[-1] + count)
        positions += list(range(before, before + count))
        seq_of_token += [r] * count
    ints = lambda values: torch.tensor(values, dtype=torch.int32, device=device)
    seqs = len(counts)
    singles = next((r for r, count in enumerate(counts) if count != 1), seqs)        # single tokens come first in a step
    return SimpleNamespace(num_decode_seqs=singles, max_new_tokens=max(counts), num_seqs=seqs, num_tokens=q_start[-1], q_start=ints(q_start), positions=ints(positions),
                           seq_of_token=ints(seq_of_token), seq_slots=ints(list(range(seqs))), host_q_start=q_start,
                           host_seq_slots=list(range(seqs)), host_seq_lens=[b + c for b, c in zip(lengths_before, counts)],
                           max_seq_len=max(b + c for b, c in zip(lengths_before, counts)))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv_heads,dim,vdim,chunk,page", [(4, 2, 16, 24, 11, 4), (3, 1, 40, 8, 64, 16), (8, 8, 64, 64, 7, 8),
                                                               (2, 1, 128, 256, 300, 16), (8, 2, 64, 32, 20, 16),
                                                               (4, 4, 32, 128, 48, 32), (1, 1, 64, 64, 5000, 16),
                                                               (2, 1, 256, 32, 40, 16)])
def test_attention_kernel_alone(hip, dtype, heads, kv_heads, dim, vdim, chunk, page):
    """Two requests in two portions each, through the unit norm with its cache write and the attention, against the plain
    attention of the whole sequences.  Scores are made sharp, and one key a request - the first of a chunk - is made to
    stand out for every later query: it counts up to its chunk's last position and not beyond."""
    torch.manual_seed(heads * 100 + dim)
    lengths, eps, scale, softcap = (75, 2 * chunk + 3 if chunk < 100 else 330 if chunk < 1000 else 2100), 1e-6, 1.2, 9.0
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, mask=dict(size=chunk), scale=scale, softcap=softcap)
    width = heads * dim + kv_heads * (dim + vdim) + heads
    rows = [torch.randn(n, width) for n in lengths]
    for projected, n in zip(rows, lengths):
        needle = min(chunk, n - 2) if chunk < n else 0
        projected[needle, heads * dim:heads * dim + kv_heads * dim] = projected[needle + 1:, :dim].mean(0).repeat(kv_heads) * 30
    rows = [r.to(dtype).float() for r in rows]
    pages_needed = sum((n + page - 1) // page for n in lengths)
    k_pages = torch.zeros(pages_needed + 2, kv_heads, page, dim, dtype=dtype, device=DEVICE)
    v_pages = torch.zeros(pages_needed + 2, kv_heads, vdim, page, dtype=dtype, device=DEVICE)
    order = torch.randperm(pages_needed + 2).tolist()
    table = torch.full((2, max((n + page - 1) // page for n in lengths)), -1, dtype=torch.int32)
    for r, n in enumerate(lengths):
        for i in range((n + page - 1) // page):
            table[r, i] = order.pop()
    got = [torch.zeros(n, heads * vdim) for n in lengths]
    # two portions each, then the last token of each alone (sixteen waves share a row whose request is long)
    for step, befores in enumerate([(0, 0), (41, 5), (lengths[0] - 1, lengths[1] - 1)]):
        counts = [[41, 5], [lengths[0] - 42, lengths[1] - 6], [1, 1]][step]
        ctx = _ctx(befores, counts)
        projected = torch.cat([rows[r][b:b + c] for r, (b, c) in enumerate(zip(befores, counts))]).to(dtype).to(DEVICE)
        slot_map = torch.tensor([int(table[r, p // page]) * page + p % page for r, (b, c) in enumerate(zip(befores, counts))
                                 for p in range(b, b + c)], dtype=torch.int32, device=DEVICE)
        meta = SimpleNamespace(block_table=table.to(DEVICE), rows=None, width=table.shape[1], slot_map=slot_map)
        q = torch.empty(ctx.num_tokens, heads * dim, dtype=dtype, device=DEVICE)
        out = torch.empty(ctx.num_tokens, heads * vdim, dtype=dtype, device=DEVICE)
        hip.unit_norm_write(projected, heads, kv_heads, dim, vdim, eps, slot_map, k_pages, v_pages, q)
        hip.gated_attention(q, k_pages, v_pages, projected, heads * dim + kv_heads * (dim + vdim), ctx, meta, heads, kv_heads,
                            dim, vdim, scale, softcap, chunk, None, True, out)
        at = 0
        for r, (b, c) in enumerate(zip(befores, counts)):
            got[r][b:b + c] = out[at:at + c].float().cpu()
            at += c
    for r, n in enumerate(lengths):
        x = rows[r]
        qk = heads * dim + kv_heads * dim
        identity = lambda size: torch.eye(size)
        # the plain function with identity projections: its input IS the projected row, cut by selecting matrices
        pick = lambda lo, hi: torch.eye(width)[lo:hi]
        w = {"q": pick(0, heads * dim), "q.b": torch.zeros(heads * dim), "k": pick(heads * dim, qk), "k.b": torch.zeros(kv_heads * dim),
             "v": pick(qk, qk + kv_heads * vdim), "v.b": torch.zeros(kv_heads * vdim), "g": pick(qk + kv_heads * vdim, width),
             "o": identity(heads * vdim)}
        want = plain.chunked_attention(x, w, m, eps)
        limit = 2e-5 if dtype == torch.float32 else 0.03
        error = (got[r] - want).abs().max() / want.abs().max()
        assert error < limit, f"request {r}: {error:.2e}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,dim,vdim,rot", [(2, 16, 12, 8), (1, 64, 32, 64), (3, 24, 40, 0), (2, 128, 128, 32), (1, 256, 256, 2)])
def test_retention_kernel_alone(hip, dtype, heads, dim, vdim, rot):
    torch.manual_seed(dim + vdim)
    lengths, eps, base = (70, 9), 1e-6, 1000.0
    m = dict(heads=heads, dim=dim, vdim=vdim, decay=[0.9, 0.99, 1.0][:heads], rot=dict(dims=rot or 2, base=base))
    width = 2 * heads * (dim + vdim)
    rows = [torch.randn(n, width).to(dtype).float() for n in lengths]
    table = None
    if rot:
        freq = torch.tensor([base ** (-2.0 * i / rot) for i in range(rot // 2)], dtype=torch.float32, device=DEVICE)
        table = torch.empty(128, rot // 2, 2, dtype=torch.float32, device=DEVICE)
        hip.rope_table(freq, table)
    state = torch.zeros(3, heads * dim * vdim, dtype=torch.float32, device=DEVICE)
    decay = torch.tensor(m["decay"], dtype=torch.float32, device=DEVICE)
    got = [torch.zeros(n, heads * vdim) for n in lengths]
    for befores, counts in (((0, 0), (33, 2)), ((33, 2), (1, 1)), ((34, 3), (36, 6))):
        ctx = _ctx(befores, counts)
        projected = torch.cat([rows[r][b:b + c] for r, (b, c) in enumerate(zip(befores, counts))]).to(dtype).to(DEVICE)
        out = torch.empty(ctx.num_tokens, heads * vdim, dtype=dtype, device=DEVICE)
        hip.retention(projected, heads, dim, vdim, rot, table, dim ** -0.5, decay, eps, state, ctx, out)
        at = 0
        for r, (b, c) in enumerate(zip(befores, counts)):
            got[r][b:b + c] = out[at:at + c].float().cpu()
            at += c
    assert not state[2].any()
    qk, vs = heads * dim, heads * vdim
    pick = lambda lo, hi: torch.eye(width)[lo:hi]
    w = {"q": pick(0, qk), "k": pick(qk, 2 * qk), "v": pick(2 * qk, 2 * qk + vs), "g": pick(2 * qk + vs, width), "o": torch.eye(vs)}
    for r, n in enumerate(lengths):
        want = plain.retention(rows[r], w, m, eps) if rot else _retention_without_rotation(rows[r], w, m, eps)
        error = (got[r] - want).abs().max() / want.abs().max()
        assert error < (3e-5 if dtype == torch.float32 else 0.03), f"request {r}: {error:.2e}"


def _retention_without_rotation(x, w, m, eps):
    heads, dim, vdim = m["heads"], m["dim"], m["vdim"]
    n = x.shape[0]
    q, k = (x @ w["q"].T).view(n, heads, dim), (x @ w["k"].T).view(n, heads, dim) * dim ** -0.5
    v = (x @ w["v"].T).view(n, heads, vdim)
    S = torch.zeros(heads, dim, vdim)
    out = torch.zeros(n, heads, vdim)
    for t in range(n):
        S = torch.tensor(m["decay"])[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", S, q[t])
    return plain.unit_rms(out, eps).reshape(n, -1) * plain.silu(x @ w["g"].T)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width,blocks,taps", [(80, 5, 4), (64, 1, 1), (300, 3, 2)])
def test_recurrent_unit_kernels_alone(hip, dtype, width, blocks, taps):
    """Convolution without an activation, the gates' block-diagonal product and the scan, three steps of two requests."""
    torch.manual_seed(width)
    lengths = (50, 12)
    bw = width // blocks
    xy = [torch.randn(n, 2 * width).to(dtype).float() for n in lengths]
    conv, conv_b = (torch.randn(width, taps) * 0.5).to(dtype), (torch.randn(width) * 0.1).to(dtype)
    ra, ri = (torch.randn(blocks, bw, bw) * 0.3).to(dtype), (torch.randn(blocks, bw, bw) * 0.3).to(dtype)
    ra_b, ri_b = (torch.randn(blocks, bw) * 0.3).to(dtype), (torch.randn(blocks, bw) * 0.3).to(dtype)
    lam = (-5.0 + 4.0 * torch.rand(width)).to(dtype)
    gate_weight = torch.cat((ra.transpose(1, 2), ri.transpose(1, 2)), dim=2).contiguous().to(DEVICE)
    gate_bias = torch.cat((ra_b, ri_b), dim=1).float().contiguous().to(DEVICE)
    rate = (-8.0 * torch.nn.functional.softplus(lam.float())).to(DEVICE)
    state = torch.zeros(2, width * taps, dtype=torch.float32, device=DEVICE)
    got = [torch.zeros(n, width) for n in lengths]
    for befores, counts in (((0, 0), (20, 2)), ((20, 2), (1, 1)), ((21, 3), (29, 9))):
        ctx = _ctx(befores, counts)
        both = torch.cat([xy[r][b:b + c] for r, (b, c) in enumerate(zip(befores, counts))]).to(dtype).to(DEVICE)
        tokens = both.shape[0]
        u = torch.empty(tokens, width, dtype=dtype, device=DEVICE)
        hip.conv_silu(both, width, conv.to(DEVICE), conv_b.to(DEVICE), state, 1, ctx, u, activation="none")
        gates = torch.empty(tokens, blocks, 2 * bw, dtype=torch.float32, device=DEVICE)
        hip.heads_linear(u.view(tokens, blocks, bw), bw, gate_weight, gates, 2 * bw)
        out = torch.empty(tokens, width, dtype=dtype, device=DEVICE)
        hip.gated_linear_scan(u, gates, gate_bias, rate, both, blocks, state, taps, ctx, out)
        at = 0
        for r, (b, c) in enumerate(zip(befores, counts)):
            got[r][b:b + c] = out[at:at + c].float().cpu()
            at += c
    for r, n in enumerate(lengths):
        x, y = xy[r][:, :width], xy[r][:, width:]
        u = plain.causal_conv(x, conv.float(), conv_b.float())
        S = plain.rglru_scan(u, plain.block_gate(u, ra.float(), ra_b.float()), plain.block_gate(u, ri.float(), ri_b.float()), lam.float())
        want = S * plain.gelu_tanh(y)
        error = (got[r] - want).abs().max() / want.abs().max()
        assert error < (2e-5 if dtype == torch.float32 else 0.04), f"request {r}: {error:.2e}"


@pytest.mark.parametrize("experts,top,ff,shared", [(6, 3, 20, 28), (4, 1, 16, 0), (2, 2, 8, 8), (70, 5, 4, 12), (1, 1, 8, 0),
                                                   (5, 2, 24, 40)])
def test_routing_and_the_experts_activation(hip, experts, top, ff, shared):
    torch.manual_seed(experts)
    tokens = 37
    scored = experts + (1 if shared else 0)
    logits = torch.randn(tokens, scored) * 3
    logits[0, :min(experts, 2)] = 1.25                 # equal logits: the lower index wins
    gates = torch.empty(tokens, scored, device=DEVICE)
    hip.route_chosen(logits.to(DEVICE), gates, experts, top)
    want = torch.zeros(tokens, scored)
    for t in range(tokens):
        order = sorted(range(experts), key=lambda e: (-float(logits[t, e]), e))[:top]
        weights = torch.softmax(logits[t, order], 0)
        want[t, order] = weights
    chosen, weights = plain.route(logits[1:, :experts], torch.eye(experts), torch.zeros(experts), top)      # (rows without equal logits)
    torch.testing.assert_close(torch.zeros(tokens - 1, experts).scatter_(1, chosen, weights), want[1:, :experts])
    if shared:
        want[:, experts] = torch.sigmoid(logits[:, experts])
    torch.testing.assert_close(gates.cpu(), want, rtol=1e-5, atol=1e-6)
    columns = experts * ff + shared
    for dtype in (torch.float32, torch.bfloat16):
        gate_up = torch.randn(tokens, 2 * columns).to(dtype)
        act = torch.empty(tokens, columns, dtype=dtype, device=DEVICE)
        hip.gate_silu_mul(gate_up.to(DEVICE), gates, act, experts, ff)
        g, u = gate_up[:, :columns].float(), gate_up[:, columns:].float()
        weight = torch.cat([want[:, :experts].repeat_interleave(ff, dim=1)] + ([want[:, experts:].expand(-1, shared)] if shared else []), dim=1)
        torch.testing.assert_close(act.float().cpu(), (weight * plain.silu(g) * u).to(dtype).float(), rtol=2e-2 if dtype == torch.bfloat16 else 1e-5, atol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_scaled_residual_norm_and_scaled_sum(hip, dtype):
    torch.manual_seed(3)
    for hidden in (96, 100, 4096):
        stream = torch.randn(9, hidden, device=DEVICE)
        delta = torch.randn(9, hidden, device=DEVICE).to(dtype)
        weight = 1 + 0.1 * torch.randn(hidden, device=DEVICE)
        want_stream = stream + 0.7 * delta.float()
        want = plain.rms_norm(want_stream, weight, 1e-6)
        out = torch.empty(9, hidden, dtype=dtype, device=DEVICE)
        hip.norm_add_norm(stream, delta, None, 0.0, weight, 1e-6, out, delta_scale=0.7)
        torch.testing.assert_close(stream, want_stream, rtol=1e-6, atol=1e-6)
        torch.testing.assert_close(out.float(), want.to(dtype).float(), rtol=1e-2 if dtype == torch.bfloat16 else 1e-5, atol=1e-5)
        a, b = torch.randn(9, hidden, device=DEVICE).to(dtype), torch.randn(9, hidden, device=DEVICE).to(dtype)
        total = torch.empty_like(a)
        hip.scaled_sum(a, 0.8, b, 1.1, total)
        torch.testing.assert_close(total.float(), (a.float() * 0.8 + b.float() * 1.1).to(dtype).float(), rtol=1e-2 if dtype == torch.bfloat16 else 1e-6, atol=1e-6)
