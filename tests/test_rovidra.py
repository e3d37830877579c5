"""The Rovidra decoder in the engine against the plain implementation (``plain_rovidra.py``): every mechanism
alone; whole prompts, prefill against token-by-token decoding, portions down to two tokens, mixed batches with
pages and state slots that are used again; keys just inside and just outside a window, in prompts and in
decoding; the first tokens; long decoding; configurations whose sizes fit no fast path or are equal or 1;
greedy generation through the engine's own entry point and scheduler; the configuration reader's errors.
On the CPU with the plain ops (cache, state, batch and step logic), on the GPU with the HIP kernels."""
import collections
import dataclasses
import json
import os
import subprocess
import sys
import types

import numpy as np
import pytest
import torch

import plain_rovidra as P
import traces
from jax_llm_examples_amd import Engine, SamplingParams, load_model
from jax_llm_examples_amd.cache import CacheManager, CacheView
from jax_llm_examples_amd.config import ConfigError, get_architecture, load_config
from jax_llm_examples_amd.engine import StepEntry, build_context, get_ops
from jax_llm_examples_amd.engine.replay import make_runner
from jax_llm_examples_amd.parts.residual import GatedBranch, Residual
from jax_llm_examples_amd.weights import WeightsError
from rovidra_configs import ROVIDRA, ROVIDRA_FAST, rovidra_config_json, write_rovidra

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEVICES = [pytest.param("cpu", id="cpu-plain-ops"), pytest.param("cuda:0", id="gpu-hip", marks=pytest.mark.gpu)]
LENGTHS = {"RA": [1, 80, 33, 47, 64, 9, 130], "RB": [70, 2, 49, 96, 31, 17], "RS": [61, 40, 5, 83], "RF": [420, 40, 170, 33], "RG": [150, 2, 61, 33, 97]}
MODES = {"whole": traces.whole, "tail": traces.tail, "portions": traces.portions, "mixed": traces.mixed}
TOL = {"float32": 2e-5, "bfloat16": 3e-2}  # of the largest logit of the request
# (bfloat16 with the sharp scores of RS: a rounding of a score of 40 by 2^-9 moves its weight by a tenth)
TOL_OF = {("RS", "bfloat16"): 1e-1}


def _ops(device):
    return get_ops(device, reference_ops=(device == "cpu"))


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("rovidra")
    return {name: write_rovidra(name, str(root / name), torch.float32) for name in ROVIDRA}


@pytest.fixture(scope="module")
def folders_bf16(tmp_path_factory):
    root = tmp_path_factory.mktemp("rovidra_bf16")
    return {name: write_rovidra(name, str(root / name), torch.bfloat16) for name in {**ROVIDRA, **ROVIDRA_FAST}}


# ---------------------------------------------------------------------------------------------- mechanisms alone
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("width", [28, 40, 1024, 1500])
def test_polynomial_activation_alone(device, width):
    g = torch.Generator().manual_seed(width)
    z = torch.randn(7, width, generator=g) * 1.7
    bias, coef = torch.randn(width, generator=g) * 0.3, torch.tensor([0.7, -0.4, 0.2, 0.1])
    want = P.poly_norm((z + bias).double(), coef.double(), 1e-4).float()
    got = _ops(device).polynorm(z.to(device), bias.to(device), coef.to(device), 1e-4).cpu()
    assert torch.allclose(got, want, rtol=2e-5, atol=2e-6), (got - want).abs().max()


def _step_ctx(device, seg_lens, seg_starts, slots, phases):
    """The per-token and per-segment arrays a step's kernels read, made by hand."""
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=device)
    pos, seg, cu = [], [], [0]
    for i, (n, s) in enumerate(zip(seg_lens, seg_starts)):
        pos += list(range(s, s + n))
        seg += [i] * n
        cu.append(cu[-1] + n)
    return types.SimpleNamespace(positions=i32(pos), token_segment=i32(seg), cu_seqlens=i32(cu), state_slots=i32(slots),
                                 state_phase=i32(phases), dtype=torch.float32)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("width", [54, 64, 1024])
def test_gated_sum_norm_and_token_shift_alone(device, width):
    """Two sequences cut into unequal steps that share batches; the shift's state carries each sequence's last row
    from step to step in the half that the step before wrote.  Also: a block of the kernel that takes several rows
    gives what one row per block gives (the GPU's kernel picks by the step's size; here both are forced)."""
    ops = _ops(device)
    g = torch.Generator().manual_seed(width)
    eps, eps_b = 1e-4, 1e-3
    lens = {"a": 23, "b": 9}
    x = {k: torch.randn(n, width, generator=g) for k, n in lens.items()}
    y = {k: torch.randn(n, width, generator=g) for k, n in lens.items()}
    gt = {k: torch.randn(n, width, generator=g) for k, n in lens.items()}
    yb, gb = torch.randn(width, generator=g) * 0.2, torch.randn(width, generator=g)
    wb, w, sw = (torch.rand(width, generator=g) + 0.5 for _ in range(3))
    want = {}
    for k in lens:
        t = (y[k] + yb).double() * torch.sigmoid((gt[k] + gb).double())
        xs = x[k].double() + P.rms_norm(t, wb.double(), eps_b)
        h = P.rms_norm(xs, w.double(), eps)
        want[k] = (xs.float(), h.float(), P.token_shift(h, sw.double()).float())
    dev = lambda t: t.to(device)
    cuts = [[("a", 0, 5)], [("a", 5, 7), ("b", 0, 2)], [("b", 2, 9), ("a", 7, 8)], [("a", 8, 23)]]
    for rows_per_block in ([None] if device == "cpu" else [1, 3]):
        if rows_per_block is not None:
            ops.SHIFT_ROWS_PER_BLOCK = rows_per_block
            ops._compute_units_saved, ops._compute_units = ops._compute_units, 0  # (any step counts as large)
        state = torch.full((3, 2, width), float("nan"), device=device)  # (position 0 must not read it)
        slot, steps_done = {"a": 2, "b": 0}, {"a": 0, "b": 0}
        got = {k: [[], [], []] for k in lens}
        for cut in cuts:
            ctx = _step_ctx(device, [b - a for _, a, b in cut], [a for _, a, _ in cut], [slot[k] for k, _, _ in cut],
                            [steps_done[k] & 1 for k, _, _ in cut])
            cat = lambda src: dev(torch.cat([src[k][a:b] for k, a, b in cut]))
            delta = GatedBranch(cat(y), dev(yb), cat(gt), dev(gb), dev(wb), eps_b)
            xs, h, hs = ops.add_norm_shift(cat(x), delta, dev(w), eps, torch.float32, (dev(sw), state), ctx)
            o = 0
            for k, a, b in cut:
                for j, t in enumerate((xs, h, hs)):
                    got[k][j].append(t[o:o + b - a].cpu())
                o += b - a
                steps_done[k] += 1
        if rows_per_block is not None:
            ops._compute_units = ops._compute_units_saved
        for k in lens:
            for j, what in enumerate(("sum", "normed rows", "shifted rows")):
                a, b = torch.cat(got[k][j]), want[k][j]
                assert torch.allclose(a, b, rtol=2e-5, atol=3e-6), f"{k} {what}: {(a - b).abs().max()}"


@pytest.mark.parametrize("device", DEVICES)
def test_a_step_run_twice_before_its_commit_reads_the_same_state(device):
    """A recorded step is first run launch by launch and then replayed: the second run must find the state that
    the first found, not what the first wrote."""
    ops = _ops(device)
    g = torch.Generator().manual_seed(1)
    d = 48
    state = torch.randn(2, 2, d, generator=g).to(device)
    before = state.clone()
    x, w, sw = torch.randn(1, d, generator=g).to(device), torch.ones(d, device=device), torch.rand(d, generator=g).to(device)
    ctx = _step_ctx(device, [1], [7], [1], [1])
    first = ops.add_norm_shift(x, None, w, 1e-5, torch.float32, (sw, state), ctx)[2].clone()
    again = ops.add_norm_shift(x, None, w, 1e-5, torch.float32, (sw, state), ctx)[2]
    assert torch.equal(first, again)
    assert torch.equal(state[1, 1], before[1, 1]) and torch.equal(state[0], before[0])  # only the other half is written
    assert not torch.equal(state[1, 0], before[1, 0])


def _mixer_alone(folder, device, layer, sizes, x, dtype="float32"):
    """Runs one layer's mixer over the paged cache in the given portions; a reader of another layer's latent gets
    pages that the writer's mixer filled from the same rows."""
    model = load_model(folder, dtype, device)
    cfg = model.config
    ops = _ops(device)
    mixer = model.blocks[layer].mixer
    src = cfg.cache_of(layer)
    writer = model.blocks[src].mixer
    cache = CacheManager({0: mixer.cache_need()}, page_size=16, num_pages=12, max_requests=1, dtype=model.dtype,
                         device=device, poison=True)
    outs, o = [], 0
    for n in sizes:
        if not cache.has_request("r"):
            cache.add_request("r")
        cache.reserve("r", n)
        ctx = build_context(ops, model.dtype, device, cache, [StepEntry("r", [0] * n, [])], cfg.vocab)
        gctx = ctx.groups[0]
        view = CacheView(0, True, block_table=gctx.block_table, slot_mapping=gctx.slot_mapping, attn_meta=gctx, group=0,
                         pages=cache.groups[0].pages[0])
        rows = x[o:o + n].to(device).to(model.dtype)
        if src != layer:
            writer.forward(rows, ctx, view)
            view = dataclasses.replace(view, writes=False)
        outs.append(mixer.forward(rows, ctx, view).float().cpu())
        cache.commit("r")
        o += n
    return torch.cat(outs)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name,layer", [("RA", 0), ("RA", 1), ("RA", 2), ("RA", 3), ("RA", 5), ("RB", 0), ("RB", 1),
                                        ("RB", 2), ("RS", 0)])
def test_latent_attention_alone(folders, device, name, layer):
    """The mixer over the paged latent, whole and in portions, equals the plain mixer, which forms every head's keys
    and values (the engine never does).  Readers of another layer's latent, a layer without a window, rotations
    over part of the rotated elements, a window of one token."""
    plain = P.PlainRovidra(folders[name])
    cfg, w = plain.cfg, plain.w
    m = cfg["layers"][layer]["mixer"]
    src = m.get("kv_from", layer)
    T = 75
    x = torch.randn(T, cfg["width"], generator=torch.Generator().manual_seed(layer + 1))
    pos = list(range(T))
    ms = cfg["layers"][src]["mixer"]
    latent, rope_key = P.latent_of(x.double(), w[f"l{src}.mix.dkv"], w[f"l{src}.mix.dkv.norm"], cfg["norm"]["eps"],
                                   ms["kv_rank"], pos, ms["rot"]["base"], ms["rot"]["dims"])
    p = f"l{layer}.mix."
    want = P.latent_attention(x.double(), latent, rope_key, m, w[p + "q"], w[p + "uk"], w[p + "uv"], w[p + "o"], pos).float()
    for sizes in ([T], [30, 2, 17, 1, 1, 24]):
        got = _mixer_alone(folders[name], device, layer, sizes, x)
        assert torch.allclose(got, want, rtol=2e-4, atol=2e-5), (got - want).abs().max()


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("decoding", [False, True])
def test_one_key_that_stands_out_at_the_windows_edge(folders, device, decoding):
    """One earlier token's shared key part is made to match every later query (its row is scaled up), so whoever
    sees it puts all weight on it.  Queries for which it is the oldest visible key must find it; for the next
    query it must be gone.  The same far back among all other keys, in a prompt and in decoding."""
    name, layer = "RS", 0
    plain = P.PlainRovidra(folders[name])
    cfg, w = plain.cfg, plain.w
    m = cfg["layers"][layer]["mixer"]
    W = m["mask"]["size"]
    T, special = 70, 11
    x = torch.randn(T, cfg["width"], generator=torch.Generator().manual_seed(9))
    x[special] *= 25.0  # its latent is normed, its rotated key part is not: that part dominates the scores
    pos = list(range(T))
    latent, rope_key = P.latent_of(x.double(), w["l0.mix.dkv"], w["l0.mix.dkv.norm"], cfg["norm"]["eps"],
                                   m["kv_rank"], pos, m["rot"]["base"], m["rot"]["dims"])
    want = P.latent_attention(x.double(), latent, rope_key, m, w["l0.mix.q"], w["l0.mix.uk"], w["l0.mix.uv"],
                              w["l0.mix.o"], pos).float()
    sizes = [special + 3] + [1] * (T - special - 3) if decoding else [T]
    got = _mixer_alone(folders[name], device, layer, sizes, x)
    last_in, first_out = special + W - 1, special + W
    assert torch.allclose(got, want, rtol=2e-4, atol=2e-5), (got - want).abs().max()
    # the test has teeth: the row that still sees the key differs much from what it would be without it
    x2 = x.clone()
    x2[special] /= 25.0
    l2, r2 = P.latent_of(x2.double(), w["l0.mix.dkv"], w["l0.mix.dkv.norm"], cfg["norm"]["eps"], m["kv_rank"], pos,
                         m["rot"]["base"], m["rot"]["dims"])
    other = P.latent_attention(x2.double(), l2, r2, m, w["l0.mix.q"], w["l0.mix.uk"], w["l0.mix.uv"], w["l0.mix.o"],
                               pos).float()
    assert (other[last_in] - want[last_in]).abs().max() > 1e-2
    assert torch.allclose(other[first_out], want[first_out], atol=1e-6)


# ---------------------------------------------------------------------------------------------- whole models
def _check(name, folder, dtype, device, mode, record=True, page_size=16, lengths=None):
    lengths = lengths or (LENGTHS[name] + (LENGTHS[name][::-1] if mode == "mixed" else []))
    reqs = traces.random_requests(rovidra_config_json(name)["vocab"], lengths, seed=5)
    steps = MODES[mode](reqs)
    runner = make_runner(folder, dtype, traces.max_live_tokens(steps), device, reference_ops=(device == "cpu"),
                         poison=True, max_requests=4, page_size=page_size, decode_graphs=None if not record else False)
    handed = [collections.Counter() for _ in runner.cache.groups]
    for g, seen in zip(runner.cache.groups, handed):  # which pages every pool hands out, how often
        def alloc(n, inner=g.pool.alloc, seen=seen):
            pages = inner(n)
            seen.update(pages)
            return pages
        g.pool.alloc = alloc
    got = traces.run_trace(runner, steps)
    if not record:
        assert runner.graphs is not None and runner.graphs.replays > 0
    if mode == "mixed":  # pages and slots were used again (a pool hands out the page that came back last)
        assert all(max(seen.values()) > 1 for seen in handed)
        assert len(reqs) > runner.cache.max_requests
    runner.cache.check()
    assert runner.cache.num_live() == 0 and all(g.pool.num_held == 0 for g in runner.cache.groups)
    plain = P.PlainRovidra(folder)
    for rid, toks in reqs.items():
        ref = plain.logits(toks).float()
        assert got[rid].shape == ref.shape and torch.isfinite(got[rid]).all(), f"{rid}: non-finite logits"
        err = (got[rid] - ref).abs().max(dim=-1).values / ref.abs().max()
        bad = (err > TOL_OF.get((name, dtype), TOL[dtype])).nonzero().squeeze(-1).tolist()
        assert not bad, f"{name} {dtype} {mode} {rid}: first wrong position {bad[0]} of {len(toks)}, error {err[bad[0]]:.3g}"


@pytest.mark.parametrize("mode", list(MODES))
@pytest.mark.parametrize("name", list(ROVIDRA))
def test_cpu_plain_ops_float32(folders, name, mode):
    _check(name, folders[name], "float32", "cpu", mode)


@pytest.mark.parametrize("page_size", [4, 64])
def test_cpu_other_page_sizes(folders, page_size):
    _check("RA", folders["RA"], "float32", "cpu", "mixed", page_size=page_size)


@pytest.mark.gpu
@pytest.mark.parametrize("mode", list(MODES))
@pytest.mark.parametrize("name", list(ROVIDRA))
def test_gpu_float32(folders, name, mode):
    _check(name, folders[name], "float32", "cuda:0", mode)


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["tail", "mixed"])
@pytest.mark.parametrize("name", list(ROVIDRA))
def test_gpu_float32_with_recorded_decode_steps(folders, name, mode):
    _check(name, folders[name], "float32", "cuda:0", mode, record=False)


@pytest.mark.gpu
@pytest.mark.parametrize("mode", list(MODES))
@pytest.mark.parametrize("name", list(ROVIDRA) + list(ROVIDRA_FAST))
def test_gpu_bfloat16(folders_bf16, name, mode):
    _check(name, folders_bf16[name], "bfloat16", "cuda:0", mode, record=(mode != "tail"))


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["whole", "portions", "mixed"])
@pytest.mark.parametrize("name", ["RA", "RF", "RG"])
def test_gpu_bfloat16_with_keys_shared_through_shared_memory(folders_bf16, monkeypatch, name, mode):
    """Steps of many tokens go through the attention kernel whose blocks share their keys; here every step of more
    than a few rows does (tiles of several tokens, blocks that end inside a segment, windows that start inside a
    step of 32 keys)."""
    from jax_llm_examples_amd.ops.hip import HipOps

    monkeypatch.setattr(HipOps, "LATENT_LDS_TILES", 2)
    _check(name, folders_bf16[name], "bfloat16", "cuda:0", mode)


@pytest.mark.gpu
def test_gpu_float32_at_vector_sizes(tmp_path):
    folder = write_rovidra("RF", str(tmp_path / "RF"), torch.float32)
    for mode in ("portions", "mixed"):
        _check("RF", folder, "float32", "cuda:0", mode)


@pytest.mark.parametrize("device", DEVICES)
def test_residual_stream_behind_every_layer(folders, device):
    """What a watcher of the step sees behind every run of a layer equals the plain model's stream."""
    folder = folders["RA"]
    toks = traces.random_requests(300, [29], seed=2)["r0"]
    want = []
    P.PlainRovidra(folder).logits(toks, residuals=want)
    runner = make_runner(folder, "float32", 64, device, reference_ops=(device == "cpu"), max_requests=2)
    seen = []
    runner.step([StepEntry("r", toks, [])], tap=lambda part, name, value: seen.append(value()) if name == "residual" else None)
    assert len(seen) == len(want)
    for a, b in zip(seen, want):
        assert torch.allclose(a.cpu(), b.float(), rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_a_token_beyond_every_window_and_shift_changes_nothing(folders, device):
    """One layer with a window of W: the logits at position i depend on tokens i - W .. i (the shift brings in the
    token before the oldest visible key) and on nothing earlier, in a prompt and in decoding."""
    folder = folders["RS"]
    W = rovidra_config_json("RS")["layers"][0]["mixer"]["mask"]["size"]
    toks = traces.random_requests(128, [60], seed=4)["r0"]
    i = 50
    outside, inside = list(toks), list(toks)
    outside[i - W - 1] = (toks[i - W - 1] + 1) % 128
    inside[i - W] = (toks[i - W] + 1) % 128

    def logits_at(seq, decoding):
        runner = make_runner(folder, "float32", 128, device, reference_ops=(device == "cpu"), max_requests=2)
        if not decoding:
            return runner.step([StepEntry("r", seq[: i + 1], [i])])[0].cpu().clone()
        runner.step([StepEntry("r", seq[:20], [])])
        for t in range(20, i):
            runner.step([StepEntry("r", [seq[t]], [])])
        return runner.step([StepEntry("r", [seq[i]], [0])])[0].cpu().clone()

    for decoding in (False, True):
        base = logits_at(toks, decoding)
        assert torch.allclose(logits_at(outside, decoding), base, atol=1e-5)
        assert (logits_at(inside, decoding) - base).abs().max() > 1e-3


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", ["RA", "RB"])
def test_first_tokens_and_long_decoding(folders, device, name):
    """A sequence fed one token at a time from its very first token, far past every window and over many pages."""
    folder = folders[name]
    V = rovidra_config_json(name)["vocab"]
    toks = traces.random_requests(V, [150], seed=6)["r0"]
    runner = make_runner(folder, "float32", 192, device, reference_ops=(device == "cpu"), poison=True, max_requests=2)
    rows = [runner.step([StepEntry("r", [t], [0])])[0].cpu().clone() for t in toks]
    ref = P.PlainRovidra(folder).logits(toks).float()
    err = (torch.stack(rows) - ref).abs().max(dim=-1).values / ref.abs().max()
    assert float(err.max()) < TOL["float32"], f"first wrong position {int((err > TOL['float32']).nonzero()[0])}"


def _greedy(plain, prompt, n):
    seq = list(prompt)
    for _ in range(n):
        seq.append(int(plain.logits(seq)[-1].argmax()))
    return seq[len(prompt):]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", ["RA", "RB"])
def test_greedy_generation_through_the_engine(folders, device, name):
    """``Engine.generate``: the scheduler admits, cuts prompts into portions under a small token budget, decodes four
    requests together, and frees; six requests on four slots."""
    plain = P.PlainRovidra(folders[name])
    V = plain.cfg["vocab"]
    g = torch.Generator().manual_seed(3)
    prompts = [torch.randint(0, V, (n,), generator=g).tolist() for n in (5, 61, 1, 33, 17, 2)]
    eng = Engine(load_model(folders[name], "float32", device), reference_ops=(device == "cpu"), poison=True,
                 cache_tokens=320, decode_batch_size=4, max_num_batched_tokens=48)
    outs = eng.generate(prompts, SamplingParams(max_decode_length=12))
    assert outs == [_greedy(plain, p, 12) for p in prompts]
    eng.cache.check()
    assert eng.cache.num_live() == 0 and all(g_.pool.num_held == 0 for g_ in eng.cache.groups)


@pytest.mark.gpu
def test_greedy_generation_in_bfloat16(folders_bf16):
    """Every generated token is the plain model's first choice after the same tokens, or within bfloat16's
    rounding of it."""
    plain = P.PlainRovidra(folders_bf16["RF"])
    g = torch.Generator().manual_seed(5)
    prompts = [torch.randint(0, 1000, (n,), generator=g).tolist() for n in (40, 3, 120)]
    eng = Engine(load_model(folders_bf16["RF"], "bfloat16", "cuda:0"), cache_tokens=1024, decode_batch_size=4,
                 max_num_batched_tokens=64)
    outs = eng.generate(prompts, SamplingParams(max_decode_length=16))
    for p, out in zip(prompts, outs):
        logits = plain.logits(list(p) + list(out)).float()
        for i, tok in enumerate(out):
            row = logits[len(p) + i - 1]
            assert float(row.max() - row[tok]) <= 5e-2 * float(row.abs().max()), f"token {i} of {out}"


@pytest.mark.gpu
def test_command_line(folders, capsys):
    """``python -m jax_llm_examples_amd.main`` picks the design by config.json like every other entry point."""
    from jax_llm_examples_amd.main import main

    plain = P.PlainRovidra(folders["RA"])
    rc = main(["--ckpt-path", folders["RA"], "--dtype", "float32", "--prompt-ids", "5,6,7,8", "--prompt-ids", "9",
               "--max-decode-length", "6", "--decode-batch-size", "2", "--max-seq-len", "64"])
    assert rc == 0
    lines = [json.loads(ln) for ln in capsys.readouterr().out.strip().splitlines()]
    assert [ln["tokens"] for ln in lines] == [_greedy(plain, [5, 6, 7, 8], 6), _greedy(plain, [9], 6)]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(folders_bf16, tmp_path, dtype):
    """``bin/trace_run`` as a program, on a folder that holds config.json and bfloat16 weights."""
    folder = folders_bf16["RA"]
    reqs = traces.random_requests(300, [40, 9, 70, 21, 33], seed=11)
    steps = traces.mixed(reqs)
    out_dir = tmp_path / "out"
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
                           "--out", str(out_dir), "--max-tokens", str(traces.max_live_tokens(steps)),
                           "--max-requests", "4"],
                          input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [ln for ln in proc.stdout.splitlines() if ln.startswith("done")] == [f"done {s['step']}" for s in steps]
    plain = P.PlainRovidra(folder)
    ref = {rid: plain.logits(toks).float() for rid, toks in reqs.items()}
    at = {rid: 0 for rid in reqs}
    for s in steps:
        got = np.fromfile(out_dir / f"{s['step']}.f32", dtype="<f4").reshape(-1, 300)
        o = 0
        for e in s["entries"]:
            for wnt in e["want"]:
                r = ref[e["id"]][at[e["id"]] + wnt]
                assert float((torch.from_numpy(got[o].copy()) - r).abs().max() / ref[e["id"]].abs().max()) < TOL[dtype]
                o += 1
            at[e["id"]] += len(e["tokens"])


@pytest.mark.gpu
def test_library_of_the_designs_own_sources(folders, tmp_path):
    """A process that starts with the library of only the sources this design names runs the design, and brings the
    whole library in when another model calls a kernel that the partial one lacks."""
    from jax_llm_examples_amd.ops import build

    arch = get_architecture("Rovidra")
    partial = build.find_library(only=arch.kernel_sources)
    if partial is None or build.find_library() is None:
        pytest.skip("the partial kernel library is not built in this tree")
    code = f"""
import sys, torch
sys.path.insert(0, {ROOT!r}); sys.path.insert(0, {os.path.join(ROOT, 'tests')!r})
from jax_llm_examples_amd.ops import hip
hip._LIB = hip._bind({partial!r})
assert not hip._LIB._jle_whole and not hasattr(hip._LIB, "jle_moe_route")
from jax_llm_examples_amd.engine.replay import make_runner
from jax_llm_examples_amd.engine import StepEntry
import plain_rovidra as P
toks = [5, 9, 200, 31, 7, 7, 100, 3]
runner = make_runner({folders['RA']!r}, "float32", 64, "cuda:0", max_requests=2)
got = runner.step([StepEntry("r", toks, list(range(len(toks))))]).cpu()
ref = P.PlainRovidra({folders['RA']!r}).logits(toks).float()
assert float((got - ref).abs().max() / ref.abs().max()) < 2e-5
assert not runner.ops.lib._jle_whole
x = torch.randn(4, 64, device="cuda:0"); r = torch.randn(8, 64, device="cuda:0")
ids, gates = runner.ops.moe_route(x, r, 1)  # a kernel of another source
assert runner.ops.lib._jle_whole and ids.shape == (4, 1)
print("ok")
"""
    proc = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0 and proc.stdout.strip().endswith("ok"), proc.stderr[-2000:]


# ---------------------------------------------------------------------------------------------- configuration, weights
def test_configuration_round_trip_and_plan(folders):
    arch, cfg = load_config(folders["RA"])
    assert arch is get_architecture("Rovidra")
    assert arch.parse_config(json.loads(json.dumps(arch.config_to_dict(cfg)))) == cfg
    plan = arch.plan(cfg)
    assert [(e.layer, e.cache, e.writes_cache) for e in plan.order] == [
        (0, 0, True), (1, 0, False), (2, 2, True), (3, 2, False), (4, 4, True), (5, 4, False)]
    # a cache keeps what its farthest-looking reader needs
    assert plan.layers[0].mixer.retention == ("window", 20) and plan.layers[1].mixer.window == 9
    assert plan.layers[2].mixer.retention == ("all",) and plan.layers[3].mixer.window == 37
    assert plan.layers[4].mixer.retention == ("window", 50) and plan.layers[4].mixer.window == 33
    assert plan.layers[1].feed_forward is None


def test_configuration_errors():
    arch = get_architecture("Rovidra")
    good = rovidra_config_json("RA")

    def broken(change):
        top = json.loads(json.dumps(good))
        change(top)
        return top

    for change, match in [
        (lambda t: t["layers"][1]["mixer"].update(kv_from=1), "earlier layer"),
        (lambda t: t["layers"][3]["mixer"].update(kv_from=1), "latent of its own"),
        (lambda t: t["layers"][1]["mixer"].update(kv_rank=8), "differ"),
        (lambda t: t["layers"][0]["mixer"].pop("vdim"), "vdim"),
        (lambda t: t["layers"][0]["mixer"].update(sink=4), "unknown key"),
        (lambda t: t["layers"][0].update(type="convolution"), "not known"),
        (lambda t: t["layers"][0]["mlp"].update(kind="experts"), "not known"),
        (lambda t: t["layers"][2]["mixer"]["rot"].update(dims=3), "even"),
        (lambda t: t.pop("norm"), "norm"),
    ]:
        with pytest.raises(ConfigError, match=match):
            arch.parse_config(broken(change))


def test_weights_error_names_what_is_missing(folders, tmp_path):
    from safetensors.torch import load_file, save_file

    w = load_file(os.path.join(folders["RB"], "model.safetensors"))
    w.pop("l1.mix.dkv.norm")
    w["l2.mix.dkv"] = torch.zeros(20, 54)  # a reader of another layer's latent has none of its own
    (tmp_path / "m").mkdir()
    save_file(w, str(tmp_path / "m" / "model.safetensors"))
    with open(os.path.join(folders["RB"], "config.json")) as f:
        (tmp_path / "m" / "config.json").write_text(f.read())
    with pytest.raises(WeightsError) as e:
        load_model(str(tmp_path / "m"), "float32", "cpu")
    assert e.value.missing == ["l1.mix.dkv.norm"] and e.value.unexpected == ["l2.mix.dkv"]
