"""Senavik in the engine against the plain implementation (tests/plain_senavik.py): every way of
cutting the work, both precisions, small configurations that differ in every size and branch;
sharp attention over many pages, at the edges of windows and of the kept first tokens; the
denominator's extra term; pages and slots used again; recorded steps; generation through the
entry points."""
import copy
import json
import os
import subprocess
import sys

import pytest
import torch

import cuttings
import plain_senavik
from engine_helpers import (TOL, first_mismatch, load_graph_runner, load_runner,
                            random_sequences, replay, replay_wanted)
from senavik_configs import senavik

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LENGTHS = {"S1": [5, 9, 33, 70, 130, 47], "S2": [3, 17, 40, 65, 31], "S3": [12, 50, 90, 20, 2, 150],
           "S4": [7, 30, 64, 81, 120], "S5": [9, 44, 66, 1], "S6": [150, 21, 77]}
DTYPES = [torch.float32, torch.bfloat16]
NAMES = ["S1", "S2", "S3", "S4", "S5", "S6"]
ROUTER_GAIN = 2.0       # routers this much larger than the other matrices (more would saturate the sigmoid)


def matrix_names(cfg):
    """The tensors an engine holds in its own dtype (the others stay float32)."""
    from pytriton_llama_amd.config import build_model
    return {n for n, (_, src) in build_model(copy.deepcopy(cfg)).expected_tensors().items() if src.kind == "matrix"}


def read_folder(folder, weights_as=None):
    from safetensors.torch import load_file
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    w = load_file(os.path.join(folder, "model.safetensors"))
    if weights_as is not None:      # the values an engine of that dtype holds: matrices are rounded
        rounded = matrix_names(cfg)
        w = {k: (v.to(weights_as).float() if k in rounded else v) for k, v in w.items()}
    return cfg, w


def write_folder(tmp_path_factory, name, seed, sharpen=1.0, cfg=None, sink_shift=0.0):
    """A model folder of random weights. ``sharpen`` multiplies the query projections, which makes
    the softmax pick few keys, so that one key lost or misplaced shows in the logits.
    ``sink_shift`` is added to every sink (the denominator's term without a key)."""
    from safetensors.torch import load_file, save_file
    from pytriton_llama_amd.weights import write_random_model
    base, std, page = senavik(name)
    folder = str(tmp_path_factory.mktemp(f"senavik_{name}"))
    write_random_model(cfg or base, folder, seed=seed, dtype=torch.float32, norm_std=0.1, std=std)
    path = os.path.join(folder, "model.safetensors")
    w = load_file(path)
    for k in list(w):
        if k.endswith(".mix.q") or k.endswith(".mix.uq"):
            w[k] = w[k] * sharpen
        if k.endswith(".mix.sink"):
            w[k] = w[k] + sink_shift
        if k.endswith(".mlp.router"):
            w[k] = w[k] * ROUTER_GAIN
        if k.endswith(".mlp.correction"):
            w[k] = w[k] * 5.0           # (corrections that change which experts are chosen)
    save_file(w, path)
    return folder, page


def plain_logits(folder, seqs, weights_as=None, touchy=None, cfg_change=None, w_change=None):
    """``weights_as``: the plain model with matrices and stored results rounded as an engine of that
    dtype rounds them. ``touchy``: a dict that receives, per request, the positions at which a
    comparison says nothing: those that rounding alone moves by more than half the tolerance in
    the plain model, and those at which a router's choice is a close call that rounding may turn
    (plain_senavik.ROUTER_MARGINS)."""
    cfg, w = read_folder(folder, weights_as)
    if cfg_change is not None:
        cfg_change(cfg)
    if w_change is not None:
        w_change(w)
    out = {}
    with torch.no_grad():
        for rid, toks in seqs.items():
            plain_senavik.ROUTER_MARGINS = [] if touchy is not None else None
            out[rid] = plain_senavik.forward(cfg, w, toks, round_to=weights_as).float()
            if touchy is not None:
                margins, plain_senavik.ROUTER_MARGINS = plain_senavik.ROUTER_MARGINS, None
                exact = plain_senavik.forward(cfg, w, toks).float()
                moved = (out[rid] - exact).abs().amax(dim=-1) / exact.abs().max()
                touchy[rid] = moved > 0.5 * TOL[weights_as]
                for close in margins:
                    touchy[rid] |= close
    plain_senavik.ROUTER_MARGINS = None
    return out


def wrong_places(got, want, dtype):
    """None, or a text that says what is wrong. float32: no place may differ by more than the
    tolerance. bfloat16: a router's choice that rounding turns in the engine and not in the plain
    model (one that the plain model's own margins did not give away) moves a single position by
    any amount, so a few positions may lie beyond the tolerance: at most one in fifty, and none
    by more than four times the tolerance. A key lost, a window off by one or a sink left out
    moves many positions (the sharpened tests make sure of it) and does not pass."""
    tol = TOL[dtype]
    if dtype == torch.float32:
        bad = first_mismatch(got, want, tol)
        return None if bad is None else f"first wrong place (request, position, error) = {bad}"
    errs = []
    for rid in want:
        err = (got[rid] - want[rid]).abs().amax(dim=-1) / float(want[rid].abs().max())
        errs.append(torch.where(torch.isnan(err), torch.full_like(err, float("inf")), err))
    errs = torch.cat(errs)
    over = int((errs > tol).sum())
    if over * 50 > len(errs) + 49 or float(errs.max()) > 4 * tol:
        return f"{over} of {len(errs)} places beyond {tol}, the worst by {float(errs.max()):.3g}"
    return None


def skip_touchy(got, want, touchy):
    for rid, t in touchy.items():
        if rid in got:
            got[rid][t] = want[rid][t]


@pytest.fixture(scope="module")
def cases(tmp_path_factory, gpu_device):
    out = {}
    for i, name in enumerate(NAMES):
        folder, page = write_folder(tmp_path_factory, name, seed=91 + i)
        seqs = random_sequences(senavik(name)[0]["vocab"], LENGTHS[name], seed=37 + i)
        touchy = {}
        want = {torch.float32: plain_logits(folder, seqs),
                torch.bfloat16: plain_logits(folder, seqs, torch.bfloat16, touchy)}
        assert sum(int(c.sum()) for c in touchy.values()) * 2 < sum(len(c) for c in touchy.values()), name
        want["touchy"] = touchy
        out[name] = (folder, page, seqs, want)
    return out


def run_cutting(cases, name, dtype, steps, num_pages=None, max_num_seqs=4):
    folder, page, seqs, want = cases[name]
    if num_pages is None:
        num_pages = -(-cuttings.max_live_tokens(steps, round_to=page) // page)
    runner = load_runner(folder, dtype, page, num_pages, max_num_seqs=max_num_seqs)
    got = replay(runner, steps, seqs)
    if dtype == torch.bfloat16:
        skip_touchy(got, want[dtype], want["touchy"])
    bad = wrong_places(got, {r: want[dtype][r] for r in seqs}, dtype)
    assert bad is None, f"config {name} {dtype}: {bad}"
    assert all(g.pool.num_free == g.pool.num_pages for g in runner.manager.paged)
    assert runner.manager.num_free_slots == max_num_seqs


@pytest.mark.parametrize("dtype", DTYPES, ids=["fp32", "bf16"])
@pytest.mark.parametrize("name", NAMES)
def test_whole(cases, name, dtype):
    run_cutting(cases, name, dtype, cuttings.whole(cases[name][2]))


@pytest.mark.parametrize("dtype", DTYPES, ids=["fp32", "bf16"])
@pytest.mark.parametrize("name", NAMES)
def test_last_tokens_one_by_one(cases, name, dtype):
    run_cutting(cases, name, dtype, cuttings.tail_decode(cases[name][2], 40))


@pytest.mark.parametrize("dtype", DTYPES, ids=["fp32", "bf16"])
@pytest.mark.parametrize("name", NAMES)
def test_portions_down_to_two_tokens(cases, name, dtype):
    run_cutting(cases, name, dtype, cuttings.portions(cases[name][2]))


@pytest.mark.parametrize("name", NAMES)
def test_first_tokens_one_by_one_then_portions(cases, name):
    """The first tokens of a sequence alone: a window that is not full yet, kept tokens that are
    still inside it, the first pages."""
    run_cutting(cases, name, torch.float32,
                cuttings.portions(cases[name][2], sizes=(1, 1, 2, 1, 3, 16, 1, 15, 2, 32)))


@pytest.mark.parametrize("name", NAMES)
def test_every_token_alone(cases, name):
    """Token-by-token decoding from the first token on against the whole prompt."""
    folder, page, seqs, want = cases[name]
    short = {r: t for r, t in seqs.items() if len(t) <= 70}
    steps = cuttings.portions(short, sizes=(1,))
    runner = load_runner(folder, torch.float32, page, 32, max_num_seqs=4)
    got = replay(runner, steps, short)
    assert first_mismatch(got, {r: want[torch.float32][r] for r in short}, TOL[torch.float32]) is None


@pytest.mark.parametrize("dtype", DTYPES, ids=["fp32", "bf16"])
@pytest.mark.parametrize("name", NAMES)
def test_mixed_batches_with_pages_and_slots_used_again(cases, name, dtype):
    folder, page, seqs, want = cases[name]
    seqs = {r: t for r, t in seqs.items() if len(t) >= 2}      # (a prompt portion and a decoded token each)
    steps = cuttings.mixed(seqs, seed=5, max_live=3)
    need = cuttings.max_live_tokens(steps, round_to=page) // page
    assert need < sum(-(-len(t) // page) for t in seqs.values())
    run_cutting({name: (folder, page, seqs, want)}, name, dtype, steps, need, max_num_seqs=3)


@pytest.mark.parametrize("name", NAMES)
def test_slots_and_pages_that_are_used_again(cases, name):
    """Two slots for all requests, one after the other: every request but the first two gets a
    slot and pages that another one has filled."""
    folder, page, seqs, want = cases[name]
    runner = load_runner(folder, torch.float32, page, 48, max_num_seqs=2)
    got = replay(runner, cuttings.portions(seqs, sizes=(9, 1, 30)), seqs)
    assert first_mismatch(got, want[torch.float32], TOL[torch.float32]) is None
    got = replay(runner, cuttings.whole(seqs), seqs)          # and once more, on used pages throughout
    assert first_mismatch(got, want[torch.float32], TOL[torch.float32]) is None


@pytest.mark.parametrize("name", NAMES)
def test_a_batch_gives_what_each_request_gives_alone(cases, name):
    """Unequal requests in one step against each alone (float32: the differences are those of
    the order of sums only)."""
    folder, page, seqs, _ = cases[name]
    runner = load_runner(folder, torch.float32, page, 96, max_num_seqs=8)
    alone = replay(runner, cuttings.whole(seqs), seqs)
    together = [{"step": 0, "end": list(seqs),
                 "entries": [{"id": r, "tokens": t, "want": list(range(len(t)))} for r, t in seqs.items()]}]
    batch = replay(runner, together, seqs)
    assert first_mismatch(batch, alone, 2e-6) is None


def _windows(cfg, by):
    for l in cfg["layers"]:
        if l["type"] == "attention" and "mask" in l["mixer"]:
            l["mixer"]["mask"]["size"] += by


def _kept(cfg, by):
    for l in cfg["layers"]:
        if l["type"] == "attention" and "mask" in l["mixer"]:
            l["mixer"]["mask"]["keep_first"] += by


def _no_sinks(w):
    for k in list(w):
        if k.endswith(".mix.sink"):
            w[k] = torch.full_like(w[k], -1e4)


def _long_steps(seqs, decoded, sizes=(33, 2, 61, 16, 7, 90)):
    steps = []
    for rid, toks in seqs.items():
        n, lo, k = len(toks), 0, 0
        head = max(1, n - decoded)
        while lo < head:
            hi = min(head, lo + sizes[k % len(sizes)])
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[lo:hi],
                                                           "want": list(range(hi - lo))}], "end": []})
            lo, k = hi, k + 1
        for i in range(head, n):
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[i:i + 1], "want": [0]}],
                          "end": [rid] if i == n - 1 else []})
    return steps


@pytest.mark.parametrize("dtype", DTYPES, ids=["fp32", "bf16"])
def test_sharp_attention_over_many_pages_at_the_windows_edges_and_the_kept_tokens(tmp_path_factory, gpu_device, dtype):
    """Query projections six times as large in a model of attention layers only: the softmax picks
    few keys, so a key lost at a page border, counted twice, one token inside or outside a
    window's edge, or a kept token more or less changes the logits. A long prompt in portions that
    end inside pages and inside windows, and 150 tokens decoded one by one across page borders
    while the windows move on and the pages behind them are given back."""
    folder, page = write_folder(tmp_path_factory, "S4", seed=77, sharpen=6.0)
    seqs = random_sequences(200, [420, 37], seed=3)
    # scores six times as large carry the rounding of the angles six times as far; the float32 run
    # is held to 1e-3 here, still far below what a lost key or an edge off by one does (checked first)
    tol = 1e-3 if dtype == torch.float32 else TOL[dtype]
    rounded = None if dtype == torch.float32 else dtype
    touchy = {}
    want = plain_logits(folder, seqs, rounded, touchy if rounded else None)
    # the test means something only if single far keys, the edges and the sinks matter
    moved = seqs["r0"][:2] + [(seqs["r0"][2] + 1) % 200] + seqs["r0"][3:]
    other = plain_logits(folder, {"r0": moved}, rounded)["r0"]
    assert float((other[-50:] - want["r0"][-50:]).abs().max() / want["r0"].abs().max()) > 2.5 * tol
    changes = [dict(cfg_change=lambda c: _windows(c, 1)), dict(cfg_change=lambda c: _windows(c, -1)),
               dict(cfg_change=lambda c: _kept(c, 1)), dict(cfg_change=lambda c: _kept(c, -1)),
               dict(w_change=_no_sinks)]
    for change in changes:
        other = plain_logits(folder, {"r0": seqs["r0"]}, rounded, **change)["r0"]
        off = (other - want["r0"]).abs().amax(-1) / want["r0"].abs().max()
        assert int((off[60:270] > 2.5 * tol).sum()) > 20 and int((off[270:] > 2.5 * tol).sum()) > 20
    runner = load_runner(folder, dtype, page, 64, max_num_seqs=2)
    got = replay(runner, _long_steps(seqs, 150), seqs)
    skip_touchy(got, want, touchy)
    bad = first_mismatch(got, want, tol) if dtype == torch.float32 else wrong_places(got, want, dtype)
    assert bad is None, bad


@pytest.mark.parametrize("name", ["S1", "S3"])
def test_sharp_latent_attention_and_large_sinks(tmp_path_factory, gpu_device, name):
    """The same for models with latent layers (their keys are never given back: position 2 is read
    from hundreds of tokens on), with sinks far above and far below the scores in turn."""
    for shift in (4.0, -6.0):
        folder, page = write_folder(tmp_path_factory, name, seed=79, sharpen=4.0, sink_shift=shift)
        vocab = senavik(name)[0]["vocab"]
        seqs = random_sequences(vocab, [300, 21], seed=5)
        want = plain_logits(folder, seqs)
        moved = seqs["r0"][:2] + [(seqs["r0"][2] + 1) % vocab] + seqs["r0"][3:]
        other = plain_logits(folder, {"r0": moved})["r0"]
        assert float((other[-50:] - want["r0"][-50:]).abs().max() / want["r0"].abs().max()) > 2.5e-3
        other = plain_logits(folder, {"r0": seqs["r0"]}, w_change=_no_sinks)["r0"]
        assert float((other - want["r0"]).abs().max() / want["r0"].abs().max()) > 2.5e-3
        runner = load_runner(folder, torch.float32, page, 96, max_num_seqs=2)
        got = replay(runner, _long_steps(seqs, 100, sizes=(17, 2, 45, 16, 5)), seqs)
        assert first_mismatch(got, want, 1e-3) is None


def test_long_decoding(cases):
    """300 tokens one by one behind a short prompt: the windows leave their pages behind, the kept
    pages stay, the latent layers read everything."""
    folder, page = cases["S1"][0], cases["S1"][1]
    seqs = random_sequences(200, [320], seed=9)
    want = plain_logits(folder, seqs)
    runner = load_runner(folder, torch.float32, page, 96, max_num_seqs=2)
    got = replay(runner, cuttings.tail_decode(seqs, 300), seqs)
    assert first_mismatch(got, want, TOL[torch.float32]) is None


def test_pages_behind_a_window_are_given_back_and_the_kept_ones_stay(cases):
    """A model whose attention layers all have windows holds a bounded number of their pages however
    long the request grows: those of the window, of the step's portion and of the kept tokens."""
    folder, page = cases["S5"][0], cases["S5"][1]
    seqs = random_sequences(120, [260], seed=11)
    want = plain_logits(folder, seqs)
    runner = load_runner(folder, torch.float32, page, [12, 70, 12, 70], max_num_seqs=1)
    groups = runner.manager.paged
    windowed = [g for g in groups if g.spec.window is not None and g.spec.window < 100]
    assert len(windowed) == 2 and len(groups) == 4
    got = replay(runner, cuttings.portions(seqs, sizes=(16, 3, 1, 1, 9)), seqs)
    assert first_mismatch(got, want, TOL[torch.float32]) is None


@pytest.mark.parametrize("dtype", DTYPES, ids=["fp32", "bf16"])
@pytest.mark.parametrize("name", ["S1", "S3", "S5", "S6"])
def test_cuttings_replayed_as_graphs(cases, name, dtype):
    """Decode steps and single portions replayed as HIP graphs (padded layouts: rows that belong
    to nobody) against the plain model."""
    folder, page, seqs, want = cases[name]
    longer = {r: t for r, t in seqs.items() if len(t) >= 2}
    for steps in (cuttings.tail_decode(seqs, 24), cuttings.mixed(longer, seed=9, max_live=3)):
        for st in steps:
            for e in st["entries"]:
                e["want"] = e["want"][-1:]
        places = cuttings.wanted_places(steps)
        runner = load_graph_runner(folder, dtype, page, 128, max_model_len=160, max_num_seqs=4)
        got = replay_wanted(runner, steps)
        rows = {r: want[dtype][r][torch.as_tensor(places[r])] for r in got}
        if dtype == torch.bfloat16:
            skip_touchy(got, rows, {r: want["touchy"][r][torch.as_tensor(places[r])] for r in got})
        bad = wrong_places(got, rows, dtype)
        assert bad is None, f"{name} {dtype}: {bad}"


@pytest.mark.parametrize("seed", range(12))
def test_drawn_configurations(tmp_path_factory, gpu_device, seed):
    """Configurations drawn at random from the ranges of the design, pages of 16: whole prompts,
    the last tokens one by one, and mixed batches on few pages, in both precisions."""
    from senavik_configs import drawn
    cfg, std, page = drawn(seed)
    folder, _ = write_folder(tmp_path_factory, "S1", seed=200 + seed, cfg=cfg)
    seqs = random_sequences(cfg["vocab"], [190, 45, 3, 101], seed=seed)
    touchy = {}
    want = {torch.float32: plain_logits(folder, seqs), torch.bfloat16: plain_logits(folder, seqs, torch.bfloat16, touchy),
            "touchy": touchy}
    cases = {"D": (folder, page, seqs, want)}
    for dtype in DTYPES:
        run_cutting(cases, "D", dtype, cuttings.tail_decode(seqs, 36))
        steps = cuttings.mixed(seqs, seed=seed, max_live=3)
        run_cutting(cases, "D", dtype, steps, cuttings.max_live_tokens(steps, round_to=page) // page, max_num_seqs=3)
    run_cutting(cases, "D", torch.float32, cuttings.portions(seqs))


def plain_greedy(folder, prompt, n):
    cfg, w = read_folder(folder)
    toks = list(prompt)
    with torch.no_grad():
        for _ in range(n):
            toks.append(int(plain_senavik.forward(cfg, w, toks)[-1].argmax()))
    return toks[len(prompt):]


def test_greedy_generation_through_the_entry_point(cases):
    from pytriton_llama_amd.generate import GenerateText
    folder, page = cases["S1"][0], cases["S1"][1]
    g = torch.Generator().manual_seed(4)
    prompts = [torch.randint(0, 200, (n,), generator=g).tolist() for n in (4, 11, 19, 26)]
    want = [plain_greedy(folder, p, 10) for p in prompts]
    gen = GenerateText(folder, max_seq_len=64, max_gpu_num_blocks=64, dtype="float32", page_size=page,
                       max_batch_size=4)
    got, _ = gen.generate(prompts, max_gen_len=10, temperature=0.0)
    assert got == want


def test_scheduler_with_few_pages_preempts_and_gives_the_same_tokens(cases):
    from pytriton_llama_amd.config import EngineConfig
    from pytriton_llama_amd.engine import Engine, SamplingParams
    folder, page = cases["S2"][0], cases["S2"][1]
    g = torch.Generator().manual_seed(6)
    prompts = [torch.randint(0, 150, (n,), generator=g).tolist() for n in (6, 9, 14, 17)]
    sp = SamplingParams(temperature=0.0, max_new_tokens=12)
    want = [plain_greedy(folder, p, 12) for p in prompts]
    tight = Engine(folder, EngineConfig(dtype="float32", page_size=page, num_pages=8, max_num_seqs=4,
                                        max_model_len=64, max_num_batched_tokens=16, prefill_chunk=6))
    got = tight.generate(prompts, sp)
    assert tight.scheduler.num_preemptions > 0
    assert got == want
    tight.runner.manager.check()
    assert tight.runner.manager.num_free_slots == 4


def test_command_line_and_trace_replay(cases, tmp_path):
    folder, page, seqs, want = cases["S3"]
    prompt = seqs["r0"]
    out = subprocess.run(
        [sys.executable, os.path.join(ROOT, "cli.py"), "--checkpoints_dir", folder, "--dtype", "float32",
         "--temperature", "0", "--max_gen_len", "4", "--max_seq_len", "64", "--max_gpu_num_blocks", "16",
         "--page_size", str(page), "--prompt_ids", ",".join(map(str, prompt))],
        capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    assert " ".join(map(str, plain_greedy(folder, prompt, 4))) in " ".join(out.stdout.split())
    steps = cuttings.mixed(seqs, seed=2, max_live=4)
    lines = "\n".join(json.dumps(s) for s in steps) + "\n"
    run = subprocess.run(
        [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32",
         "--out", str(tmp_path), "--max-tokens", str(cuttings.max_live_tokens(steps))],
        input=lines, capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr[-2000:]
    assert [l for l in run.stdout.splitlines() if l.startswith("done")] == [f"done {s['step']}" for s in steps]
    import numpy as np
    fed = {r: 0 for r in seqs}
    for s in steps:
        got = torch.from_numpy(np.fromfile(str(tmp_path / f"{s['step']}.f32"), dtype="<f4")).view(-1, 180)
        row = 0
        for e in s["entries"]:
            n = len(e["tokens"])
            ref = want[torch.float32][e["id"]][fed[e["id"]]:fed[e["id"]] + n]
            assert float((got[row:row + n] - ref).abs().max() / ref.abs().max()) < 2e-5
            row, fed[e["id"]] = row + n, fed[e["id"]] + n
