"""Virusun in the engine against the plain implementation (tests/plain_virusun.py): every way of
cutting the work, both precisions, small configurations that differ in every size and branch;
sharp attention over many pages; state and pages used again; recorded steps; generation through
the entry points."""
import json
import os
import subprocess
import sys

import pytest
import torch

import cuttings
import plain_virusun
from engine_helpers import (TOL, first_mismatch, first_wrong_row, load_graph_runner, load_runner,
                            random_sequences, replay, replay_wanted)
from virusun_configs import virusun

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LENGTHS = {"V1": [5, 9, 33, 70, 130, 47], "V2": [3, 17, 40, 65, 31], "V3": [12, 50, 90, 20, 2],
           "V4": [7, 30, 64, 81], "V5": [9, 140, 66, 35]}
DTYPES = [torch.float32, torch.bfloat16]
NAMES = ["V1", "V2", "V3", "V4", "V5"]


def read_folder(folder, weights_as=None):
    from safetensors.torch import load_file
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    w = load_file(os.path.join(folder, "model.safetensors"))
    if weights_as is not None:      # the values an engine of that dtype holds: matrices are rounded
        w = {k: (v.to(weights_as).float() if v.dim() == 2 and not k.endswith(".conv") else v) for k, v in w.items()}
    return cfg, w


def write_folder(tmp_path_factory, name, seed, sharpen=1.0, tame=False):
    """A model folder of random weights. ``sharpen`` multiplies the weights of the query norms,
    which makes the softmax pick few keys, so that one key lost or misplaced shows in the logits
    (the queries are normed: a larger projection would change nothing). ``tame``: the recurrent
    mixers' key projections (and convolutions) are their query projections, so that a token's
    query is never at right angles to its own key: behind few tokens the read-out S^T q is then
    never the small rest of a cancellation whose sign the rounding of bfloat16 decides, which the
    norm behind the mixer would blow up and later attention layers would spread over the positions
    that follow. The float32 tests run on the untamed weights."""
    from safetensors.torch import load_file, save_file
    from pytriton_llama_amd.weights import write_random_model
    cfg, std, page = virusun(name)
    folder = str(tmp_path_factory.mktemp(f"virusun_{name}"))
    write_random_model(cfg, folder, seed=seed, dtype=torch.float32, norm_std=0.1, std=std)
    if sharpen != 1.0 or tame:
        path = os.path.join(folder, "model.safetensors")
        w = load_file(path)
        for k in list(w):
            if k.endswith(".q.norm"):
                w[k] = w[k] * sharpen
            if tame and k.endswith(".mix.right.k"):
                w[k] = w[k[:-1] + "q"].clone()
            if tame and k.endswith(".mix.A_log"):
                pre = k[:-len("A_log")]
                w[pre + "k"], w[pre + "k.conv"] = w[pre + "q"].clone(), w[pre + "q.conv"].clone()
        save_file(w, path)
    return folder, page


def plain_logits(folder, seqs, weights_as=None, touchy=None):
    """``weights_as``: the plain model with matrices and sublayer inputs rounded as an engine of
    that dtype rounds them. ``touchy``: a dict that receives, per request, the positions at which a
    comparison says nothing: those that rounding alone moves by more than half the tolerance in the
    plain model, and those at which a recurrent mixer's read-out keeps less than a twentieth of its
    size after cancellation (behind a single token: a query nearly at right angles to the key).
    The norm behind the mixer keeps the direction of the read-out and drops its size, so there the
    direction is decided by the rounding."""
    cfg, w = read_folder(folder, weights_as)
    out = {}
    with torch.no_grad():
        for rid, toks in seqs.items():
            out[rid] = plain_virusun.forward(cfg, w, toks, round_inputs=weights_as).float()
            if touchy is not None:
                left = []
                exact = plain_virusun.forward(cfg, w, toks, cancellation_out=left).float()
                moved = (out[rid] - exact).abs().amax(dim=-1) / exact.abs().max()
                touchy[rid] = moved > 0.5 * TOL[weights_as]
                for ratio in left:
                    touchy[rid] |= ratio < 1.0 / 20
    return out


def skip_touchy(got, want, touchy):
    for rid, t in touchy.items():
        if rid in got:
            got[rid][t] = want[rid][t]


@pytest.fixture(scope="module")
def cases(tmp_path_factory, gpu_device):
    out = {}
    for i, name in enumerate(NAMES):
        folder, page = write_folder(tmp_path_factory, name, seed=41 + i)
        tamed, _ = write_folder(tmp_path_factory, name, seed=41 + i, tame=True)
        seqs = random_sequences(virusun(name)[0]["vocab"], LENGTHS[name], seed=17 + i)
        touchy = {}
        want = {torch.float32: plain_logits(folder, seqs),
                torch.bfloat16: plain_logits(tamed, seqs, torch.bfloat16, touchy)}
        assert sum(int(c.sum()) for c in touchy.values()) * 3 < sum(len(c) for c in touchy.values())
        want["touchy"] = touchy
        out[name] = ({torch.float32: folder, torch.bfloat16: tamed}, page, seqs, want)
    return out


def run_cutting(cases, name, dtype, steps, num_pages=None):
    folders, page, seqs, want = cases[name]
    if num_pages is None:
        num_pages = -(-cuttings.max_live_tokens(steps, round_to=page) // page)
    runner = load_runner(folders[dtype], dtype, page, num_pages, max_num_seqs=4)
    got = replay(runner, steps, seqs)
    if dtype == torch.bfloat16:
        skip_touchy(got, want[dtype], want["touchy"])
    bad = first_mismatch(got, want[dtype], TOL[dtype])
    assert bad is None, f"config {name} {dtype}: first wrong place (request, position, error) = {bad}"
    assert all(g.pool.num_free == g.pool.num_pages for g in runner.manager.paged)
    assert runner.manager.num_free_slots == 4


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
    """The first tokens of a sequence alone: convolutions that reach before the start, a state
    that starts from zero, a running maximum that starts at 0."""
    run_cutting(cases, name, torch.float32,
                cuttings.portions(cases[name][2], sizes=(1, 1, 2, 1, 3, 16, 1, 15, 2, 32)))


@pytest.mark.parametrize("name", NAMES)
def test_every_token_alone(cases, name):
    """Token-by-token decoding from the first token on against the whole prompt."""
    folders, page, seqs, want = cases[name]
    folder = folders[torch.float32]
    short = {r: t for r, t in seqs.items() if len(t) <= 70}
    steps = cuttings.portions(short, sizes=(1,))
    runner = load_runner(folder, torch.float32, page, 32, max_num_seqs=4)
    got = replay(runner, steps, short)
    assert first_mismatch(got, {r: want[torch.float32][r] for r in short}, TOL[torch.float32]) is None


@pytest.mark.parametrize("dtype", DTYPES, ids=["fp32", "bf16"])
@pytest.mark.parametrize("name", NAMES)
def test_mixed_batches_with_pages_and_slots_used_again(cases, name, dtype):
    _, page, seqs, _ = cases[name]
    steps = cuttings.mixed(seqs, seed=5, max_live=3)
    need = cuttings.max_live_tokens(steps, round_to=page) // page
    assert need < sum(-(-len(t) // page) for t in seqs.values())
    run_cutting(cases, name, dtype, steps, need)


@pytest.mark.parametrize("name", NAMES)
def test_a_slot_that_is_used_again_starts_from_zero(cases, name):
    """Two state slots for all requests, one after the other: every request but the first two
    gets a slot (and pages) that another one has filled."""
    folders, page, seqs, want = cases[name]
    runner = load_runner(folders[torch.float32], torch.float32, page, 24, max_num_seqs=2)
    got = replay(runner, cuttings.portions(seqs, sizes=(9, 1, 30)), seqs)
    assert first_mismatch(got, want[torch.float32], TOL[torch.float32]) is None
    got = replay(runner, cuttings.whole(seqs), seqs)          # and once more, on used slots throughout
    assert first_mismatch(got, want[torch.float32], TOL[torch.float32]) is None


@pytest.mark.parametrize("name", NAMES)
def test_a_batch_gives_what_each_request_gives_alone(cases, name):
    """Unequal requests in one step against each alone (float32: the differences are those of
    the order of sums only)."""
    folders, page, seqs, _ = cases[name]
    runner = load_runner(folders[torch.float32], torch.float32, page, 64, max_num_seqs=8)
    alone = replay(runner, cuttings.whole(seqs), seqs)
    together = [{"step": 0, "end": list(seqs),
                 "entries": [{"id": r, "tokens": t, "want": list(range(len(t)))} for r, t in seqs.items()]}]
    batch = replay(runner, together, seqs)
    assert first_mismatch(batch, alone, 2e-6) is None


@pytest.mark.parametrize("dtype", DTYPES, ids=["fp32", "bf16"])
def test_sharp_attention_over_many_pages(tmp_path_factory, gpu_device, dtype):
    """Query norms six times as large in a model of attention layers only: the softmax picks few
    keys, near and far, so a key lost at a page border or counted twice changes the logits. A long
    prompt in portions that end inside pages, and 150 tokens decoded one by one across page
    borders."""
    folder, page = write_folder(tmp_path_factory, "V4", seed=77, sharpen=6.0)
    seqs = random_sequences(200, [420, 37], seed=3)
    rounded = None if dtype == torch.float32 else dtype
    touchy = {}
    want = plain_logits(folder, seqs, rounded, touchy if rounded else None)
    # the test means something only if single far keys matter: change the third token and the
    # last logits move by much more than the tolerance
    moved = seqs["r0"][:2] + [(seqs["r0"][2] + 1) % 200] + seqs["r0"][3:]
    other = plain_logits(folder, {"r0": moved}, rounded)["r0"]
    shift = float((other[-50:] - want["r0"][-50:]).abs().max() / want["r0"].abs().max())
    assert shift > 2.5 * TOL[dtype], shift
    steps = []
    for rid, toks in seqs.items():
        n, lo, k = len(toks), 0, 0
        sizes = (33, 2, 61, 16, 7, 90)
        head = max(1, n - 150)
        while lo < head:
            hi = min(head, lo + sizes[k % len(sizes)])
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[lo:hi],
                                                           "want": list(range(hi - lo))}], "end": []})
            lo, k = hi, k + 1
        for i in range(head, n):
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[i:i + 1], "want": [0]}],
                          "end": [rid] if i == n - 1 else []})
    runner = load_runner(folder, dtype, page, 32, max_num_seqs=2)
    got = replay(runner, steps, seqs)
    skip_touchy(got, want, touchy)
    bad = first_mismatch(got, want, TOL[dtype])
    assert bad is None, bad


def test_long_decoding_keeps_the_state(cases):
    """300 tokens one by one behind a short prompt: the matrices, the running maximum and the
    convolutions' inputs are carried through every step."""
    folder, page = cases["V1"][0][torch.float32], cases["V1"][1]
    seqs = random_sequences(200, [320], seed=9)
    want = plain_logits(folder, seqs)
    runner = load_runner(folder, torch.float32, page, 24, max_num_seqs=2)
    got = replay(runner, cuttings.tail_decode(seqs, 300), seqs)
    assert first_mismatch(got, want, TOL[torch.float32]) is None


@pytest.mark.parametrize("dtype", DTYPES, ids=["fp32", "bf16"])
@pytest.mark.parametrize("name", ["V1", "V3", "V5"])
def test_cuttings_replayed_as_graphs(cases, name, dtype):
    """Decode steps and single portions replayed as HIP graphs (padded layouts: rows that belong
    to nobody, the padding state slot) against the plain model."""
    folders, page, seqs, want = cases[name]
    folder = folders[dtype]
    for steps in (cuttings.tail_decode(seqs, 24), cuttings.mixed(seqs, seed=9, max_live=3)):
        for st in steps:
            for e in st["entries"]:
                e["want"] = e["want"][-1:]
        places = cuttings.wanted_places(steps)
        runner = load_graph_runner(folder, dtype, page, 64, max_model_len=160, max_num_seqs=4)
        got = replay_wanted(runner, steps)
        rows = {r: want[dtype][r][torch.as_tensor(places[r])] for r in got}
        if dtype == torch.bfloat16:
            skip_touchy(got, rows, {r: want["touchy"][r][torch.as_tensor(places[r])] for r in got})
        bad = first_wrong_row(got, rows, places, TOL[dtype])
        assert bad is None, f"{name} {dtype}: {bad}"


def plain_greedy(folder, prompt, n):
    cfg, w = read_folder(folder)
    toks = list(prompt)
    with torch.no_grad():
        for _ in range(n):
            toks.append(int(plain_virusun.forward(cfg, w, toks)[-1].argmax()))
    return toks[len(prompt):]


def test_greedy_generation_through_the_entry_point(cases):
    from pytriton_llama_amd.generate import GenerateText
    folder, page = cases["V1"][0][torch.float32], cases["V1"][1]
    g = torch.Generator().manual_seed(4)
    prompts = [torch.randint(0, 200, (n,), generator=g).tolist() for n in (4, 11, 19, 26)]
    want = [plain_greedy(folder, p, 10) for p in prompts]
    gen = GenerateText(folder, max_seq_len=64, max_gpu_num_blocks=16, dtype="float32", page_size=page,
                       max_batch_size=4)
    got, _ = gen.generate(prompts, max_gen_len=10, temperature=0.0)
    assert got == want


def test_scheduler_with_few_pages_preempts_and_gives_the_same_tokens(cases):
    from pytriton_llama_amd.config import EngineConfig
    from pytriton_llama_amd.engine import Engine, SamplingParams
    folder, page = cases["V2"][0][torch.float32], cases["V2"][1]
    g = torch.Generator().manual_seed(6)
    prompts = [torch.randint(0, 150, (n,), generator=g).tolist() for n in (6, 9, 14, 17)]
    sp = SamplingParams(temperature=0.0, max_new_tokens=12)
    want = [plain_greedy(folder, p, 12) for p in prompts]
    tight = Engine(folder, EngineConfig(dtype="float32", page_size=page, num_pages=15, max_num_seqs=4,
                                        max_model_len=64, max_num_batched_tokens=16, prefill_chunk=6))
    got = tight.generate(prompts, sp)
    assert tight.scheduler.num_preemptions > 0
    assert got == want
    tight.runner.manager.check()
    assert tight.runner.manager.num_free_slots == 4


def test_command_line_and_trace_replay(cases, tmp_path):
    folders, page, seqs, want = cases["V3"]
    folder = folders[torch.float32]
    prompt = seqs["r0"]
    out = subprocess.run(
        [sys.executable, os.path.join(ROOT, "cli.py"), "--checkpoints_dir", folder, "--dtype", "float32",
         "--temperature", "0", "--max_gen_len", "4", "--max_seq_len", "64", "--max_gpu_num_blocks", "8",
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
        got = torch.from_numpy(np.fromfile(str(tmp_path / f"{s['step']}.f32"), dtype="<f4")).view(-1, 120)
        row = 0
        for e in s["entries"]:
            n = len(e["tokens"])
            ref = want[torch.float32][e["id"]][fed[e["id"]]:fed[e["id"]] + n]
            assert float((got[row:row + n] - ref).abs().max() / ref.abs().max()) < 2e-5
            row, fed[e["id"]] = row + n, fed[e["id"]] + n


@pytest.mark.parametrize("graphs", [False, True], ids=["eager", "graphs"])
def test_long_portions_take_the_recurrences_in_segments(cases, graphs):
    """Portions of 900 and 300 tokens (the recurrent mixers walk them in segments side by side), the
    first followed by portions that start inside a segment and by tokens one by one from the state
    the segments left; launched kernel by kernel and replayed as graphs."""
    from pytriton_llama_amd import ops
    folders, page, _, _ = cases["V5"]
    folder = folders[torch.float32]
    seqs = random_sequences(180, [1240, 310], seed=21)
    assert 900 >= ops.DELTA_SEGMENTS_FROM and 300 >= ops.MEMORY_SEGMENTS_FROM
    want = plain_logits(folder, seqs)
    steps, at = [], {"r0": 0, "r1": 0}
    for rid, n in (("r0", 900), ("r1", 300), ("r0", 330), ("r1", 1), ("r1", 1)) + (("r0", 1),) * 10 + (("r1", 8),):
        lo = at[rid]
        at[rid] = hi = lo + n
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": seqs[rid][lo:hi], "want": [n - 1]}],
                      "end": [rid] if hi == len(seqs[rid]) else []})
    assert at == {r: len(t) for r, t in seqs.items()}
    places = cuttings.wanted_places(steps)
    if graphs:
        runner = load_graph_runner(folder, torch.float32, page, 128, max_model_len=1280, max_num_seqs=2)
    else:
        runner = load_runner(folder, torch.float32, page, 128, max_num_seqs=2)
    got = replay_wanted(runner, steps)
    rows = {r: want[r][torch.as_tensor(places[r])] for r in got}
    bad = first_wrong_row(got, rows, places, TOL[torch.float32])
    assert bad is None, bad
