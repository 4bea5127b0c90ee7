"""The engine against the plain implementation, in 32-bit and in bfloat16,
under every way of cutting the same requests into steps."""

import json
import os
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

import traces
from helpers import assert_close, make_runner, plain_logits, run_trace, save_model_folder
from plain_llama import TINY_A, TINY_B, TINY_C, plain_forward, plain_random_weights

# one kv head for 32 query heads (wider than the MFMA kernels' groups), head size 24 (not a multiple of 16)
TINY_D = dict(TINY_A, hidden_size=32 * 24, num_attention_heads=32, num_key_value_heads=1, intermediate_size=136,
              num_hidden_layers=1, vocab_size=131, tie_word_embeddings=False)

pytestmark = pytest.mark.gpu

REPO = Path(__file__).resolve().parent.parent
DTYPES = [torch.float32, torch.bfloat16]
# config, weight seed, page size, request lengths
CASES = {
    "A": (TINY_A, 0, 16, {"a": 5, "b": 17, "c": 33, "d": 100, "e": 64, "f": 1}),
    "B": (TINY_B, 1, 32, {"a": 1, "b": 12, "c": 40, "d": 90, "e": 150, "f": 129}),
    "C": (TINY_C, 2, 64, {"a": 70, "b": 200, "c": 2, "d": 64, "e": 131}),
    "D": (TINY_D, 3, 8, {"a": 9, "b": 70, "c": 33, "d": 3, "e": 40}),
}


def sharpen(weights, factor=10.0):
    """Random N(0, 0.02) projections give nearly flat attention, which would
    hide a key that is missed or read from a wrong page; larger q/k
    projections make single scores stand out."""
    return {k: v * factor if ("q_proj" in k or "k_proj" in k) else v for k, v in weights.items()}


@pytest.fixture(scope="module", params=sorted(CASES))
def case(request, tmp_path_factory):
    cfg, seed, page, lengths = CASES[request.param]
    weights = sharpen(plain_random_weights(cfg, seed))
    # the bfloat16 engine sees bfloat16 weights; the plain runs get the same values
    weights = {k: v.to(torch.bfloat16).float() for k, v in weights.items()}
    folder = save_model_folder(tmp_path_factory.mktemp(f"tiny{request.param}"), cfg, weights)
    g = torch.Generator().manual_seed(100 + seed)
    tokens = {rid: torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist() for rid, n in lengths.items()}
    want = plain_logits(weights, cfg, tokens)
    noise = plain_logits(weights, cfg, tokens, torch.bfloat16)
    return dict(cfg=cfg, page=page, lengths=lengths, folder=folder, tokens=tokens, want=want, noise=noise,
                weights=weights)


def _check(case, dtype, trace, max_tokens=None, what=""):
    need = traces.max_live_tokens(trace, round_to=max(64, case["page"]))
    runner = make_runner(case["folder"], dtype, case["page"], max_tokens or need)
    got = run_trace(runner, trace, case["tokens"])
    assert runner.cache.live_requests() == []
    assert_close(got, case["want"], dtype, case["noise"], what)


@pytest.mark.parametrize("dtype", DTYPES)
def test_whole(case, dtype):
    _check(case, dtype, traces.whole(case["lengths"]), what="whole")


@pytest.mark.parametrize("dtype", DTYPES)
def test_last_32_one_by_one(case, dtype):
    _check(case, dtype, traces.tail(case["lengths"], 32), what="tail")


@pytest.mark.parametrize("dtype", DTYPES)
def test_portions_of_changing_size(case, dtype):
    _check(case, dtype, traces.chunks(case["lengths"]), what="chunks")
    _check(case, dtype, traces.chunks(case["lengths"], sizes=(2, 2, 3, 16, 1, 31, 33)), what="chunks2")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("seed", [0, 1])
def test_mixed_with_pages_used_again(case, dtype, seed):
    trace = traces.mixed(case["lengths"], max_live=4, seed=seed)
    assert any(len(e) >= 3 for e, _ in trace)
    need = traces.max_live_tokens(trace, round_to=max(64, case["page"]))
    total = sum(-(-n // 64) * 64 for n in case["lengths"].values())
    assert need < total  # so few pages that finished requests' pages are used again
    _check(case, dtype, trace, max_tokens=need, what=f"mixed{seed}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_token_by_token_from_the_first(case, dtype):
    """The first tokens of a sequence, and long decoding: one token a step
    from position 0 on."""
    rid = max(case["lengths"], key=case["lengths"].get)
    n = case["lengths"][rid]
    trace = [([(rid, p, 1)], [rid] if p == n - 1 else []) for p in range(n)]
    runner = make_runner(case["folder"], dtype, case["page"], 64 * -(-n // 64))
    got = run_trace(runner, trace, case["tokens"])
    assert_close(got, {rid: case["want"][rid]}, dtype, case["noise"], "one-by-one")


@pytest.mark.parametrize("dtype,min_tiles", [(torch.float32, 4), (torch.bfloat16, 4), (torch.bfloat16, 1)])
def test_long_decoding_of_a_batch(dtype, min_tiles, tmp_path, monkeypatch):
    """Three requests decode together for hundreds of steps (the captured decode
    step is replayed while block tables grow over dozens of small pages, the
    requests' key ranges are cut into more and more chunks, of four tiles and
    of one, and the requests end one after the other), every position against
    the plain run."""
    from fastgen_amd.kernels import ops

    monkeypatch.setattr(ops, "_SPLIT_MIN_TILES", min_tiles)
    cfg = TINY_C
    weights = sharpen(plain_random_weights(cfg, 7))
    weights = {k: v.to(torch.bfloat16).float() for k, v in weights.items()}
    folder = save_model_folder(tmp_path / "long", cfg, weights)
    prompt = {"a": 20, "b": 35, "c": 7}
    lengths = {"a": 500, "b": 420, "c": 300}
    g = torch.Generator().manual_seed(11)
    tokens = {rid: torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist() for rid, n in lengths.items()}
    trace = [([(rid, 0, n)], []) for rid, n in prompt.items()]
    at = dict(prompt)
    while at:
        trace.append(([(rid, p, 1) for rid, p in at.items()], [rid for rid, p in at.items() if p + 1 == lengths[rid]]))
        at = {rid: p + 1 for rid, p in at.items() if p + 1 < lengths[rid]}
    runner = make_runner(folder, dtype, 16, sum(-(-n // 64) * 64 for n in lengths.values()))
    got = run_trace(runner, trace, tokens)
    assert runner.cache.live_requests() == []
    noise = plain_logits(weights, cfg, tokens, torch.bfloat16) if dtype == torch.bfloat16 else None
    assert_close(got, plain_logits(weights, cfg, tokens), dtype, noise, "long decoding")


def test_float32_does_not_depend_on_the_cut(case):
    """In 32-bit the logits at a position are the same numbers however the
    tokens were cut and batched (every reduction runs in an order fixed by
    the row itself)."""
    a = run_trace(make_runner(case["folder"], torch.float32, case["page"], 1024), traces.whole(case["lengths"]),
                  case["tokens"])
    b = run_trace(make_runner(case["folder"], torch.float32, case["page"], 1024),
                  traces.mixed(case["lengths"], seed=3), case["tokens"])
    for rid in a:
        assert torch.equal(a[rid], b[rid]), rid


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_stale_or_foreign_page_is_never_read(case, dtype):
    """Pages are poisoned with NaN before every step except where the live
    requests hold tokens: what lies beyond a request's length, in free pages
    or in other requests' pages, must not reach its logits."""
    from fastgen_amd.engine import StepEntry

    runner = make_runner(case["folder"], dtype, case["page"], 512)
    for t in runner.storage.k + runner.storage.v:
        t.fill_(float("nan"))
    toks = case["tokens"]
    rid = max(case["lengths"], key=case["lengths"].get)
    n = case["lengths"][rid]
    cut = n // 2
    got = [runner.step([StepEntry(rid, toks[rid][:cut], list(range(cut)))])]
    got.append(runner.step([StepEntry(rid, toks[rid][cut : n - 3], list(range(n - 3 - cut)))]))
    for p in range(n - 3, n):  # and the last tokens one by one (the decode kernels)
        got.append(runner.step([StepEntry(rid, [toks[rid][p]], [0])]).clone())
    got = torch.cat(got).cpu()
    assert torch.isfinite(got).all()
    assert_close({rid: got}, {rid: case["want"][rid]}, dtype, case["noise"] if dtype == torch.bfloat16 else None, "poison")


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_trace_run_program(case, dtype_name, tmp_path):
    """bin/trace_run as a user runs it: JSON lines in, <step>.f32 files and
    ``done`` lines out."""
    dtype = getattr(torch, dtype_name)
    trace = traces.mixed(case["lengths"], seed=5)
    need = traces.max_live_tokens(trace, 64)
    lines, wants = [], []
    for i, (entries, ends) in enumerate(trace):
        ents = []
        for rid, s, n in entries:
            want = list(range(n)) if i % 3 else ([n - 1] if n > 1 else [])  # sometimes only the last, or nothing
            ents.append({"id": rid, "tokens": case["tokens"][rid][s : s + n], "want": want})
            wants += [(i, rid, s + w) for w in want]
        lines.append(json.dumps({"step": i, "entries": ents, "end": ends}))
    out = tmp_path / "out"
    cmd = [sys.executable, str(REPO / "bin" / "trace_run"), "--model", str(case["folder"]), "--dtype", dtype_name,
           "--out", str(out), "--max-tokens", str(need), "--page-size", str(case["page"])]
    proc = subprocess.run(cmd, input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-3000:]
    assert proc.stdout.split() == [x for i in range(len(trace)) for x in ("done", str(i))]
    V = case["cfg"]["vocab_size"]
    # rows that were not asked for keep the plain values, so that the tolerance
    # is that of whole requests as in the other tests
    got = {rid: w.clone() for rid, w in case["want"].items()}
    by_step = {}
    for i, rid, p in wants:
        by_step.setdefault(i, []).append((rid, p))
    for i, items in by_step.items():
        arr = np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, V)
        assert arr.shape[0] == len(items)
        for row, (rid, p) in zip(arr, items):
            got[rid][p] = torch.from_numpy(row.copy())
    for i in range(len(trace)):
        assert (i in by_step) == (out / f"{i}.f32").exists()
    assert_close(got, case["want"], dtype, case["noise"], "trace_run")


def test_unsharpened_model_and_loader_round_trip(tmp_path):
    """The random-weights mode writes a folder that the plain implementation
    reads under checkpoint names; logits agree."""
    from safetensors.torch import load_file

    from fastgen_amd.weights import write_model_folder

    folder = write_model_folder(tmp_path / "m", TINY_B, seed=11)
    cfg = json.load(open(folder / "config.json"))
    weights = load_file(str(folder / "model.safetensors"))
    toks = {"x": list(range(3, 90))}
    want = plain_logits(weights, cfg, toks)
    runner = make_runner(folder, torch.float32, 16, 128)
    got = run_trace(runner, traces.chunks({"x": 87}), toks)
    assert_close(got, want, torch.float32, None, "written folder")


def test_trace_run_with_random_weights_and_more_live_requests(tmp_path):
    """``--random-weights SEED``: a folder with config.json alone (or the file) is enough; the same
    seed gives the same logits however the tokens are cut (bit for bit in 32-bit).  ``--max-live``:
    six requests live at once; a seventh is refused with a message that names the option."""
    cfg = tmp_path / "cfg"
    cfg.mkdir()
    (cfg / "config.json").write_text(json.dumps(TINY_A))
    toks = {f"r{i}": [(7 * i + 3 * j) % 256 for j in range(20 + i)] for i in range(6)}

    def run(lines, out, *more):
        cmd = [sys.executable, str(REPO / "bin" / "trace_run"), "--model", str(cfg), "--dtype", "float32", "--out",
               str(out), "--max-tokens", str(6 * 64), "--page-size", "16", "--random-weights", "5", *more]
        return subprocess.run(cmd, input="\n".join(json.dumps(l) for l in lines) + "\n", capture_output=True,
                              text=True, timeout=600)

    whole = [{"step": 0, "entries": [{"id": r, "tokens": t, "want": [len(t) - 1]} for r, t in toks.items()],
              "end": list(toks)}]
    cut = [{"step": 0, "entries": [{"id": r, "tokens": t[:7], "want": []} for r, t in toks.items()], "end": []},
           {"step": 1, "entries": [{"id": r, "tokens": t[7:], "want": [len(t) - 8]} for r, t in toks.items()],
            "end": list(toks)}]
    p = run(whole, tmp_path / "a", "--max-live", "6")
    assert p.returncode == 0, p.stderr[-2000:]
    p = run(cut, tmp_path / "b", "--max-live", "6")
    assert p.returncode == 0, p.stderr[-2000:]
    a = np.fromfile(tmp_path / "a" / "0.f32", dtype="<f4").reshape(6, 256)
    b = np.fromfile(tmp_path / "b" / "1.f32", dtype="<f4").reshape(6, 256)
    assert np.isfinite(a).all() and np.array_equal(a, b) and np.abs(a).max() > 0
    assert len({tuple(row) for row in a.round(4).tolist()}) == 6  # six requests, six different rows
    p = run(whole, tmp_path / "c", "--model", str(cfg / "config.json"))  # the default: four live requests
    assert p.returncode != 0 and "--max-live is 4" in p.stderr


@pytest.mark.parametrize("n_live,captured", [(24, False), (24, True), (61, False), (61, True)])
def test_many_requests_decode_together_bfloat16(n_live, captured, tmp_path):
    """Dozens of live requests of different lengths, prompts fed in portions, then 45 decode steps
    of all of them together: the split and combine attention kernels with dozens of items, the wide
    products at 17..64 rows, and (captured) the recorded step with a batch filled up to its capacity
    (61 -> 64) by stand-in sequences.  Every position against the plain implementation."""
    cfg = TINY_C
    weights = sharpen(plain_random_weights(cfg, 8))
    weights = {k: v.to(torch.bfloat16).float() for k, v in weights.items()}
    folder = save_model_folder(tmp_path / "many", cfg, weights)
    rng = np.random.default_rng(n_live)
    n_decode = 45
    prompts = {f"r{i}": int(n) for i, n in enumerate(rng.integers(1, 300, n_live))}
    prompts["r0"], prompts["r1"] = 1, 460  # the shortest there is, and one far longer than the others
    g = torch.Generator().manual_seed(12)
    tokens = {rid: torch.randint(0, cfg["vocab_size"], (n + n_decode,), generator=g).tolist()
              for rid, n in prompts.items()}
    trace = traces.many_decoding_together(prompts, n_decode, seed=n_live)
    runner = make_runner(folder, torch.bfloat16, 16, traces.max_live_tokens(trace, 64), max_requests=n_live)
    runner.use_graphs = captured
    got = run_trace(runner, trace, tokens)
    assert runner.cache.live_requests() == []
    assert bool(runner.graphs) == captured
    if captured:
        assert {c for c, _ in runner.graphs} == {24 if n_live == 24 else 64}
    assert_close(got, plain_logits(weights, cfg, tokens), torch.bfloat16,
                 plain_logits(weights, cfg, tokens, torch.bfloat16), f"{n_live} live")


@pytest.mark.parametrize("forced,packed", [("narrow", True), ("narrow", False), ("wide", True), ("wide", False),
                                           ("tiled", True), ("tiled256", False), ("library", True), (None, True),
                                           (None, False)])
def test_every_kernel_that_may_be_chosen_gives_the_plain_logits(forced, packed, tmp_path, monkeypatch):
    """Which kernel takes a matrix product is measured at run time (``fastgen_amd.kernels.linear``), so which
    one an engine test meets depends on the machine.  Here the engine runs once under each kernel's name
    (taken wherever it is among the candidates of a product) and once as measured: whole prompts (up to 150
    rows), mixed steps, and 20 requests decoding together (17..32 rows), every position against the plain
    implementation.  ``packed``: with and without the second copy of the matrices in the streaming kernels'
    order (a model too large for two copies runs without)."""
    from fastgen_amd.kernels import linear

    monkeypatch.setattr(linear, "force", forced)
    monkeypatch.setattr(linear, "choices", {})
    monkeypatch.setenv("FG_PACKED_WEIGHTS", "1" if packed else "0")
    cfg = TINY_B
    weights = sharpen(plain_random_weights(cfg, 9))
    weights = {k: v.to(torch.bfloat16).float() for k, v in weights.items()}
    folder = save_model_folder(tmp_path / "forced", cfg, weights)
    lengths = {"a": 100, "b": 33, "c": 64, "d": 7, "e": 150}
    g = torch.Generator().manual_seed(13)
    tokens = {rid: torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist() for rid, n in lengths.items()}
    want, noise = plain_logits(weights, cfg, tokens), plain_logits(weights, cfg, tokens, torch.bfloat16)
    for name, trace in (("whole", traces.whole(lengths)), ("mixed", traces.mixed(lengths, seed=3))):
        runner = make_runner(folder, torch.bfloat16, 32, traces.max_live_tokens(trace, 64))
        from fastgen_amd.kernels.linear import StreamedMatrix

        held = [v for p in runner.model.parts.all_parts for v in vars(p).values() if isinstance(v, StreamedMatrix)]
        assert len(held) == 4 * cfg["num_hidden_layers"] + 1 and all((m.packed is not None) == packed for m in held)
        got = run_trace(runner, trace, tokens)
        assert_close(got, want, torch.bfloat16, noise, f"forced {forced}, {name}")
    prompts = {f"r{i}": 5 + 3 * i for i in range(20)}
    tokens = {rid: torch.randint(0, cfg["vocab_size"], (n + 12,), generator=g).tolist() for rid, n in prompts.items()}
    trace = traces.many_decoding_together(prompts, 12, seed=1)
    runner = make_runner(folder, torch.bfloat16, 32, traces.max_live_tokens(trace, 64), max_requests=20)
    got = run_trace(runner, trace, tokens)
    assert_close(got, plain_logits(weights, cfg, tokens), torch.bfloat16,
                 plain_logits(weights, cfg, tokens, torch.bfloat16), f"forced {forced}, 20 live")
    if forced is None:
        assert linear.choices and set(linear.choices.values()) <= {"narrow", "wide", "tiled", "tiled256", "library"}
