"""Generation through the entry points: greedy against the plain
implementation, sampling with seeds, preemption, the reference-style
interface and the command line."""

import json
import os
import queue
import subprocess
import sys
from pathlib import Path

import pytest
import torch

from helpers import save_model_folder
from plain_llama import TINY_A, TINY_B, TINY_C, plain_forward, plain_greedy, plain_random_weights

pytestmark = pytest.mark.gpu
REPO = Path(__file__).resolve().parent.parent


@pytest.fixture(scope="module")
def tiny_b(tmp_path_factory):
    w = plain_random_weights(TINY_B, 1)
    w = {k: v * 8 if ("q_proj" in k or "k_proj" in k or "lm_head" in k) else v for k, v in w.items()}
    folder = save_model_folder(tmp_path_factory.mktemp("genB"), TINY_B, w)
    g = torch.Generator().manual_seed(9)
    prompts = [torch.randint(0, 384, (n,), generator=g).tolist() for n in (1, 12, 40, 90, 150)]
    return dict(folder=folder, weights=w, prompts=prompts)


def test_greedy_generation_matches_the_plain_implementation(tiny_b):
    """Prompts of 1, 12, 40, 90 and 150 tokens, 16
    new tokens each, portions of at most 24 tokens a step beside decodes."""
    from fastgen_amd.engine import Engine
    from fastgen_amd.sampling import SamplingParams

    eng = Engine.from_folder(tiny_b["folder"], torch.float32, page_size=32, max_tokens=1024, max_batch=4,
                             max_step_tokens=24)
    got = eng.generate(tiny_b["prompts"], SamplingParams(temperature=0.0, max_new_tokens=16))
    want = [plain_greedy(tiny_b["weights"], TINY_B, p, 16) for p in tiny_b["prompts"]]
    assert got == want
    assert eng.runner.cache.live_requests() == []
    eng.runner.cache.check()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_decode_batches_between_the_captured_sizes(tiny_b, dtype, monkeypatch):
    """21 requests of different lengths decode together and end one after the
    other: batches of 21, 20, ... run on captured steps of 24 and fewer
    sequences filled up with stand-ins.  float32: each request's tokens are those
    of the plain implementation.  bfloat16: an engine-against-engine check, the
    captured steps against the same engine stepped eagerly (the comparison of this
    path with the plain implementation is
    ``test_gpu_engine.py::test_many_requests_decode_together_bfloat16``)."""
    from fastgen_amd.engine import Engine
    from fastgen_amd.engine.runner import graph_capacity_for
    from fastgen_amd.sampling import SamplingParams

    assert [graph_capacity_for(n) for n in (1, 16, 17, 24, 25, 64, 65, 128, 129)] == [1, 16, 24, 24, 32, 64, 80, 128, 160]
    g = torch.Generator().manual_seed(21)
    prompts = [torch.randint(0, 384, (3 + 2 * i,), generator=g).tolist() for i in range(21)]
    params = [SamplingParams(temperature=0.0, max_new_tokens=4 + i) for i in range(21)]
    eng = Engine.from_folder(tiny_b["folder"], dtype, page_size=16, max_tokens=21 * 96, max_batch=32,
                             max_step_tokens=256)
    got = eng.generate(prompts, params)
    caps = sorted({cap for cap, _ in eng.runner.graphs})  # keys: (sequences, block-table width)
    assert caps and max(caps) == 24 and 17 not in caps and 21 not in caps  # padded, not captured per size
    assert {w for _, w in eng.runner.graphs} == {16}  # short requests: narrow tables, not the pool's 126 pages
    if dtype == torch.float32:
        want = [plain_greedy(tiny_b["weights"], TINY_B, p, sp.max_new_tokens) for p, sp in zip(prompts, params)]
        assert got == want
    else:
        # bfloat16 rounding differs between kernels for few and for many rows: the same engine with
        # the same batches, stepped eagerly, is what the captured steps must reproduce
        monkeypatch.setenv("FG_NO_GRAPHS", "1")
        eager = Engine.from_folder(tiny_b["folder"], dtype, page_size=16, max_tokens=21 * 96, max_batch=32,
                                   max_step_tokens=256)
        assert not eager.runner.use_graphs
        want = eager.generate(prompts, params)
        assert got == want
    assert eng.runner.cache.live_requests() == []
    eng.runner.cache.check()


@pytest.mark.parametrize("seed", [0, 1, 2, 3])
def test_random_serving_load_matches_the_plain_implementation(seed, tmp_path):
    """Requests of random lengths, caps and stop tokens through a small pool
    (so that some are preempted and recomputed) with few slots, prompt portions
    beside decodes, decode runs between host checks: every request's tokens are
    those the plain implementation generates for it alone."""
    import random

    from fastgen_amd.engine import Engine
    from fastgen_amd.sampling import SamplingParams

    rng = random.Random(seed)
    w = plain_random_weights(TINY_A, 5)
    w = {k: v * 8 if ("q_proj" in k or "k_proj" in k or "embed" in k) else v for k, v in w.items()}
    folder = save_model_folder(tmp_path / "load", TINY_A, w)
    g = torch.Generator().manual_seed(seed)
    reqs = []
    for _ in range(22):
        prompt = torch.randint(0, 256, (rng.randint(1, 60),), generator=g).tolist()
        max_new = rng.randint(1, 24)
        alone = plain_greedy(w, TINY_A, prompt, max_new)
        stop = ()
        if rng.random() < 0.4 and len(alone) > 2:
            stop = (alone[rng.randrange(1, len(alone))],)  # a token it will generate: ends there
            alone = alone[: alone.index(stop[0]) + 1]
        reqs.append((prompt, SamplingParams(temperature=0.0, max_new_tokens=max_new, stop_ids=stop), alone))
    eng = Engine.from_folder(folder, torch.float32, page_size=16, max_tokens=176, max_batch=5, max_step_tokens=32,
                             sync_freq=4, admit_reserve=0)
    got = eng.generate([r[0] for r in reqs], [r[1] for r in reqs])
    assert got == [r[2] for r in reqs]
    assert eng.scheduler.n_preemptions > 0
    assert eng.runner.cache.live_requests() == []
    eng.runner.cache.check()


def test_captured_steps_give_way_to_new_ones(tiny_b):
    """With room for two captured steps, batches of four sizes still decode
    from captured steps (the least recently used one gives way) and give the
    tokens of the plain implementation."""
    from fastgen_amd.engine import Engine
    from fastgen_amd.sampling import SamplingParams

    eng = Engine.from_folder(tiny_b["folder"], torch.float32, page_size=32, max_tokens=1024, max_batch=4,
                             max_step_tokens=64, sync_freq=3)
    eng.runner.max_graphs = 2
    prompts = tiny_b["prompts"][:4]
    params = [SamplingParams(temperature=0.0, max_new_tokens=n) for n in (5, 9, 13, 17)]  # batch shrinks 4, 3, 2, 1
    got = eng.generate(prompts, params)
    assert got == [plain_greedy(tiny_b["weights"], TINY_B, p, sp.max_new_tokens) for p, sp in zip(prompts, params)]
    assert len(eng.runner.graphs) == 2 and {cap for cap, _ in eng.runner.graphs} == {1, 2}


def test_preemption_gives_the_same_tokens(tiny_b):
    from fastgen_amd.engine import Engine
    from fastgen_amd.sampling import SamplingParams

    prompts = tiny_b["prompts"][1:4]
    sp = SamplingParams(temperature=0.0, max_new_tokens=40)
    roomy = Engine.from_folder(tiny_b["folder"], torch.float32, page_size=16, max_tokens=1024, max_batch=3,
                               max_step_tokens=64)
    want = roomy.generate(prompts, sp)
    # 12+40+90 prompt tokens and 120 new ones in 15 pages of 16: not all fit at once
    tight = Engine.from_folder(tiny_b["folder"], torch.float32, page_size=16, max_tokens=240, max_batch=3,
                               max_step_tokens=64, admit_reserve=0)
    got = tight.generate(prompts, sp)
    assert tight.scheduler.n_preemptions > 0
    assert got == want
    # with the admission reserve (the default) the third request waits for room instead: nobody gives way
    calm = Engine.from_folder(tiny_b["folder"], torch.float32, page_size=16, max_tokens=240, max_batch=3,
                              max_step_tokens=64)
    assert calm.generate(prompts, sp) == want and calm.scheduler.n_preemptions == 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_temperature_sampling_is_seeded_and_independent_of_the_batch(tiny_b, dtype):
    from fastgen_amd.engine import Engine
    from fastgen_amd.sampling import SamplingParams

    mk = lambda budget, mb: Engine.from_folder(tiny_b["folder"], dtype, page_size=32, max_tokens=1024, max_batch=mb,
                                               max_step_tokens=budget)
    sps = [SamplingParams(temperature=0.8, top_p=0.95, seed=100 + i, max_new_tokens=16) for i in range(5)]
    together = mk(24, 4).generate(tiny_b["prompts"], sps)
    again = mk(24, 4).generate(tiny_b["prompts"], sps)
    assert together == again
    if dtype == torch.float32:
        alone = [mk(512, 1).generate([p], [sp])[0] for p, sp in zip(tiny_b["prompts"], sps)]
        assert together == alone  # neither batch-mates nor the cut of the prompt change a request's draw
    other = mk(24, 4).generate(tiny_b["prompts"], [SamplingParams(temperature=0.8, top_p=0.95, seed=7 + i,
                                                                  max_new_tokens=16) for i in range(5)])
    assert other != together
    greedy = mk(24, 4).generate(tiny_b["prompts"], SamplingParams(temperature=0.0, max_new_tokens=16))
    assert greedy != together


def test_sampled_tokens_follow_the_models_distribution(tiny_b):
    """The first sampled token of one prompt under many seeds against
    softmax(logits / T) of the plain implementation."""
    from fastgen_amd.engine import Engine
    from fastgen_amd.sampling import SamplingParams

    prompt = tiny_b["prompts"][2]
    probs = torch.softmax(plain_forward(tiny_b["weights"], TINY_B, prompt)[-1] / 0.7, -1)
    eng = Engine.from_folder(tiny_b["folder"], torch.float32, page_size=32, max_tokens=64 * 64, max_batch=64,
                             max_step_tokens=4096)
    n = 2048
    counts = torch.zeros(384)
    for s0 in range(0, n, 64):
        outs = eng.generate([prompt] * 64, [SamplingParams(temperature=0.7, seed=1 + s0 + i, max_new_tokens=1)
                                            for i in range(64)])
        for o in outs:
            counts[o[0]] += 1
    big = probs * n >= 5
    chi2 = (((counts - n * probs) ** 2 / (n * probs))[big]).sum()
    assert chi2 < 2.0 * int(big.sum()) + 30, (float(chi2), int(big.sum()))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_decode_runs_give_the_same_tokens_as_single_steps(tiny_b, dtype):
    """sync_freq decode steps between host checks (tokens fed back on the
    device) against one check a step: greedy, seeded sampling, a stop id that
    falls inside a run, and log-probabilities."""
    from fastgen_amd.engine import Engine
    from fastgen_amd.sampling import SamplingParams

    mk = lambda sf: Engine.from_folder(tiny_b["folder"], dtype, page_size=32, max_tokens=1024, max_batch=4,
                                       max_step_tokens=256, sync_freq=sf)
    prompts = tiny_b["prompts"][:4]
    greedy = SamplingParams(temperature=0.0, max_new_tokens=37)
    one, many = mk(1), mk(10)
    want = one.generate(prompts, greedy)
    got = many.generate(prompts, greedy)
    assert got == want
    assert many.n_steps == one.n_steps  # as many model steps, fewer host checks
    if dtype == torch.float32:
        assert want == [plain_greedy(tiny_b["weights"], TINY_B, p, 37) for p in prompts]
    sps = [SamplingParams(temperature=0.9, top_p=0.9, seed=11 + i, max_new_tokens=30, logprobs=True) for i in range(4)]
    assert mk(10).generate(prompts, sps) == mk(1).generate(prompts, sps)
    # a stop id in the middle of a run: the request ends with it
    alone = mk(1).generate([prompts[1]], greedy)[0]
    stop = alone[20]
    sp = SamplingParams(temperature=0.0, max_new_tokens=37, stop_ids=(stop,))
    eng = mk(10)
    rid = eng.add_request(prompts[1], sp)
    done = []
    while eng.has_work():
        done += eng.step()
    assert done[0].generated == alone[: alone.index(stop) + 1] and done[0].finish_reason == "stop"
    assert eng.runner.cache.live_requests() == []
    eng.runner.cache.check()


def test_stop_ids_and_logprobs(tiny_b):
    from fastgen_amd.engine import Engine
    from fastgen_amd.sampling import SamplingParams

    eng = Engine.from_folder(tiny_b["folder"], torch.float32, page_size=32, max_tokens=512, max_batch=2)
    prompt = tiny_b["prompts"][1]
    free = plain_greedy(tiny_b["weights"], TINY_B, prompt, 10)
    rid = eng.add_request(prompt, SamplingParams(max_new_tokens=10, stop_ids=(free[4],), logprobs=True))
    done = []
    while eng.has_work():
        done += eng.step()
    assert done[0].rid == rid and done[0].finish_reason == "stop"
    stop_at = free.index(free[4])
    assert done[0].generated == free[: stop_at + 1]  # ends with the stop token
    toks = prompt + done[0].generated
    lp = torch.log_softmax(plain_forward(tiny_b["weights"], TINY_B, toks), -1)
    want = [float(lp[len(prompt) - 1 + i, t]) for i, t in enumerate(done[0].generated)]
    assert done[0].logprobs == pytest.approx(want, abs=1e-4)


@pytest.mark.parametrize("overlap", [True, False])
def test_single_steps_with_the_host_a_step_behind(tiny_b, overlap):
    """More requests than places, so that steps are single steps: with the host one step behind
    the device (a stop id is seen a step late, log-probabilities arrive a step late) and with every
    step waited for, each request gets the tokens and log-probabilities of the plain implementation."""
    from fastgen_amd.engine import Engine
    from fastgen_amd.sampling import SamplingParams

    eng = Engine.from_folder(tiny_b["folder"], torch.float32, page_size=32, max_tokens=1024, max_batch=2,
                             max_step_tokens=48, overlap_steps=overlap)
    prompts = tiny_b["prompts"][:5]
    want_tokens, params = [], []
    for i, p in enumerate(prompts):
        free = plain_greedy(tiny_b["weights"], TINY_B, p, 9)
        stop = (free[3 + i % 3],) if i % 2 == 0 else ()
        if stop:
            free = free[: free.index(stop[0]) + 1]
        want_tokens.append(free)
        params.append(SamplingParams(max_new_tokens=9, stop_ids=stop, logprobs=True))
    rids = [eng.add_request(p, sp) for p, sp in zip(prompts, params)]
    done = {}
    while eng.has_work():
        for r in eng.step():
            assert r.rid not in done and r.n_pending == 0
            done[r.rid] = r
    assert eng.runner.cache.live_requests() == []
    for rid, p, want in zip(rids, prompts, want_tokens):
        r = done[rid]
        assert r.generated == want and r.finish_reason == ("stop" if len(want) < 9 or want[-1] in r.stop_ids else "length")
        lp = torch.log_softmax(plain_forward(tiny_b["weights"], TINY_B, p + r.generated), -1)
        assert r.logprobs == pytest.approx([float(lp[len(p) - 1 + i, t]) for i, t in enumerate(r.generated)], abs=1e-4)


@pytest.mark.parametrize("dtype,stops", [(torch.bfloat16, False), (torch.float32, True)])
def test_overlap_and_graphs_do_not_change_a_token(dtype, stops, monkeypatch):
    """A load of 120 requests (prompts of 1..700 tokens, greedy and sampled, log-probabilities, few
    places so that requests wait and steps are single steps) gives every request the same tokens,
    end and log-probabilities with steps overlapped or waited for and decode steps captured or
    not.  In float32, where no result depends on the batch, also with stop ids (which an overlapped
    step sees a step late, so that later batches differ); in bfloat16 without them."""
    import random

    from fastgen_amd.engine import Engine
    from fastgen_amd.sampling import SamplingParams

    cfg = dict(TINY_C, hidden_size=512, intermediate_size=1376, num_attention_heads=8, num_key_value_heads=2,
               num_hidden_layers=2, vocab_size=2051, max_position_embeddings=1024)
    rng = random.Random(5)
    n = 120
    plens = [rng.choice([1, 2, 7, 63, 64, 65, 200, 700]) + rng.randint(0, 30) for _ in range(n)]
    olens = [rng.choice([1, 2, 5, 40, 90]) for _ in range(n)]
    g = torch.Generator().manual_seed(0)
    prompts = [torch.randint(0, cfg["vocab_size"], (k,), generator=g).tolist() for k in plens]

    def run(overlap, graphs):
        monkeypatch.setenv("FG_NO_GRAPHS", "0" if graphs else "1")
        eng = Engine.from_config(cfg, seed=3, dtype=dtype, page_size=32, max_tokens=20 * 1100, max_batch=20,
                                 max_step_tokens=300, overlap_steps=overlap, sync_freq=6)
        assert eng.runner.use_graphs == graphs
        for i, (p, o) in enumerate(zip(prompts, olens)):
            eng.add_request(p, SamplingParams(
                temperature=0.0 if i % 3 else 0.8, top_p=0.9, seed=1000 + i, max_new_tokens=o,
                stop_ids=(17, 1042, 2000, 5, 900) if stops and i % 2 == 0 else (), logprobs=(i % 5 == 0)), rid=i)
        out = {}
        while eng.has_work():
            for r in eng.step():
                assert r.rid not in out and r.n_pending == 0
                out[r.rid] = (list(r.generated), r.finish_reason, list(r.logprobs))
        assert eng.runner.cache.live_requests() == []
        eng.runner.cache.check()
        return out

    base = run(False, True)
    assert len(base) == n and all(len(base[i][0]) <= olens[i] for i in base)
    if stops:
        assert any(v[1] == "stop" for v in base.values())
    for overlap, graphs in ((True, True), (True, False), (False, False)):
        assert run(overlap, graphs) == base, (overlap, graphs)


@pytest.mark.parametrize("overlap", [True, False])
def test_abort_in_the_middle_leaves_the_others_alone(tiny_b, overlap):
    """A request is aborted while it decodes (with overlapped steps: while its last sample is still on
    the device), another while it waits: each comes out once, as aborted, with the tokens it had and
    nothing unresolved among them; the others generate what they generate without them (float32: the
    plain implementation's tokens); every page comes back."""
    from fastgen_amd.engine import Engine
    from fastgen_amd.sampling import SamplingParams

    eng = Engine.from_folder(tiny_b["folder"], torch.float32, page_size=32, max_tokens=1024, max_batch=3,
                             max_step_tokens=24, overlap_steps=overlap, sync_freq=1)
    params = SamplingParams(temperature=0.0, max_new_tokens=12)
    rids = [eng.add_request(p, params) for p in tiny_b["prompts"]]  # five requests, three at a time
    ended = {}
    steps = 0
    while eng.has_work():
        for r in eng.step():
            assert r.rid not in ended
            ended[r.rid] = r
        steps += 1
        if steps == 4:
            assert eng.abort(rids[1])      # decoding by now (a prompt of 12 tokens)
            assert eng.abort(rids[4])      # still waiting for a place
            assert not eng.abort("nobody")
    assert sorted(ended) == sorted(rids)
    for i in (1, 4):
        r = ended[rids[i]]
        assert r.finish_reason == "aborted" and r.n_pending == 0 and all(t >= 0 for t in r.generated)
    assert 0 < len(ended[rids[1]].generated) < 12 and ended[rids[4]].generated == []
    assert ended[rids[1]].generated == plain_greedy(tiny_b["weights"], TINY_B, tiny_b["prompts"][1], 12)[: len(ended[rids[1]].generated)]
    for i in (0, 2, 3):
        assert ended[rids[i]].finish_reason == "length"
        assert ended[rids[i]].generated == plain_greedy(tiny_b["weights"], TINY_B, tiny_b["prompts"][i], 12)
    assert eng.runner.cache.live_requests() == []
    eng.runner.cache.check()


def test_reference_style_interface(tiny_b):
    from fastgen_amd.generate import Fastgen, GenArgs, Packet

    fg = Fastgen.build(tiny_b["folder"], GenArgs(use_sampling=False, max_batch=3, max_seq=1024, max_gen=8,
                                                cache_block=32, max_prefill=48, dtype=torch.float32), stop_tokens=())
    q = queue.Queue()
    for i, p in enumerate(tiny_b["prompts"]):
        q.put(Packet(thread_id=f"t{i}", tokens=p, max_gen=5 if i == 0 else None))
    q.put(None)
    out = {pkt.thread_id: pkt.tokens for pkt in fg.generate(q)}
    assert set(out) == {f"t{i}" for i in range(5)}
    for i, p in enumerate(tiny_b["prompts"]):
        assert out[f"t{i}"] == plain_greedy(tiny_b["weights"], TINY_B, p, 5 if i == 0 else 8)
    # one generator serves request after request, as the chat tool uses it (fastgen/tools/chat.py:67-80):
    # every finished request comes out once
    q2: "queue.Queue" = queue.Queue()
    gen = fg.generate(q2)
    for turn in range(3):
        q2.put(Packet(thread_id=turn, tokens=tiny_b["prompts"][2]))
        pkt = next(gen)
        assert pkt.thread_id == turn and pkt.tokens == out["t2"]
    # sizing from a memory budget (fastgen/utils/tune.py:68-84); the reference's way of calling:
    # a loader object and keywords (fastgen/tools/chat.py:50-65)
    from fastgen_amd.generate import HfLoader

    loader = HfLoader(tiny_b["folder"])
    assert loader.load_model_args().n_layers == 3 and loader.load_tokenizer() is None
    with pytest.raises(RuntimeError, match="one GPU"):
        Fastgen.build(loader=loader, gen_args=GenArgs(), tp_mesh=object(), device="cuda:0")
    fg2 = Fastgen.build(loader=loader, gen_args=GenArgs(gpu_gb=0.6, prefill_gb=0.5, dtype=torch.bfloat16),
                        tp_mesh=None, device="cuda:0")
    per_token = 2 * 3 * 32 * 2 * 3
    pool = fg2.engine.runner.cache.n_pages[0] * 64
    assert pool == pytest.approx((0.1e9 - fg2.engine.model.weight_bytes()) / per_token, abs=64)
    assert fg2.engine.scheduler.max_seq == 256  # one request is capped by max_position_embeddings
    # the second copy of the matrices (in the streaming kernels' order) is made where the weights twice leave
    # half of the budget to the cache: with 0.6 GB it is, with a budget of three times the weights it is not
    assert fg2.engine.model.packed()
    one_copy = fg2.engine.model.weight_bytes() / 2
    fg3 = Fastgen.build(loader=loader, gen_args=GenArgs(gpu_gb=3 * one_copy / 1e9, prefill_gb=0,
                                                        dtype=torch.bfloat16), tp_mesh=None, device="cuda:0")
    assert not fg3.engine.model.packed() and fg3.engine.model.weight_bytes() < 1.1 * one_copy


def test_command_line(tiny_b):
    prompt = tiny_b["prompts"][1]
    cmd = [sys.executable, str(REPO / "bin" / "fgchat"), str(tiny_b["folder"]), "--prompt-ids",
           ",".join(map(str, prompt)), "--max-tokens", "6", "--temperature", "0", "--dtype", "float32",
           "--max-seq", "256", "--gpu-gb", "1"]
    proc = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    got = [int(x) for x in proc.stdout.strip().splitlines()[0].split(",")]
    assert got == plain_greedy(tiny_b["weights"], TINY_B, prompt, 6)
    assert "tok/s" in proc.stderr


def test_command_line_with_a_tokenizer(tiny_b, tmp_path):
    """A text prompt through the folder's tokenizer and chat template; and the
    dialogue loop on standard input (a turn, /r, a turn, /q)."""
    import shutil

    from helpers import write_tiny_tokenizer

    from fastgen_amd.tools.tokenizer import FolderTokenizer

    folder = tmp_path / "with_tokenizer"
    shutil.copytree(tiny_b["folder"], folder)
    write_tiny_tokenizer(folder, n_words=380)  # as many words as the model has tokens
    tok = FolderTokenizer(folder)
    base = [sys.executable, str(REPO / "bin" / "fgchat"), str(folder), "--max-tokens", "5", "--temperature", "0",
            "--dtype", "float32", "--max-seq", "256", "--gpu-gb", "1"]
    proc = subprocess.run(base + ["--prompt", "w1 w2 w3"], capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    ids = tok.encode_dialog([{"role": "user", "content": "w1 w2 w3"}])
    want = plain_greedy(tiny_b["weights"], TINY_B, ids, 5)
    stop = tok.stop_tokens[0]
    if stop in want:  # generation ends with the stop token
        want = want[: want.index(stop) + 1]
    lines = proc.stdout.strip().splitlines()
    assert [int(x) for x in lines[0].split(",")] == want
    assert lines[1] == tok.decode([t for t in want if t != stop])
    # the dialogue loop: the first answer is the same generation
    # (the prompts "1> ", "2> " of the rounds stand in front of what follows them on stdout), then a reset to
    # before round 1 and the same message in several lines' form
    import re

    proc = subprocess.run(base, input="w1 w2 w3\n/r 1\n/m\nw1 w2 w3\n.\n/q\n", capture_output=True, text=True,
                          timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    answers = [a for a in (re.sub(r"\d+>+ ", "", l).strip() for l in proc.stdout.splitlines()) if a]
    assert len(answers) == 2 and answers[0] == answers[1] == lines[1]
    assert "1> " in proc.stdout and "1>> " in proc.stdout and "2> " in proc.stdout


def test_smoke_entry():
    sys.path.insert(0, str(REPO))
    import __graft_entry__

    __graft_entry__.smoke()


def test_bench_line():
    """bench.py with one of the 32 layers and a few steps: one JSON line with the fields of its
    contract (value = decoded tokens a second, prefill, roofline, a flat config that names both
    layer counts)."""
    import json

    bench = Path(__file__).resolve().parent.parent / "bench.py"
    r = subprocess.run([sys.executable, str(bench), "--layers", "1", "--steps", "3", "--warmup", "1", "--no-points"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [ln for ln in r.stdout.strip().splitlines() if ln.startswith("{")]
    assert len(lines) == 1
    j = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "prefill", "roofline"):
        assert key in j, key
    assert j["n_gpus"] == 1 and j["steps"] == 3 and j["warmup"] == 1 and j["dtype"] == "bf16" and j["value"] > 0
    assert j["config"]["layers"] == 1 and j["config"]["layers_full"] == 32 and len(j["config"]) <= 20
    assert all(not isinstance(v, (dict, list)) for v in j["config"].values())
    assert set(j["prefill"]) >= {"value", "tokens", "ms", "frac"} and j["prefill"]["tokens"] == 2048
    assert j["prefill"]["repeats"] >= 3 and j["prefill"]["best_ms"] <= j["prefill"]["ms"]
    # the capacity that the line names is the capacity that the cache has
    assert j["config"]["seq_len"] == 8192 and j["config"]["cache_tokens"] == 8 * 8192
    assert j["roofline"]["bound"] == "hbm" and j["roofline"]["peak"] == 8000.0 and 0 < j["roofline"]["frac"] < 1


def test_stop_token_kept_or_dropped_and_seed_zero(tiny_b):
    """``keep_stop_token=False`` reports the request without the stop id that ended it (the
    reference's generator keeps it, its chat tool drops it); seed 0 is a seed like any other."""
    from fastgen_amd.engine import Engine
    from fastgen_amd.sampling import SamplingParams

    eng = Engine.from_folder(tiny_b["folder"], torch.float32, page_size=32, max_tokens=1024, max_batch=4)
    prompt = tiny_b["prompts"][1]
    free = plain_greedy(tiny_b["weights"], TINY_B, prompt, 10)
    stop = free[4]
    cut = free.index(stop)
    for overlap in (True, False):
        eng.overlap_steps = overlap
        kept, dropped = eng.generate([prompt] * 2, [
            SamplingParams(max_new_tokens=10, stop_ids=(stop,), logprobs=True),
            SamplingParams(max_new_tokens=10, stop_ids=(stop,), keep_stop_token=False, logprobs=True)])
        assert kept == free[: cut + 1] and dropped == free[:cut]
    # max_new_tokens reached on the very token that is a stop id: it is dropped all the same
    assert eng.generate([prompt], SamplingParams(max_new_tokens=cut + 1, stop_ids=(stop,), keep_stop_token=False)) \
        == [free[:cut]]
    # seeds: 0 is a seed of its own, None derives one from the engine's seed and the arrival number
    hot = lambda seed: SamplingParams(temperature=1.5, max_new_tokens=12, seed=seed)
    a = eng.generate([prompt], hot(0))
    b = eng.generate([prompt], hot(0))
    c = eng.generate([prompt], hot(None))
    d = eng.generate([prompt], hot(None))
    e = eng.generate([prompt], hot(1))
    assert a == b and c != d and a != e


def test_a_request_that_never_fits_is_refused_or_cut(tiny_b):
    from fastgen_amd.engine import Engine
    from fastgen_amd.sampling import SamplingParams

    eng = Engine.from_folder(tiny_b["folder"], torch.float32, page_size=32, max_tokens=128, max_batch=2)
    prompt = tiny_b["prompts"][3]  # 90 tokens
    with pytest.raises(ValueError, match="can never fit"):
        eng.generate([tiny_b["prompts"][1], prompt], SamplingParams(max_new_tokens=40))
    assert not eng.has_work() and eng.runner.cache.live_requests() == []  # all or nothing
    out = eng.generate([prompt], SamplingParams(max_new_tokens=40, truncate=True))[0]
    assert out == plain_greedy(tiny_b["weights"], TINY_B, prompt, 38)  # 90 + 38 = the 128 tokens of the cache


def test_a_refused_packet_comes_back_and_the_others_go_on(tiny_b):
    from fastgen_amd.generate import Fastgen, GenArgs, Packet

    fg = Fastgen.build(tiny_b["folder"], GenArgs(use_sampling=False, max_batch=3, max_seq=256, max_gen=6,
                                                cache_block=32, dtype=torch.float32), stop_tokens=())
    q = queue.Queue()
    q.put(Packet(thread_id="good0", tokens=tiny_b["prompts"][1]))
    q.put(Packet(thread_id="empty", tokens=[]))
    q.put(Packet(thread_id="alien", tokens=[1, 2, 10**6]))
    q.put(Packet(thread_id="long", tokens=[1] * 300))
    q.put(Packet(thread_id="good1", tokens=tiny_b["prompts"][2]))
    q.put(None)
    out = {p.thread_id: p for p in fg.generate(q)}
    assert set(out) == {"good0", "empty", "alien", "long", "good1"}
    for bad in ("empty", "alien", "long"):
        assert out[bad].tokens == [] and out[bad].error
    assert out["good0"].error is None
    assert out["good0"].tokens == plain_greedy(tiny_b["weights"], TINY_B, tiny_b["prompts"][1], 6)
    assert out["good1"].tokens == plain_greedy(tiny_b["weights"], TINY_B, tiny_b["prompts"][2], 6)
    assert fg.engine.runner.cache.live_requests() == []


def test_cache_sized_to_the_memory_that_is_free(tiny_b):
    """``max_tokens=None``: the cache takes what the device has free beside a reserve, in whole
    pages, and never more than all requests at their longest can use."""
    from fastgen_amd.engine import Engine, Model
    from fastgen_amd.generate import Fastgen, GenArgs

    model = Model.from_folder(tiny_b["folder"], torch.bfloat16, "cuda:0")
    eng = Engine(model, page_size=32, max_tokens=None, max_batch=3)
    assert eng.scheduler.pool_tokens == 3 * 256  # max_position_embeddings 256 a request: no more is ever needed
    del eng
    torch.cuda.empty_cache()
    free = torch.cuda.mem_get_info()[0] + torch.cuda.memory_reserved() - torch.cuda.memory_allocated()
    per_token = 2 * 3 * 32 * 2 * 3  # K and V, 3 kv heads of 32, bfloat16, 3 layers
    reserve = free - 1000 * per_token - 17  # room for 1,000 tokens and a bit
    eng = Engine(model, page_size=32, max_tokens=None, max_batch=64, reserve_bytes=reserve)
    assert eng.scheduler.pool_tokens == 992  # whole pages
    with pytest.raises(RuntimeError, match="no room for one cache page"):
        Engine(model, page_size=32, max_tokens=None, max_batch=64, reserve_bytes=free + (1 << 30))
    fg = Fastgen.from_model(model, GenArgs(gpu_gb=0, max_batch=2, cache_block=32))
    assert fg.engine.scheduler.pool_tokens == 2 * 256
    fg = Fastgen.from_model(model, GenArgs(max_batch=2, cache_block=32), num_pages=5)
    assert fg.engine.scheduler.pool_tokens == 160


def test_command_line_with_random_weights_and_pages(tiny_b, tmp_path):
    """``fgchat --config FILE --random-weights SEED --num-pages N``: no weights on disk; the same
    seed gives the same tokens, another seed other tokens; the cache has the pages asked for."""
    cfg = tmp_path / "config.json"
    cfg.write_text(json.dumps(TINY_B))
    base = [sys.executable, str(REPO / "bin" / "fgchat"), "--config", str(cfg), "--prompt-ids", "5,6,7,8",
            "--max-tokens", "12", "--temperature", "0", "--dtype", "float32", "--page-size", "16", "--verbose"]

    def run(*more):
        proc = subprocess.run(base + list(more), capture_output=True, text=True, timeout=300)
        assert proc.returncode == 0, proc.stderr[-2000:]
        return [int(x) for x in proc.stdout.strip().splitlines()[0].split(",")], proc.stderr

    a, log = run("--random-weights", "3", "--num-pages", "4")
    assert "cache of 64 tokens in pages of 16" in log
    b, _ = run("--random-weights", "3", "--num-pages", "4")
    c, _ = run("--random-weights", "4", "--num-pages", "4")
    assert a == b and a != c and len(a) == 12
    # 2 pages of 16: the prompt's 4 tokens and 28 more fit; the reference's clamp cuts the generation short
    d, _ = run("--random-weights", "3", "--num-pages", "2", "--max-tokens", "100")
    assert len(d) == 28 and d[:12] == a
    proc = subprocess.run(base[:2] + ["--prompt-ids", "1"], capture_output=True, text=True, timeout=60)
    assert proc.returncode == 2 and "--random-weights" in proc.stderr


def test_profile_trace_on_request(tiny_b, tmp_path, monkeypatch):
    """``request_profile()`` (the reference's hook, also bound to SIGUSR2): the next FG_PROFILE_ITERS
    iterations of the generation loop are traced and a chrome trace is written to FG_PROFILE_DIR; the
    generation itself is not disturbed."""
    import gzip
    import signal

    from fastgen_amd.generate import Fastgen, GenArgs, Packet

    monkeypatch.setenv("FG_PROFILE_ITERS", "3")
    monkeypatch.setenv("FG_PROFILE_DIR", str(tmp_path))
    old = signal.getsignal(signal.SIGUSR2)
    try:
        fg = Fastgen.build(tiny_b["folder"], GenArgs(use_sampling=False, max_batch=2, max_seq=512, max_gen=12,
                                                    cache_block=32, dtype=torch.bfloat16, sync_freq=2), stop_tokens=())
        assert fg.trace.n_iters == 3 and not fg.trace.pending and not fg.trace.recording
        from fastgen_amd import generate as generate_module

        if old is signal.SIG_DFL or old is generate_module._on_profile_signal:
            os.kill(os.getpid(), signal.SIGUSR2)  # nobody else handles it: the signal asks the engine built last
        else:
            fg.request_profile()
        assert fg.trace.pending
        q = queue.Queue()
        for i in (1, 2):
            q.put(Packet(thread_id=i, tokens=tiny_b["prompts"][i]))
        q.put(None)
        out = {p.thread_id: p.tokens for p in fg.generate(q)}
        assert len(out[1]) == len(out[2]) == 12
        assert not fg.trace.pending and not fg.trace.recording and fg.trace.last_path is not None
        traces_ = list(tmp_path.glob("fastgen_*.json.gz"))
        assert len(traces_) == 1 and str(traces_[0]) == fg.trace.last_path
        with gzip.open(traces_[0], "rt") as f:
            text = f.read()
        assert "traceEvents" in text and ("gemm_skinny" in text or "attn_" in text)  # the engine's kernels are in it
    finally:
        signal.signal(signal.SIGUSR2, old)
