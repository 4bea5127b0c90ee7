"""The layer sizes of the architecture's real family, with one or two layers and a
smaller vocabulary so that the plain implementation stays fast: the kernels'
production shapes under every way of cutting, in 32-bit and in bfloat16.
Llama 3.1 8B (hidden 4096, 32 heads over 8 kv heads of 128, feed-forward 14336),
Llama 3.2 3B (3072, 24 over 8, 8192, tied head) and Llama 3.1 70B (8192, 64 over
8, 28672): which kernel takes a matrix product depends on its width, so each
width takes its own branches."""

import pytest
import torch

import traces
from helpers import assert_close, make_runner, plain_logits, run_trace, save_model_folder
from plain_llama import plain_forward, plain_random_weights

pytestmark = pytest.mark.gpu

FAMILY = dict(
    architectures=["LlamaForCausalLM"], hidden_size=4096, intermediate_size=14336, num_hidden_layers=2,
    num_attention_heads=32, num_key_value_heads=8, rms_norm_eps=1e-5, vocab_size=32003, rope_theta=500000.0,
    rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=8192),
    tie_word_embeddings=False, max_position_embeddings=131072,
)
FAMILY_3B = dict(FAMILY, hidden_size=3072, intermediate_size=8192, num_attention_heads=24, tie_word_embeddings=True,
                 rope_scaling=dict(FAMILY["rope_scaling"], factor=32.0), vocab_size=16001)
FAMILY_70B = dict(FAMILY, hidden_size=8192, intermediate_size=28672, num_attention_heads=64, num_hidden_layers=1,
                  vocab_size=8003)
SHAPES = {"8b": FAMILY, "3b": FAMILY_3B, "70b": FAMILY_70B}
LENGTHS = {"a": 200, "b": 70, "c": 129, "d": 33}


def _family(tmp_path_factory, name):
    config = SHAPES[name]
    w = plain_random_weights(config, 4)
    # larger q/k projections: attention that is not flat (N(0, 0.02) rows of 4096 give scores near 0)
    w = {k: (v * 4 if ("q_proj" in k or "k_proj" in k) else v).to(torch.bfloat16).float() for k, v in w.items()}
    folder = save_model_folder(tmp_path_factory.mktemp("family" + name), config, w, dtype=torch.bfloat16)
    g = torch.Generator().manual_seed(40)
    tokens = {r: torch.randint(0, config["vocab_size"], (n,), generator=g).tolist() for r, n in LENGTHS.items()}
    # sums over thousands of terms: the float32 runs are judged against a float64 run.  The plain
    # implementation runs its torch operations on the GPU here (it is the same code wherever its tensors
    # are); that run is pinned to the CPU run on one request.
    w_gpu = {k: v.to("cuda:0") for k, v in w.items()}
    exact = {r: plain_forward({k: v.double() for k, v in w_gpu.items()}, config, t, torch.float64).double().cpu()
             for r, t in tokens.items()}
    plain32 = {r: v.cpu() for r, v in plain_logits(w_gpu, config, tokens).items()}
    noise16 = {r: v.cpu() for r, v in plain_logits(w_gpu, config, tokens, torch.bfloat16).items()}
    del w_gpu
    pin = plain_forward(w, config, tokens["d"])
    assert torch.allclose(pin, plain32["d"], atol=1e-4 * float(pin.abs().max()), rtol=0)
    return dict(folder=folder, tokens=tokens, exact=exact, plain32=plain32, noise16=noise16, weights=w, config=config)


@pytest.fixture(scope="module", params=list(SHAPES))
def family(request, tmp_path_factory):
    """One shape's model folder and plain runs (the tests of a shape run one after the other)."""
    return _family(tmp_path_factory, request.param)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_family_shape_under_every_cut(family, dtype):
    for name, trace in (("whole", traces.whole(LENGTHS)), ("tail", traces.tail(LENGTHS, 32)),
                        ("chunks", traces.chunks(LENGTHS)), ("mixed", traces.mixed(LENGTHS, seed=7, budget=96))):
        need = traces.max_live_tokens(trace, 64)
        runner = make_runner(family["folder"], dtype, 64, need)
        got = run_trace(runner, trace, family["tokens"])
        if dtype == torch.float32:
            assert_close(got, family["exact"], dtype, family["plain32"], name)
        else:
            assert_close(got, family["plain32"], dtype, family["noise16"], name)


@pytest.mark.parametrize("n_live", [24, 61, 75, 100])
def test_family_shape_many_requests_decode_together(family, n_live):
    """The benchmark's decode path at its layer sizes: dozens of live requests of different lengths,
    prompts fed in portions, then 40 decode steps of all together, eagerly and from captured steps
    (61 requests in a step recorded for 64, 75 in one for 80, 100 in one for 128): the wide products with k splits at
    17..64 rows and, for o and down, at 65..128 (gate/up with its activation up to 80), the library's q/k/v product with the rotation kernel,
    split attention with dozens of items and both combine kernels.  Every position against the plain implementation, which for this many tokens
    runs its torch operations on the GPU; the fixture pins such a run to the CPU run on one request."""
    import numpy as np

    FAMILY = family["config"]
    if FAMILY["hidden_size"] != 4096 and n_live not in (61, 100):
        pytest.skip("the other widths take the two sizes that cover the wide products and the library's")
    w_gpu = {k: v.to("cuda:0") for k, v in family["weights"].items()}
    rng = np.random.default_rng(n_live)
    n_decode = 40
    prompts = {f"r{i}": int(n) for i, n in enumerate(rng.integers(1, 150, n_live))}
    prompts["r0"], prompts["r1"] = 1, 700
    g = torch.Generator().manual_seed(n_live)
    tokens = {r: torch.randint(0, FAMILY["vocab_size"], (n + n_decode,), generator=g).tolist()
              for r, n in prompts.items()}
    want = {r: plain_forward(w_gpu, FAMILY, t).cpu() for r, t in tokens.items()}
    noise = {r: plain_forward(w_gpu, FAMILY, t, torch.bfloat16).cpu() for r, t in tokens.items()}
    del w_gpu
    trace = traces.many_decoding_together(prompts, n_decode, seed=n_live, budget=256)
    for captured in (False, True):
        runner = make_runner(family["folder"], torch.bfloat16, 64, traces.max_live_tokens(trace, 64),
                             max_requests=n_live)
        runner.use_graphs = captured
        got = run_trace(runner, trace, tokens)
        assert bool(runner.graphs) == captured
        assert_close(got, want, torch.bfloat16, noise, f"{n_live} live, captured={captured}")
        del runner
