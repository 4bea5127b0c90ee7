"""Configuration, registry, layout and weight errors (no GPU)."""

import json

import pytest
import torch

from plain_llama import TINY_A, TINY_B, plain_random_weights, plain_rope_frequencies, plain_rope_shuffle

from fastgen_amd.config import (
    ConfigError, ModelArgs, ModelLayout, PartSpec, RunEntry, LayerSpec, get_architecture, read_config_json,
    registered_architectures,
)
from fastgen_amd.engine.model import build_parts
from fastgen_amd.parts import build_part
from fastgen_amd.weights import (
    DictSource, RandomSource, SafetensorsSource, WeightError, check_against_specs, write_model_folder,
)


def test_typed_config_from_hf_keys():
    a = ModelArgs.from_hf_config(TINY_B)
    assert (a.dim, a.ffn_dim, a.n_layers, a.n_heads, a.n_kv_heads, a.head_dim) == (192, 512, 3, 6, 3, 32)
    assert (a.norm_eps, a.vocab_size, a.tie_embeddings, a.max_position) == (1e-5, 384, False, 256)
    assert a.rope.scaled and (a.rope.theta, a.rope.factor, a.rope.original_context) == (500000.0, 8.0, 64)
    b = ModelArgs.from_hf_config(TINY_A)
    assert not b.rope.scaled and b.tie_embeddings and b.head_dim == 16
    # kv heads default to the heads (fastgen/utils/loading.py:64-67)
    c = ModelArgs.from_hf_config({k: v for k, v in TINY_A.items() if k != "num_key_value_heads"})
    assert c.n_kv_heads == c.n_heads
    # round trip through config.json keys
    assert ModelArgs.from_hf_config(a.to_hf_config()) == a


@pytest.mark.parametrize("key", ["hidden_size", "intermediate_size", "num_hidden_layers", "num_attention_heads",
                                 "rms_norm_eps", "vocab_size", "rope_theta"])
def test_missing_key_is_named(key):
    cfg = {k: v for k, v in TINY_B.items() if k != key}
    with pytest.raises(ConfigError, match=key):
        ModelArgs.from_hf_config(cfg)


def test_config_refusals():
    with pytest.raises(ConfigError, match="rope_type"):
        ModelArgs.from_hf_config(dict(TINY_B, rope_scaling=dict(TINY_B["rope_scaling"], rope_type="yarn")))
    with pytest.raises(ConfigError, match="low_freq_factor"):
        sc = {k: v for k, v in TINY_B["rope_scaling"].items() if k != "low_freq_factor"}
        ModelArgs.from_hf_config(dict(TINY_B, rope_scaling=sc))
    with pytest.raises(ConfigError, match="head_dim"):
        ModelArgs.from_hf_config(dict(TINY_B, head_dim=64))
    with pytest.raises(ConfigError, match="multiple"):
        ModelArgs.from_hf_config(dict(TINY_B, num_key_value_heads=4))
    with pytest.raises(ConfigError, match="attention_bias"):
        ModelArgs.from_hf_config(dict(TINY_B, attention_bias=True))


def test_registry():
    assert "LlamaForCausalLM" in registered_architectures()
    assert get_architecture(TINY_A).name == "LlamaForCausalLM"
    with pytest.raises(ConfigError, match="Unsupported model type 'GPT2LMHeadModel'"):
        get_architecture({"architectures": ["GPT2LMHeadModel"]})


def test_layout_is_data():
    arch = get_architecture(TINY_B)
    lay = arch.layout(arch.parse(TINY_B))
    assert len(lay.layers) == 3 and [e.layer for e in lay.order] == [0, 1, 2]
    assert lay.layers[1].mixer.kind == "attention" and lay.layers[1].ffn.kind == "swiglu"
    assert lay.layers[2].mixer.options["n_kv_heads"] == 3 and lay.layers[0].ffn.options["hidden_dim"] == 512
    assert lay.head.options["tied_to"] is None
    # the order may name a layer twice and let an entry read an earlier entry's cache
    twice = ModelLayout(lay.dim, lay.vocab_size, lay.embed, lay.layers,
                        (RunEntry(0), RunEntry(1), RunEntry(1), RunEntry(2, reads_cache_of=0)), lay.final_norm, lay.head)
    assert len(twice.order) == 4
    with pytest.raises(ValueError, match="does not run before"):
        ModelLayout(lay.dim, lay.vocab_size, lay.embed, lay.layers, (RunEntry(0, reads_cache_of=1), RunEntry(1)),
                    lay.final_norm, lay.head)
    with pytest.raises(ValueError, match="does not exist"):
        ModelLayout(lay.dim, lay.vocab_size, lay.embed, lay.layers, (RunEntry(7),), lay.final_norm, lay.head)
    with pytest.raises(KeyError, match="no mixer of kind 'nonesuch'"):
        build_part("mixer", PartSpec("nonesuch"))


def test_rope_part_matches_the_plain_formulas():
    arch = get_architecture(TINY_B)
    lay = arch.layout(arch.parse(TINY_B))
    rope = build_part("position", lay.layers[0].mixer.options["position"])
    assert torch.equal(rope.frequencies(), plain_rope_frequencies(32, 500000.0, TINY_B["rope_scaling"]))
    w = torch.randn(6 * 32, 20)
    assert torch.equal(rope.arrange_rows(w, 6), plain_rope_shuffle(w, 6))
    # a partial rotation permutes the rotary part of each head only
    part = build_part("position", PartSpec("rope", options=dict(head_dim=8, rotary_dim=4, theta=100.0)))
    rows = torch.arange(16.0)[:, None]
    assert part.arrange_rows(rows, 2)[:, 0].tolist() == [0, 2, 1, 3, 4, 5, 6, 7, 8, 10, 9, 11, 12, 13, 14, 15]
    assert part.frequencies().tolist() == pytest.approx([1.0, 0.1])


def _specs(cfg):
    arch = get_architecture(cfg)
    return build_parts(arch.layout(arch.parse(cfg))).tensor_specs()


def test_tensor_names_are_the_checkpoint_names():
    for cfg in (TINY_A, TINY_B):
        names = {s.name: s.shape for s in _specs(cfg)}
        plain = plain_random_weights(cfg, 0)
        assert names == {k: tuple(v.shape) for k, v in plain.items()}


def test_one_error_lists_everything_wrong():
    w = plain_random_weights(TINY_B, 0)
    del w["model.layers.1.mlp.up_proj.weight"], w["model.norm.weight"]
    w["model.layers.0.self_attn.q_proj.bias"] = torch.zeros(192)
    w["model.layers.2.self_attn.k_proj.weight"] = torch.zeros(96, 100)
    with pytest.raises(WeightError) as e:
        check_against_specs(DictSource(w), _specs(TINY_B))
    msg = str(e.value)
    assert "missing tensors (2): model.layers.1.mlp.up_proj.weight, model.norm.weight" in msg
    assert "unexpected tensors (1): model.layers.0.self_attn.q_proj.bias" in msg
    assert "model.layers.2.self_attn.k_proj.weight is [96, 100], expected [96, 192]" in msg


def test_tied_head_in_the_file():
    w = plain_random_weights(TINY_A, 0)
    specs = _specs(TINY_A)
    arch = get_architecture(TINY_A)
    dup = build_parts(arch.layout(arch.parse(TINY_A))).duplicates()
    w["lm_head.weight"] = w["model.embed_tokens.weight"].clone()
    check_against_specs(DictSource(w), specs, dup)  # an equal copy is tolerated
    w["lm_head.weight"] = w["lm_head.weight"] + 1
    with pytest.raises(WeightError, match="unexpected tensors .*lm_head.weight"):
        check_against_specs(DictSource(w), specs, dup)


def test_random_weights_folder(tmp_path):
    from safetensors.torch import load_file, save_file

    folder = write_model_folder(tmp_path / "m", TINY_B, seed=5)
    cfg = read_config_json(folder)
    assert ModelArgs.from_hf_config(cfg) == ModelArgs.from_hf_config(TINY_B)
    src = SafetensorsSource(folder)
    check_against_specs(src, _specs(TINY_B))
    t = load_file(str(folder / "model.safetensors"))
    assert t["model.layers.0.mlp.down_proj.weight"].dtype == torch.float32
    assert abs(float(t["model.embed_tokens.weight"].std()) - 0.02) < 2e-3
    assert abs(float(t["model.norm.weight"].mean()) - 1) < 5e-3 and float(t["model.norm.weight"].std()) < 0.02
    # the same seed gives the same tensors, another seed others; a tensor does not depend on the rest
    again = write_model_folder(tmp_path / "m2", TINY_B, seed=5)
    other = write_model_folder(tmp_path / "m3", TINY_B, seed=6)
    t2, t3 = load_file(str(again / "model.safetensors")), load_file(str(other / "model.safetensors"))
    assert all(torch.equal(t[k], t2[k]) for k in t) and not torch.equal(t["lm_head.weight"], t3["lm_head.weight"])
    one = RandomSource([s for s in _specs(TINY_B) if s.name == "lm_head.weight"], 5)
    assert torch.equal(one.get("lm_head.weight"), t["lm_head.weight"])
    bf = write_model_folder(tmp_path / "m4", TINY_A, seed=5, dtype=torch.bfloat16)
    assert load_file(str(bf / "model.safetensors"))["model.norm.weight"].dtype == torch.bfloat16
    # sharded folders with an index are read by name too
    sh = tmp_path / "sharded"
    sh.mkdir()
    keys = sorted(t)
    save_file({k: t[k] for k in keys[::2]}, str(sh / "model-00001-of-00002.safetensors"))
    save_file({k: t[k] for k in keys[1::2]}, str(sh / "model-00002-of-00002.safetensors"))
    json.dump({"weight_map": {k: f"model-0000{1 + i % 2}-of-00002.safetensors" for i, k in enumerate(keys)}},
              open(sh / "model.safetensors.index.json", "w"))
    s2 = SafetensorsSource(sh)
    assert sorted(s2.names()) == keys and torch.equal(s2.get(keys[3]), t[keys[3]])
    (sh / "model.safetensors.index.json").unlink()
    assert sorted(SafetensorsSource(sh).names()) == keys
    with pytest.raises(WeightError, match="no model.safetensors"):
        SafetensorsSource(tmp_path)
    with pytest.raises(ConfigError, match="not a model folder"):
        read_config_json(tmp_path)


def test_sizes_the_kernels_cannot_take_are_refused_when_the_model_is_built():
    arch = get_architecture(TINY_A)
    bad_head = dict(TINY_A, hidden_size=80, num_attention_heads=4, num_key_value_heads=2)  # head size 20
    with pytest.raises(ValueError, match="head size 20 is not supported"):
        build_parts(arch.layout(arch.parse(bad_head)))


def test_dtype_policy():
    from fastgen_amd.parts import MATRIX, VECTOR, TABLE_INT, place

    m32, m16 = torch.randn(4, 4), torch.randn(4, 4).bfloat16()
    assert place(m32, MATRIX, torch.bfloat16, "cpu").dtype == torch.bfloat16
    assert place(m16, MATRIX, torch.float32, "cpu").dtype == torch.float32
    assert place(torch.randn(4), VECTOR, torch.bfloat16, "cpu").dtype == torch.float32  # stored in 32-bit: stays
    assert place(torch.randn(4).bfloat16(), VECTOR, torch.bfloat16, "cpu").dtype == torch.bfloat16
    assert place(torch.arange(4), TABLE_INT, torch.bfloat16, "cpu").dtype == torch.int32


def test_second_copy_of_the_matrices_is_a_matter_of_memory(monkeypatch):
    """``packing_fits``: the switch wins; without it nothing is packed off the GPU.  ``streamed`` packs only
    while a model says so (``packing``), and only bfloat16 matrices on the GPU: the 32-bit path and a part
    that hands ``linear`` a plain tensor keep one copy."""
    from fastgen_amd.kernels import linear

    monkeypatch.delenv("FG_PACKED_WEIGHTS", raising=False)
    assert linear.packing_fits(1 << 30, "cpu") is False
    import torch

    monkeypatch.setattr(torch.cuda, "get_device_properties", lambda dev: type("P", (), {"total_memory": 288 << 30})())
    assert linear.packing_fits(16 << 30, "cuda:0") is True  # 8B: 32 of 288 GB
    assert linear.packing_fits(141 << 30, "cuda:0") is False  # 70B: one copy
    assert linear.packing_fits(16 << 30, "cuda:0", budget_bytes=int(20e9)) is False  # a budget of 20 GB for both
    assert linear.packing_fits(1 << 30, "cuda:0", budget_bytes=int(20e9)) is True
    monkeypatch.setenv("FG_PACKED_WEIGHTS", "1")
    assert linear.packing_fits(1 << 50, "cpu") is True
    monkeypatch.setenv("FG_PACKED_WEIGHTS", "0")
    assert linear.packing_fits(1, "cpu") is False
    w = torch.randn(48, 64).to(torch.bfloat16)
    with linear.packing(True):
        m = linear.streamed(w)  # on the CPU: one copy
        assert m.packed is None and m.streaming is w and m.shape == w.shape and m.dtype == w.dtype
    assert linear._pack_now is False
    m = linear.StreamedMatrix(w, ops_pack(w))
    assert m.streaming is m.packed and m.nbytes() == 2 * w.numel() * 2
    cut = m.first_rows(32)
    assert cut.rows.shape == (32, 64) and cut.packed is not None and cut.packed.shape == (32, 64)
    assert m.first_rows(20).packed is None  # no multiple of 16: the rows alone


def ops_pack(w):
    from fastgen_amd.kernels import ops

    return ops.pack_weight(w)


def test_bench_refuses_more_than_one_gpu():
    """bench.py runs on one GPU: for more it says so in one line and exits with 2."""
    import subprocess
    import sys
    from pathlib import Path

    bench = Path(__file__).resolve().parent.parent / "bench.py"
    r = subprocess.run([sys.executable, str(bench), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 2
    assert len(r.stdout.strip().splitlines()) == 1 and "one GPU" in r.stdout


def test_folder_tokenizer(tmp_path):
    """tokenizer.json and the chat template of tokenizer_config.json
    (fastgen/utils/tokenizer.py:48-118)."""
    from helpers import write_tiny_tokenizer

    from fastgen_amd.tools.tokenizer import FolderTokenizer

    assert FolderTokenizer.maybe(tmp_path) is None
    words = write_tiny_tokenizer(tmp_path)
    tok = FolderTokenizer.maybe(tmp_path)
    assert tok.stop_tokens == [words.index("<end>")]
    ids = tok.encode("w3 w0 w39")
    assert ids == [words.index(w) for w in ("w3", "w0", "w39")]
    assert tok.decode(ids) == "w3 w0 w39"
    dialog = [{"role": "user", "content": "w1 w2"}, {"role": "assistant", "content": "w5"}, {"role": "user", "content": "w7"}]
    want = "<user> w1 w2 <end> <bot> w5 <end> <user> w7 <end> <bot>".split()
    assert tok.encode_dialog(dialog) == [words.index(w) for w in want]



def test_trace_window_counts_iterations(tmp_path):
    """A trace on request covers the next ``n_iters`` iterations of the loop that ticks it, is written
    once, and a second request while one waits or runs is ignored."""
    from fastgen_amd.engine.trace_window import TraceWindow

    w = TraceWindow(2, str(tmp_path), prefix="t")
    w.tick()
    assert not w.pending and not w.recording and w.last_path is None
    w.request()
    w.request()
    assert w.pending and not w.recording
    w.tick()  # iteration 1 begins
    assert w.recording and not w.pending
    w.request()  # ignored: one is running
    assert not w.pending
    w.tick()  # iteration 2 begins
    assert w.recording
    w.tick()  # both are over
    assert not w.recording and w.last_path is not None
    assert [p.name for p in tmp_path.iterdir()] == [w.last_path.rsplit("/", 1)[1]]
    w.request()
    w.tick()
    w.close(write=False)  # a loop that ends early and wants no file
    assert not w.recording and len(list(tmp_path.iterdir())) == 1


def test_chat_dialogue_commands():
    """The dialogue loop's commands as in ``fastgen/tools/chat.py:161-195``: ``/r <N>`` resets the
    conversation to before round N, ``/m`` takes a message of several lines, ``/q`` quits."""
    from fastgen_amd.tools.chat import dialogue_loop

    class Tok:
        stop_tokens = (99,)

        def encode_dialog(self, dialog):
            return [len(dialog)] + [len(m["content"]) for m in dialog]

        def decode(self, ids):
            return "answer to " + ",".join(map(str, ids))

    seen, said = [], []
    script = iter(["hello", "more", "/r 2", "again", "/m", "line one", "line two", ".", "/r x", "/r", "last", "/q", "never"])
    prompts = []

    def read(prompt):
        prompts.append(prompt)
        return next(script)

    def run(tokens):
        seen.append(list(tokens))
        return [len(seen), 99]  # ends on a stop token, which is dropped from the text

    assert dialogue_loop(Tok(), run, read, said.append) == 0
    # round 1, round 2, back to before round 2, round 2 again, round 3 of two lines, a bad command,
    # /r alone drops round 3, round 3 again
    assert [t[0] for t in seen] == [1, 3, 3, 5, 5]
    assert seen[3][-1] == len("line one\nline two") and seen[2][-1] == len("again")
    assert said == ["answer to 1", "answer to 2", "answer to 3", "answer to 4", "answer to 5"]
    assert prompts[:3] == ["1> ", "2> ", "3> "] and "3>> " in prompts and prompts[-1] == "4> "
