"""Each part alone against its plain formula, models whose layers differ, run
orders that name a layer twice or share a cache, and a toy mixer with state
of its own that is registered, built and stepped from this file alone."""

import json
from typing import Any, Mapping, Optional

import pytest
import torch

import traces
from helpers import assert_close, run_trace
from plain_llama import (
    plain_attention, plain_rmsnorm, plain_rope_frequencies, plain_rope_interleaved, plain_rope_shuffle, plain_swiglu,
)

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _close(got, want, dtype):
    """float32: rounding of fp32 sums.  bfloat16: operands and results are
    rounded to 8 bits of mantissa, so an element may be off by about 1% of the
    largest element of its tensor."""
    err = float((got.float() - want.float()).abs().max())
    scale = float(want.float().abs().max())
    return err <= (1e-5 if dtype == torch.float32 else 1.5e-2) * scale + 1e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("F", [200, 77])  # 77: not a multiple of the 8 channels the kernels group
def test_norm_feed_forward_embedding_head_alone(dtype, F):
    from fastgen_amd.config import PartSpec
    from fastgen_amd.parts import build_part

    torch.manual_seed(0)
    D, V, T = 72, 131, 9
    norm = build_part("norm", PartSpec("rmsnorm", "n", dict(dim=D, eps=1e-3)))
    w = 1 + 0.1 * torch.randn(D)
    norm.load({"n.weight": w}, dtype, DEV)
    assert norm.weight.dtype == torch.float32  # stored in 32-bit: stays so
    h, delta = torch.randn(T, D), torch.randn(T, D).to(dtype)
    hd = h.to(DEV)
    y = norm.forward(hd, delta.to(DEV), dtype).cpu()
    assert _close(y.float(), plain_rmsnorm(h + delta.float(), w, 1e-3).to(dtype).float(), dtype)
    assert torch.equal(hd.cpu(), h + delta.float())

    ffn = build_part("feed_forward", PartSpec("swiglu", "m", dict(dim=D, hidden_dim=F)))
    ws = {f"m.{k}_proj.weight": torch.randn(*s) * 0.2 for k, s in (("gate", (F, D)), ("up", (F, D)), ("down", (D, F)))}
    ws = {k: v.to(dtype).float() for k, v in ws.items()}
    ffn.load(ws, dtype, DEV)
    x = torch.randn(T, D).to(dtype)
    got = ffn.forward(x.to(DEV)).cpu().float()
    want = plain_swiglu(x.float(), ws["m.gate_proj.weight"], ws["m.up_proj.weight"], ws["m.down_proj.weight"])
    assert _close(got, want, dtype)

    emb = build_part("embedding", PartSpec("embedding", "e", dict(vocab_size=V, dim=D)))
    table = torch.randn(V, D).to(dtype)
    emb.load({"e.weight": table}, dtype, DEV)
    tok = torch.tensor([0, V - 1, 5, 5], dtype=torch.int32)
    assert torch.equal(emb.forward(tok.to(DEV)).cpu(), table[tok.long()].float())

    head = build_part("head", PartSpec("lm_head", "lm_head", dict(vocab_size=V, dim=D, tied_to="e")))
    assert head.tensor_specs() == []
    head.tie(emb.weight)
    logits = head.forward(x.to(DEV))
    assert logits.dtype == torch.float32 and logits.shape == (T, V)
    assert _close(logits.cpu(), x.float() @ table.float().T, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,KV,hd,rot,window", [(6, 2, 32, 32, None), (5, 5, 16, 8, None), (4, 1, 48, 48, 21),
                                               (2, 2, 64, 0, None)])
def test_attention_mixer_alone(dtype, H, KV, hd, rot, window):
    """The mixer with its own cache, two sequences in two steps, against the
    plain attention over whole sequences; rotary_dim < head_dim and no
    rotation at all are other position encodings of the same mixer."""
    from fastgen_amd.cache import CacheManager
    from fastgen_amd.cache.storage import CacheStorage, group_entries
    from fastgen_amd.config import PartSpec
    from fastgen_amd.engine import StepEntry, build_context
    from fastgen_amd.parts import build_part

    torch.manual_seed(1)
    D, P = 40, 16
    pos_spec = PartSpec("rope", options=dict(head_dim=hd, rotary_dim=rot, theta=1000.0)) if rot else PartSpec("none")
    mixer = build_part("mixer", PartSpec("attention", "a", dict(
        dim=D, n_heads=H, n_kv_heads=KV, head_dim=hd, scale=hd**-0.5, window=window, position=pos_spec)))
    ws = {f"a.{k}_proj.weight": (torch.randn(*s) * 0.3).to(dtype).float()
          for k, s in (("q", (H * hd, D)), ("k", (KV * hd, D)), ("v", (KV * hd, D)), ("o", (D, H * hd)))}
    mixer.load(ws, dtype, DEV)
    need = mixer.paged_need()
    assert (need.n_kv_heads, need.head_dim, need.window) == (KV, hd, window)
    groups = group_entries([need])
    cache = CacheManager(P, [16], [window], n_slots=2)
    storage = CacheStorage(groups, [16], P, {}, 2, dtype, DEV)
    store = storage.store_for(0)
    lens = {"x": 45, "y": 20}
    xs = {r: torch.randn(n, D).to(dtype) for r, n in lens.items()}
    outs = {r: [] for r in lens}
    for r in lens:
        cache.admit(r)
    for cuts in ({"x": (0, 30), "y": (0, 1)}, {"x": (30, 45), "y": (1, 20)}):
        entries = [StepEntry(r, [0] * (b - a), []) for r, (a, b) in cuts.items()]
        for e in entries:
            cache.reserve(e.rid, len(e.tokens))
        ctx = build_context(entries, cache, dtype, DEV)
        x = torch.cat([xs[r][a:b] for r, (a, b) in cuts.items()]).to(DEV)
        y = mixer.forward(x, ctx, store).cpu()
        at = 0
        for r, (a, b) in cuts.items():
            outs[r].append(y[at : at + b - a])
            at += b - a
            cache.advance(r, b - a)
    f = plain_rope_frequencies(rot, 1000.0) if rot else None
    for r, n in lens.items():
        x = xs[r].float()
        q = (x @ ws["a.q_proj.weight"].T).view(n, H, hd)
        k = (x @ ws["a.k_proj.weight"].T).view(n, KV, hd)
        v = (x @ ws["a.v_proj.weight"].T).view(n, KV, hd)
        if rot:
            # checkpoint order rotates pairs (i, i + rot/2) of the rotary part
            def rope(t, nh):
                perm = plain_rope_shuffle(torch.eye(nh * rot), nh)  # row permutation as a matrix
                tr = t[..., :rot].reshape(n, nh * rot) @ perm.T
                tr = plain_rope_interleaved(tr.view(n, nh, rot), torch.arange(n), f)
                return torch.cat([tr, t[..., rot:]], -1)
            q, k = rope(q, H), rope(k, KV)
        want = plain_attention(q, k, v, window).reshape(n, H * hd) @ ws["a.o_proj.weight"].T
        assert _close(torch.cat(outs[r]).float(), want, dtype), r


# ------------------------------------------------- layers that differ; order
class _HybridArch:
    """A test-only architecture: per layer its own head counts, window and
    feed-forward width, and a run order given in the configuration."""

    name = "HybridTestModel"

    def parse(self, config: Mapping[str, Any]):
        return dict(config)

    def to_hf_config(self, args):
        return dict(args)

    def layout(self, a):
        from fastgen_amd.config import LayerSpec, ModelLayout, PartSpec, RunEntry

        D = a["dim"]
        norm = lambda p: PartSpec("rmsnorm", p, dict(dim=D, eps=a["eps"]))
        layers = []
        for i, l in enumerate(a["layers"]):
            p = f"blocks.{i}"
            if l["mixer"] == "attention":
                pos = PartSpec(l.get("pos", "rope"), options=dict(head_dim=l["hd"], rotary_dim=l.get("rot", l["hd"]),
                                                                  theta=a["theta"], **l.get("pos_options", {})))
                mixer = PartSpec("attention", f"{p}.attn", dict(dim=D, n_heads=l["H"], n_kv_heads=l["KV"],
                                                               head_dim=l["hd"], scale=l["hd"] ** -0.5,
                                                               window=l.get("window"), position=pos))
            else:
                mixer = PartSpec(l["mixer"], f"{p}.mix", dict(dim=D, decay=l["decay"]))
            ffn = PartSpec(l.get("ffn", "swiglu"), f"{p}.ffn", dict(dim=D, hidden_dim=l["F"], **l.get("ffn_options", {})))
            layers.append(LayerSpec(mixer, ffn, norm(f"{p}.n1"), norm(f"{p}.n2"), l.get("arrangement", "pre_norm"),
                                    {name: norm(f"{p}.{name}") for name in l.get("extra_norms", ())}))
        order = tuple(RunEntry(o[0], o[1]) for o in a["order"])
        return ModelLayout(D, a["vocab"], PartSpec(a.get("embedding", "embedding"), "emb",
                                                   dict(vocab_size=a["vocab"], dim=D, **a.get("embedding_options", {}))),
                           tuple(layers), order, norm("final"),
                           PartSpec("lm_head", "head", dict(vocab_size=a["vocab"], dim=D, tied_to=None)))


def _plain_hybrid(w, a, tokens, mixers, dtype=torch.float32, ffns=None, positions=None):
    """Plain whole-sequence forward of the hybrid model; attention entries
    that read another entry's cache use that entry's rotated k and v.
    ``mixers`` / ``ffns`` / ``positions``: plain functions of the toy parts
    by kind."""
    T = len(tokens)
    w = {k: v.to(dtype) for k, v in w.items()}
    h = w["emb.weight"][torch.tensor(tokens)]
    if a.get("embedding") == "toy_learned_positions":
        h = h + w["emb.positions.weight"][:T]
    kv_of = {}
    for idx, (li, src) in enumerate(a["order"]):
        l, p = a["layers"][li], f"blocks.{li}"
        x = plain_rmsnorm(h, w[f"{p}.n1.weight"], a["eps"])
        if l["mixer"] == "attention":
            H, KV, hd, rot = l["H"], l["KV"], l["hd"], l.get("rot", l["hd"])
            f = plain_rope_frequencies(rot, a["theta"])

            def rope(t, nh):
                if l.get("pos", "rope") != "rope":
                    return positions[l["pos"]](t, l, a)
                perm = plain_rope_shuffle(torch.eye(nh * rot, dtype=dtype), nh)
                tr = t[..., :rot].reshape(T, nh * rot) @ perm.T
                tr = plain_rope_interleaved(tr.view(T, nh, rot), torch.arange(T), f)
                return torch.cat([tr, t[..., rot:]], -1)

            q = rope((x @ w[f"{p}.attn.q_proj.weight"].T).view(T, H, hd), H)
            if src is None:
                k = rope((x @ w[f"{p}.attn.k_proj.weight"].T).view(T, KV, hd), KV)
                v = (x @ w[f"{p}.attn.v_proj.weight"].T).view(T, KV, hd)
                kv_of[idx] = (k, v)
            else:
                k, v = kv_of[src]
            m = plain_attention(q, k, v, l.get("window")).reshape(T, H * hd) @ w[f"{p}.attn.o_proj.weight"].T
        else:
            m = mixers[l["mixer"]](x, w, p, l)
        sandwich = l.get("arrangement") == "toy_sandwich"  # a norm after the mixer and after the feed-forward too
        if sandwich:
            m = plain_rmsnorm(m, w[f"{p}.post_mixer.weight"], a["eps"])
        h = h + m
        x = plain_rmsnorm(h, w[f"{p}.n2.weight"], a["eps"])
        if l.get("ffn", "swiglu") != "swiglu":
            h = h + ffns[l["ffn"]](x, w, p, l)
            continue
        f = plain_swiglu(x, w[f"{p}.ffn.gate_proj.weight"], w[f"{p}.ffn.up_proj.weight"],
                         w[f"{p}.ffn.down_proj.weight"])
        h = h + (plain_rmsnorm(f, w[f"{p}.post_ffn.weight"], a["eps"]) if sandwich else f)
    return (plain_rmsnorm(h, w["final.weight"], a["eps"]) @ w["head.weight"].T).float()


def _hybrid_case(tmp_path, args, seed=3, sharpen=8.0):
    from safetensors.torch import load_file, save_file

    from fastgen_amd.weights import write_model_folder

    folder = write_model_folder(tmp_path / "hybrid", dict(args, architectures=["HybridTestModel"]), seed=seed)
    w = load_file(str(folder / "model.safetensors"))
    w = {k: (v * sharpen if ("q_proj" in k or "k_proj" in k) else v).to(torch.bfloat16).float() for k, v in w.items()}
    save_file(w, str(folder / "model.safetensors"))
    return folder, w


@pytest.fixture
def hybrid_arch():
    from fastgen_amd.config import register_architecture, unregister_architecture

    register_architecture(_HybridArch(), replace=True)
    yield
    unregister_architecture("HybridTestModel")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_layers_differ_and_order_is_data(tmp_path, hybrid_arch, dtype):
    """Three layers with different head counts, head sizes, windows and
    widths; the order runs layer 1 twice and lets the last entry read the
    first entry's cache.  Two cache groups arise (window and no window)."""
    from fastgen_amd.engine import Model, ModelRunner

    args = dict(dim=96, vocab=211, eps=2e-6, theta=5000.0, layers=[
        dict(mixer="attention", H=4, KV=2, hd=16, F=136),
        dict(mixer="attention", H=3, KV=1, hd=32, rot=16, window=24, F=72),
        dict(mixer="attention", H=8, KV=2, hd=16, F=200),
    ], order=[(0, None), (1, None), (1, None), (2, 0)])
    folder, w = _hybrid_case(tmp_path, args)
    model = Model.from_folder(folder, dtype, DEV)
    runner = ModelRunner(model, page_size=16, max_tokens=512, max_requests=4)
    assert len(runner.groups) == 2 and sorted(len(g.entries) for g in runner.groups) == [1, 2]
    lengths = {"a": 70, "b": 33, "c": 5}
    g = torch.Generator().manual_seed(4)
    toks = {r: torch.randint(0, 211, (n,), generator=g).tolist() for r, n in lengths.items()}
    want = {r: _plain_hybrid(w, args, t, {}) for r, t in toks.items()}
    noise = {r: _plain_hybrid(w, args, t, {}, torch.bfloat16) for r, t in toks.items()}
    for tr in (traces.whole(lengths), traces.chunks(lengths), traces.mixed(lengths, seed=2)):
        got = run_trace(runner, tr, toks)
        assert_close(got, want, dtype, noise, "hybrid")
        # the window group gives pages back while the request is still live
    assert runner.cache.free_pages(0) == runner.cache.free_pages(1) == 32


# ------------------------------------------------------ a toy mixer with state
def _register_toy():
    from fastgen_amd.parts import Mixer, StateNeed, TensorSpec, place, register_part

    class ToyEma(Mixer):
        """out_t = W s_t with s_t = decay * s_{t-1} + x_t, s kept per request
        in a state slot of fixed size.  Plain torch on the device: a toy."""

        def __init__(self, spec):
            super().__init__(spec)
            self.dim, self.decay = spec.options["dim"], spec.options["decay"]

        def tensor_specs(self):
            return [TensorSpec(self._name("w.weight"), (self.dim, self.dim))]

        def load(self, tensors, dtype, device):
            self.w = place(tensors[self._name("w.weight")], "matrix", dtype, device)

        def state_need(self):
            return StateNeed((self.dim,), torch.float32)

        def forward(self, x, ctx, store):
            if int(ctx.q_lens.max()) == 1:
                # one token a sequence (the steps that are recorded and replayed): everything that changes
                # from step to step comes from the context's device tensors
                rows = ctx.slot_ids.long()
                s = store.state.index_select(0, rows) * self.decay + x.float()
                store.state.index_copy_(0, rows, s)
                return (s @ self.w.float().T).to(x.dtype)
            out = torch.empty_like(x)
            at = 0
            for b in range(ctx.n_seqs):
                s = store.state[int(ctx.slot_ids_host[b])]
                for t in range(at, at + int(ctx.q_lens[b])):
                    s.mul_(self.decay).add_(x[t].float())
                    out[t] = (self.w.float() @ s).to(x.dtype)
                at += int(ctx.q_lens[b])
            return out

    register_part("mixer", "toy_ema", ToyEma, replace=True)


def _plain_toy(x, w, p, l):
    s, out = torch.zeros(x.shape[1]), []
    for t in range(x.shape[0]):
        s = l["decay"] * s + x[t]
        out.append(w[f"{p}.mix.w.weight"] @ s)
    return torch.stack(out)


def test_toy_mixer_with_state_of_its_own(tmp_path, hybrid_arch):
    from fastgen_amd.engine import Model, ModelRunner, StepEntry
    from fastgen_amd.parts import unregister_part

    _register_toy()
    try:
        args = dict(dim=48, vocab=97, eps=1e-5, theta=100.0, layers=[
            dict(mixer="toy_ema", decay=0.9, F=64),
            dict(mixer="attention", H=3, KV=3, hd=16, F=80),
            dict(mixer="toy_ema", decay=0.5, F=64),
        ], order=[(0, None), (1, None), (2, None)])
        folder, w = _hybrid_case(tmp_path, args)
        model = Model.from_folder(folder, torch.float32, DEV)
        assert sorted(model.state_needs()) == [0, 2]
        runner = ModelRunner(model, page_size=16, max_tokens=256, max_requests=2)
        assert len(runner.groups) == 1 and runner.storage.state[0].shape == (2 + 1, 48)  # and a row that is nobody's
        lengths = {"a": 37, "b": 20, "c": 9}
        g = torch.Generator().manual_seed(5)
        toks = {r: torch.randint(0, 97, (n,), generator=g).tolist() for r, n in lengths.items()}
        want = {r: _plain_hybrid(w, args, t, {"toy_ema": _plain_toy}) for r, t in toks.items()}
        # two live at a time: c takes a slot that a or b left, and finds it cleared
        got = run_trace(runner, traces.mixed(lengths, max_live=2, seed=1), toks)
        assert_close(got, want, torch.float32, None, "toy")
        assert runner.cache.free_slots() == 2
        # state of fixed size does not keep a model from recorded decode steps: three requests decode
        # together from a step recorded for four (the stand-in's state is a row of nobody's), the
        # warm-up before the recording leaves every request's state as it was
        runner = ModelRunner(model, page_size=16, max_tokens=256, max_requests=3)
        runner.graph_capacity = lambda n: 4 if n > 1 else 1
        assert runner.use_graphs
        n_head = {"a": 12, "b": 5, "c": 1}
        trace = [([(r, 0, n)], []) for r, n in n_head.items()]
        trace += [([(r, n_head[r] + s, 1) for r in n_head], []) for s in range(8)]
        trace += [([("a", 20 + s, 1)], []) for s in range(17)]  # a alone: another recorded step
        got = run_trace(runner, trace, toks)
        assert sorted(c for c, _ in runner.graphs) == [1, 4]
        assert_close(got, {"a": want["a"], "b": want["b"][:13], "c": want["c"]}, torch.float32, None, "toy, recorded")
    finally:
        unregister_part("mixer", "toy_ema")


# ------------------------------------- a toy feed-forward with routing, a toy position encoding
def _register_toy_ffn_and_position():
    from fastgen_amd.parts import FeedForward, PositionEncoding, TensorSpec, place, register_part

    class ToyRouted(FeedForward):
        """Each row goes to the expert its router row scores highest (router in
        fp32), weighted by that expert's softmax probability; an expert is a
        SwiGLU of its own.  Plain torch on the device: a toy.  It asks the
        device which rows went where, so its steps cannot be captured."""

        capturable = False

        def __init__(self, spec):
            super().__init__(spec)
            o = spec.options
            self.dim, self.hidden, self.n_experts = o["dim"], o["hidden_dim"], o["n_experts"]

        def tensor_specs(self):
            specs = [TensorSpec(self._name("router.weight"), (self.n_experts, self.dim))]
            for e in range(self.n_experts):
                specs += [TensorSpec(self._name(f"experts.{e}.gate_proj.weight"), (self.hidden, self.dim)),
                          TensorSpec(self._name(f"experts.{e}.up_proj.weight"), (self.hidden, self.dim)),
                          TensorSpec(self._name(f"experts.{e}.down_proj.weight"), (self.dim, self.hidden))]
            return specs

        def load(self, tensors, dtype, device):
            self.router = tensors[self._name("router.weight")].to(device=device, dtype=torch.float32)
            self.experts = [tuple(place(tensors[self._name(f"experts.{e}.{k}_proj.weight")], "matrix", dtype, device)
                                  for k in ("gate", "up", "down")) for e in range(self.n_experts)]

        def forward(self, x):
            probs = torch.softmax(x.float() @ self.router.T, -1)
            weight, choice = probs.max(-1)
            out = torch.zeros_like(x)
            for e, (wg, wu, wd) in enumerate(self.experts):
                rows = (choice == e).nonzero().flatten()
                if rows.numel():
                    xe = x[rows]
                    g = xe @ wg.T
                    y = ((g * torch.sigmoid(g)) * (xe @ wu.T)) @ wd.T
                    out[rows] = (y.float() * weight[rows, None]).to(x.dtype)
            return out

    class ToyLinearRope(PositionEncoding):
        """Rotation of interleaved pairs as stored (no reordering of rows), all
        frequencies divided by a factor."""

        def __init__(self, spec):
            super().__init__(spec)
            o = spec.options
            self.rotary_dim, self.theta, self.factor = int(o["rotary_dim"]), float(o["theta"]), float(o["factor"])

        def frequencies(self):
            return plain_rope_frequencies(self.rotary_dim, self.theta) / self.factor

    register_part("feed_forward", "toy_routed", ToyRouted, replace=True)
    register_part("position", "toy_linear", ToyLinearRope, replace=True)


def _plain_toy_routed(x, w, p, l):
    probs = torch.softmax(x.float() @ w[f"{p}.ffn.router.weight"].float().T, -1)
    weight, choice = probs.max(-1)
    out = torch.zeros_like(x)
    for t in range(x.shape[0]):
        e = int(choice[t])
        y = plain_swiglu(x[t : t + 1], w[f"{p}.ffn.experts.{e}.gate_proj.weight"], w[f"{p}.ffn.experts.{e}.up_proj.weight"],
                         w[f"{p}.ffn.experts.{e}.down_proj.weight"])
        out[t] = y[0] * weight[t]
    return out


def _plain_toy_linear_rope(t, l, a):
    f = plain_rope_frequencies(l["hd"], a["theta"]) / l["pos_options"]["factor"]
    return plain_rope_interleaved(t, torch.arange(t.shape[0]), f)


def test_toy_routed_feed_forward_and_toy_position_encoding(tmp_path, hybrid_arch):
    """A feed-forward that routes rows to experts and a rotary scheme of its
    own, both defined here and registered: built, loaded and stepped without a
    change to the framework, under cuts and batches."""
    from fastgen_amd.engine import Model, ModelRunner
    from fastgen_amd.parts import unregister_part

    _register_toy_ffn_and_position()
    try:
        args = dict(dim=64, vocab=101, eps=1e-5, theta=1000.0, layers=[
            dict(mixer="attention", H=4, KV=2, hd=16, pos="toy_linear", pos_options=dict(factor=4.0), F=40,
                 ffn="toy_routed", ffn_options=dict(n_experts=3)),
            dict(mixer="attention", H=2, KV=1, hd=32, F=96),
        ], order=[(0, None), (1, None)])
        folder, w = _hybrid_case(tmp_path, args, seed=6)
        model = Model.from_folder(folder, torch.float32, DEV)
        runner = ModelRunner(model, page_size=16, max_tokens=512, max_requests=4)
        assert not runner.use_graphs
        lengths = {"a": 45, "b": 18, "c": 3}
        g = torch.Generator().manual_seed(8)
        toks = {r: torch.randint(0, 101, (n,), generator=g).tolist() for r, n in lengths.items()}
        want = {r: _plain_hybrid(w, args, t, {}, ffns={"toy_routed": _plain_toy_routed},
                                 positions={"toy_linear": _plain_toy_linear_rope}) for r, t in toks.items()}
        for tr in (traces.whole(lengths), traces.chunks(lengths), traces.mixed(lengths, seed=5)):
            assert_close(run_trace(runner, tr, toks), want, torch.float32, None, "toy ffn / position")
    finally:
        unregister_part("feed_forward", "toy_routed")
        unregister_part("position", "toy_linear")



# ------------------------------------------------- an arrangement with four norms
def test_toy_arrangement_with_norms_of_its_own(tmp_path, hybrid_arch):
    """A layer may own more norms than the two before its mixer and its feed-forward: a toy
    arrangement, registered here, norms each part's output as well before it joins the residual
    stream.  The layout names the further norms; the builder hands them over by name; their
    tensors are loaded and checked like any other part's."""
    from fastgen_amd.engine import Model, ModelRunner
    from fastgen_amd.parts import register_part, unregister_part

    class Sandwich:
        def __init__(self, mixer, ffn, mixer_norm, ffn_norm, extra):
            self.mixer, self.ffn, self.mixer_norm, self.ffn_norm = mixer, ffn, mixer_norm, ffn_norm
            self.post_mixer, self.post_ffn = extra["post_mixer"], extra["post_ffn"]

        def forward(self, h, pending, ctx, store):
            x = self.mixer_norm.forward(h, pending, ctx.act_dtype)
            mixed = self.mixer.forward(x, ctx, store)
            mixed = self.post_mixer.forward(torch.zeros_like(h), mixed, ctx.act_dtype)  # the norm of 0 + mixed
            x = self.ffn_norm.forward(h, mixed, ctx.act_dtype)
            return self.post_ffn.forward(torch.zeros_like(h), self.ffn.forward(x), ctx.act_dtype)

    register_part("arrangement", "toy_sandwich", lambda spec, *parts: Sandwich(*parts), replace=True)
    try:
        four = dict(arrangement="toy_sandwich", extra_norms=("post_mixer", "post_ffn"))
        args = dict(dim=64, vocab=101, eps=1e-5, theta=1000.0, layers=[
            dict(mixer="attention", H=4, KV=2, hd=16, F=72, **four),
            dict(mixer="attention", H=2, KV=1, hd=32, F=96),  # and a plain pre-norm layer beside it
            dict(mixer="attention", H=4, KV=4, hd=16, F=40, **four),
        ], order=[(0, None), (1, None), (2, None)])
        folder, w = _hybrid_case(tmp_path, args)
        assert "blocks.0.post_mixer.weight" in w and "blocks.1.post_mixer.weight" not in w
        lengths = {"a": 50, "b": 21, "c": 3}
        g = torch.Generator().manual_seed(6)
        toks = {r: torch.randint(0, 101, (n,), generator=g).tolist() for r, n in lengths.items()}
        want = {r: _plain_hybrid(w, args, t, {}) for r, t in toks.items()}
        noise = {r: _plain_hybrid(w, args, t, {}, torch.bfloat16) for r, t in toks.items()}
        for dtype in (torch.float32, torch.bfloat16):
            model = Model.from_folder(folder, dtype, DEV)
            runner = ModelRunner(model, page_size=16, max_tokens=256, max_requests=3)
            for tr in (traces.whole(lengths), traces.tail(lengths, 8), traces.mixed(lengths, max_live=3, seed=4)):
                assert_close(run_trace(runner, tr, toks), want, dtype, noise, "sandwich")
    finally:
        unregister_part("arrangement", "toy_sandwich")


# ------------------------------------------- positions that enter at the embedding
def test_toy_embedding_with_learned_positions(tmp_path, hybrid_arch):
    """A position encoding that is not a rotation inside a mixer: a learned table added to the token
    embedding, by a toy embedding part registered here.  The step's positions reach it through the
    context it is handed; the attention layers use the ``none`` position encoding."""
    from fastgen_amd.engine import Model, ModelRunner
    from fastgen_amd.kernels import ops
    from fastgen_amd.parts import Part, TensorSpec, place, register_part, unregister_part

    class LearnedPositions(Part):
        def __init__(self, spec):
            super().__init__(spec)
            self.vocab, self.dim, self.max_pos = spec.options["vocab_size"], spec.options["dim"], spec.options["max_pos"]

        def tensor_specs(self):
            return [TensorSpec(self._name("weight"), (self.vocab, self.dim)),
                    TensorSpec(self._name("positions.weight"), (self.max_pos, self.dim))]

        def load(self, tensors, dtype, device):
            self.weight = place(tensors[self._name("weight")], "matrix", dtype, device)
            self.positions = place(tensors[self._name("positions.weight")], "matrix", dtype, device)

        def forward(self, tokens, ctx):
            h = torch.empty((tokens.numel(), self.dim), dtype=torch.float32, device=tokens.device)
            ops.embed(self.weight, tokens, h)
            return h.add_(self.positions.index_select(0, ctx.positions.long()).float())  # plain torch: a toy

    register_part("embedding", "toy_learned_positions", LearnedPositions, replace=True)
    try:
        args = dict(dim=64, vocab=101, eps=1e-5, theta=1000.0, embedding="toy_learned_positions",
                    embedding_options=dict(max_pos=80), layers=[
                        dict(mixer="attention", H=4, KV=2, hd=16, pos="none", F=72),
                        dict(mixer="attention", H=2, KV=2, hd=32, pos="none", F=40),
                    ], order=[(0, None), (1, None)])
        folder, w = _hybrid_case(tmp_path, args)
        lengths = {"a": 61, "b": 30, "c": 2}
        g = torch.Generator().manual_seed(9)
        toks = {r: torch.randint(0, 101, (n,), generator=g).tolist() for r, n in lengths.items()}
        ident = lambda t, l, a: t  # no rotation
        want = {r: _plain_hybrid(w, args, t, {}, positions={"none": ident}) for r, t in toks.items()}
        noise = {r: _plain_hybrid(w, args, t, {}, torch.bfloat16, positions={"none": ident}) for r, t in toks.items()}
        # without the table the logits are other logits: the positions matter
        flat = _plain_hybrid({**w, "emb.positions.weight": torch.zeros_like(w["emb.positions.weight"])}, args,
                             toks["a"], {}, positions={"none": ident})
        assert (flat - want["a"]).abs().max() > 0.05 * want["a"].abs().max()
        for dtype in (torch.float32, torch.bfloat16):
            model = Model.from_folder(folder, dtype, DEV)
            runner = ModelRunner(model, page_size=16, max_tokens=256, max_requests=3)
            for tr in (traces.whole(lengths), traces.tail(lengths, 12), traces.mixed(lengths, max_live=3, seed=6)):
                assert_close(run_trace(runner, tr, toks), want, dtype, noise, "learned positions")
    finally:
        unregister_part("embedding", "toy_learned_positions")


def test_cache_pools_for_values_of_another_width():
    """A mixer may ask for values narrower (or wider) than its keys: such a need is a cache group of
    its own, with a value pool of that width, and counts so in the bytes a token takes.  The built-in
    attention kernels take equal widths only and say so."""
    from fastgen_amd.cache.storage import CacheStorage, bytes_per_token, group_entries
    from fastgen_amd.kernels import KernelArgumentError, ops
    from fastgen_amd.parts import PagedNeed

    needs = [PagedNeed(2, 32), PagedNeed(2, 32, None, 16), None, PagedNeed(2, 32, None, 16)]
    groups = group_entries(needs)
    assert [g.entries for g in groups] == [(0,), (1, 3)]
    st = CacheStorage(groups, [6, 5], 16, {}, 2, torch.bfloat16, DEV)
    assert st.k[1].shape == (2, 5, 2, 16, 32) and st.v[1].shape == (2, 5, 2, 16, 16)
    assert st.bytes_per_token() == bytes_per_token(groups, torch.bfloat16) == (2 * 64 + 2 * 2 * 48) * 2
    store = st.store_for(3)
    assert store.group == 1 and store.v_pages.shape == (5, 2, 16, 16)
    q = torch.zeros(1, 2 * 32, dtype=torch.bfloat16, device=DEV)
    i = torch.zeros(1, dtype=torch.int32, device=DEV)
    with pytest.raises(KernelArgumentError):
        ops.paged_attention_general(q, torch.empty_like(q), store.k_pages, store.v_pages, i.view(1, 1), i, i, 2, 1.0)
