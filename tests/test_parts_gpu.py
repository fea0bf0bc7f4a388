"""Each kind of part alone against the plain function it implements, at sizes of its own; a model put together from
parts in an unusual order (a layer run twice, an entry that reads another entry's cache); and a toy mixer with state of
its own, a toy feed-forward with routing, a toy position encoding and a toy norm that are defined here, registered, built
and stepped without touching the framework."""

from __future__ import annotations

from dataclasses import dataclass
from typing import ClassVar

import pytest
import torch

import plain_llama as pl
from tiny import ulps_of_row_max

pytestmark = pytest.mark.gpu
DEV = "cuda"


LLAMA_NAMES = dict(mixer_norm_name="input_layernorm.weight", ffn_norm_name="post_attention_layernorm.weight")


def llama_block(prefix, norm1, mixer, norm2, ffn):
    """A pre-norm block whose norms, attention and SwiGLU carry the Llama checkpoints' names; toy parts get their kind."""
    from nanospec_amd.config.spec import PreNormBlockSpec

    return PreNormBlockSpec(prefix, norm1, mixer, norm2, ffn, **LLAMA_NAMES,
                            mixer_prefix="self_attn." if mixer.kind == "attention" else None,
                            ffn_prefix="mlp." if ffn.kind == "swiglu" else None)


def make_ctx(lens, starts, tables, page, dtype, want=()):
    """A StepContext for hand-made requests: tables[b] lists the pages of request b."""
    import numpy as np

    from nanospec_amd.engine.arena import Arena
    from nanospec_amd.engine.context import BatchLayout, StepContext, fill_batch
    from nanospec_amd.parts.attention import TILES

    width = max(len(t) for t in tables)
    layout = BatchLayout(sum(lens), len(lens), len(want), 1, width, plans=[(TILES, TILES.shape(lens))])
    host = np.zeros(layout.total, dtype=np.int32)
    table = np.full((len(lens), width), -1, dtype=np.int32)
    for b, t in enumerate(tables):
        table[b, : len(t)] = t
    fill_batch(host, layout, [0] * sum(lens), starts, lens, list(range(len(lens))), list(want), [table])
    dev = torch.from_numpy(host).to(DEV)
    max_kv = max(s + n for s, n in zip(starts, lens))
    return StepContext(layout, dev, Arena(DEV), max_position=max_kv - 1, max_kv_len=max_kv)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_norm_part(dtype):
    from nanospec_amd.config.spec import RMSNormSpec
    from nanospec_amd.parts import build

    torch.manual_seed(0)
    part = build("norm", RMSNormSpec(dim=88, eps=2e-6), "x.norm.weight")
    assert part.wanted() == {"x.norm.weight": ((88,), "norm")}
    w = 1 + 0.1 * torch.randn(88)
    part.load({"x.norm.weight": w}.__getitem__, dtype, DEV)
    x = torch.randn(5, 88).to(dtype)
    got = part.forward(None, resid=x.to(DEV))
    tol = dict(rtol=1e-5, atol=1e-6) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(got.cpu().float(), pl.rms_norm(x, w.to(dtype), 2e-6).float(), **tol)


def test_rope_part_frequencies():
    from nanospec_amd.config.spec import RopeSpec
    from nanospec_amd.parts import build

    for scaling in (None, (8.0, 1.0, 4.0, 64), (32.0, 1.0, 4.0, 8192)):
        part = build("position", RopeSpec(rotary_dim=48, theta=5e5, scaling=scaling, max_positions=512), "")
        part.load(None, torch.float32, DEV)
        s = None if scaling is None else dict(factor=scaling[0], low_freq_factor=scaling[1], high_freq_factor=scaling[2],
                                              original_max_position_embeddings=scaling[3])
        assert torch.equal(part.inv_freq.cpu(), pl.inverse_frequencies(48, 5e5, s))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_feed_forward_part(dtype):
    from nanospec_amd.config.spec import SwiGLUSpec
    from nanospec_amd.parts import build

    torch.manual_seed(1)
    part = build("ffn", SwiGLUSpec(hidden=72, intermediate=200), "l.mlp.")
    ws = {"l.mlp.gate_proj.weight": torch.randn(200, 72) * 0.1, "l.mlp.up_proj.weight": torch.randn(200, 72) * 0.1,
          "l.mlp.down_proj.weight": torch.randn(72, 200) * 0.1}
    assert {k: v[0] for k, v in part.wanted().items()} == {k: tuple(v.shape) for k, v in ws.items()}
    part.load(ws.__getitem__, dtype, DEV)
    for rows in (3, 70):  # the streaming kernel and the many-row path
        x = torch.randn(rows, 72).to(dtype)
        ctx = make_ctx([rows], [0], [[0] * 8], 16, dtype)
        got = part.forward(ctx, x.to(DEV))
        ref = pl.swiglu(x, *(ws[k].to(dtype) for k in ws))
        if dtype == torch.float32:
            torch.testing.assert_close(got.cpu(), ref, rtol=1e-4, atol=1e-5)
        else:
            assert ulps_of_row_max(got.cpu(), ref).max() <= 4


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("window", [0, 9])
def test_attention_part_with_cache_across_steps(dtype, window):
    """The mixer alone: two requests, the first step writes a portion, the second appends a portion to one and a single
    token to the other; against plain projections + rotation + attention over the whole sequences."""
    import math

    from nanospec_amd.cache.storage import PagedView
    from nanospec_amd.config.spec import AttentionSpec, RopeSpec
    from nanospec_amd.parts import build

    torch.manual_seed(2)
    hidden, heads, kvh, hd, page = 80, 6, 2, 32, 8
    spec = AttentionSpec(hidden=hidden, heads=heads, kv_heads=kvh, head_dim=hd, position=RopeSpec(rotary_dim=hd, theta=1e4),
                         softmax_scale=1 / math.sqrt(hd), window=window)
    part = build("mixer", spec, "a.")
    ws = {"a.q_proj.weight": torch.randn(heads * hd, hidden) * 0.2, "a.k_proj.weight": torch.randn(kvh * hd, hidden) * 0.2,
          "a.v_proj.weight": torch.randn(kvh * hd, hidden) * 0.2, "a.o_proj.weight": torch.randn(hidden, heads * hd) * 0.2}
    part.load(ws.__getitem__, dtype, DEV)
    need = part.cache_need()
    assert (need.kv_heads, need.head_dim, need.window) == (kvh, hd, window)
    k = torch.zeros(12, kvh, page, hd, dtype=dtype, device=DEV)
    v = torch.zeros(12, kvh, hd, page, dtype=dtype, device=DEV)
    cache = PagedView(0, k, v)
    xs = [torch.randn(21, hidden).to(dtype), torch.randn(14, hidden).to(dtype)]
    tables = [[7, 2, 9], [4, 11]]

    def plain(x):
        t = x.shape[0]
        q = pl.linear(x, ws["a.q_proj.weight"].to(dtype)).view(t, heads, hd)
        kk = pl.linear(x, ws["a.k_proj.weight"].to(dtype)).view(t, kvh, hd)
        vv = pl.linear(x, ws["a.v_proj.weight"].to(dtype)).view(t, kvh, hd)
        cos, sin = pl.rotation_tables(torch.arange(t), pl.inverse_frequencies(hd, 1e4, None))
        q, kk = pl.rotate(q, cos, sin), pl.rotate(kk, cos, sin)
        if window:
            a = torch.cat([pl.causal_attention(q[i : i + 1], kk[max(0, i - window + 1) : i + 1], vv[max(0, i - window + 1) : i + 1],
                                               first_query=min(i, window - 1)) for i in range(t)])
        else:
            a = pl.causal_attention(q, kk, vv)
        return pl.linear(a.reshape(t, -1), ws["a.o_proj.weight"].to(dtype))

    refs = [plain(x) for x in xs]
    steps = [([17, 13], [0, 0]), ([4, 1], [17, 13])]
    for lens, starts in steps:
        ctx = make_ctx(lens, starts, tables, page, dtype)
        x = torch.cat([xs[b][s : s + n] for b, (s, n) in enumerate(zip(starts, lens))]).to(DEV)
        got = part.forward(ctx, x, cache, True).cpu()
        ref = torch.cat([refs[b][s : s + n] for b, (s, n) in enumerate(zip(starts, lens))])
        if dtype == torch.float32:
            torch.testing.assert_close(got, ref, rtol=1e-4, atol=1e-4)
        else:
            assert ulps_of_row_max(got, ref).max() <= 6


# ------------------------------------------------------------------------------------------------ a toy mixer with state


@dataclass(frozen=True)
class PrefixMeanSpec:
    """out_t = W . mean(x_0 .. x_t): a mixer whose whole memory is a running sum of fixed size."""

    kind: ClassVar[str] = "prefix_mean"
    hidden: int


class PrefixMean:
    graph_safe = False  # plain torch operations: the engine then runs it without captured graphs

    def __init__(self, spec, prefix):
        self.spec, self.prefix, self.w = spec, prefix, None

    def wanted(self):
        return {self.prefix + "weight": ((self.spec.hidden, self.spec.hidden), "linear")}

    def load(self, get, dtype, device):
        self.w = get(self.prefix + "weight").to(device=device, dtype=torch.float32)

    def cache_need(self):
        from nanospec_amd.parts import StateNeed

        return StateNeed((self.spec.hidden,), torch.float32)

    def forward(self, ctx, x, cache, owns_cache=True, out=None):
        indptr, slots = ctx.qo_indptr.tolist(), ctx.state_slots.tolist()
        pos = ctx.positions.to(torch.float32)
        res = torch.empty(x.shape, dtype=torch.float32, device=x.device)
        for b, slot in enumerate(slots):
            lo, hi = indptr[b], indptr[b + 1]
            sums = cache.state[slot] + torch.cumsum(x[lo:hi].float(), 0)
            cache.state[slot] = sums[-1]
            res[lo:hi] = (sums / (pos[lo:hi, None] + 1)) @ self.w.T
        res = res.to(x.dtype)
        return res if out is None else out.copy_(res)


def toy_model(dtype):
    """Layer 0: the toy mixer.  Layer 1: attention.  Run order: 0, 1, 1 again (a cache of its own), then 1 reading the
    cache of its first run."""
    import math

    from nanospec_amd.config.spec import (AttentionSpec, LayerCall, ModelSpec, PreNormBlockSpec, RMSNormSpec, RopeSpec, SwiGLUSpec)
    from nanospec_amd.parts import DecoderModel, register
    from nanospec_amd.weights import DictSource, random_tensors

    register("mixer", "prefix_mean", PrefixMean)
    hidden, vocab = 48, 97
    norm = RMSNormSpec(hidden, 1e-5)
    ffn = SwiGLUSpec(hidden, 80)
    attn = AttentionSpec(hidden, 3, 1, 16, RopeSpec(16, 1e4), 1 / math.sqrt(16))
    layers = (llama_block("model.layers.0.", norm, PrefixMeanSpec(hidden), norm, ffn),
              llama_block("model.layers.1.", norm, attn, norm, ffn))
    spec = ModelSpec(vocab, hidden, "model.embed_tokens.weight", layers,
                     (LayerCall(0), LayerCall(1), LayerCall(1), LayerCall(1, cache_from=1)), norm, "model.norm.weight", "lm_head.weight", True)
    net = DecoderModel(spec)
    assert "model.layers.0.prefix_mean.weight" in net.wanted()
    tensors = random_tensors(net.wanted(), seed=5, skip={"lm_head.weight"})
    tensors = {k: v * (6.0 if k.endswith("proj.weight") or k.endswith("mean.weight") else 1.0) for k, v in tensors.items()}
    return net.load(DictSource(tensors), dtype, DEV), tensors, spec


def toy_plain(tensors, tokens):
    """The toy model over a whole sequence with the plain functions."""
    w = tensors
    x = w["model.embed_tokens.weight"][torch.tensor(tokens)]
    t = len(tokens)
    cos, sin = pl.rotation_tables(torch.arange(t), pl.inverse_frequencies(16, 1e4, None))

    def ffn(x, p):
        h = pl.rms_norm(x, w[p + "post_attention_layernorm.weight"], 1e-5)
        return x + pl.swiglu(h, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])

    p0, p1 = "model.layers.0.", "model.layers.1."
    h = pl.rms_norm(x, w[p0 + "input_layernorm.weight"], 1e-5)
    x = ffn(x + (torch.cumsum(h, 0) / torch.arange(1, t + 1)[:, None]) @ w[p0 + "prefix_mean.weight"].T, p0)
    first_kv = None
    for run in range(3):
        h = pl.rms_norm(x, w[p1 + "input_layernorm.weight"], 1e-5)
        q = pl.rotate(pl.linear(h, w[p1 + "self_attn.q_proj.weight"]).view(t, 3, 16), cos, sin)
        if run < 2:
            k = pl.rotate(pl.linear(h, w[p1 + "self_attn.k_proj.weight"]).view(t, 1, 16), cos, sin)
            v = pl.linear(h, w[p1 + "self_attn.v_proj.weight"]).view(t, 1, 16)
            if run == 0:
                first_kv = (k, v)
        else:
            k, v = first_kv  # the third run reads the cache its first run wrote
        a = pl.causal_attention(q, k, v).reshape(t, -1)
        x = ffn(x + pl.linear(a, w[p1 + "self_attn.o_proj.weight"]), p1)
    return pl.rms_norm(x, w["model.norm.weight"], 1e-5) @ w["model.embed_tokens.weight"].T


def test_toy_mixer_with_state_layer_twice_and_borrowed_cache():
    from nanospec_amd.engine.replay import Replayer

    model, tensors, spec = toy_model(torch.float32)
    assert not model.graph_safe
    kinds = [type(n).__name__ for n in model.cache_needs]
    assert kinds == ["StateNeed", "PagedNeed", "PagedNeed", "NoneType"]
    g = torch.Generator().manual_seed(0)
    seqs = {r: torch.randint(0, 97, (n,), generator=g).tolist() for r, n in (("a", 37), ("b", 12), ("c", 29))}
    refs = {r: toy_plain(tensors, t) for r, t in seqs.items()}
    rep = Replayer(model, 128, page_size=4)
    assert len(rep.storage.states) == 1 and rep.storage.k[0].shape[0] == 2  # one state tensor; two attention caches in one group
    assert rep.storage.views[3] is rep.storage.views[1]

    def step(entries, end=()):
        out = rep.step([{"id": r, "tokens": seqs[r][s:e], "want": list(range(e - s))} for r, s, e in entries], list(end))
        want = torch.cat([refs[r][s:e] for r, s, e in entries])
        err = ((out - want).abs().amax(-1) / want.abs().amax(-1)).max()
        assert err < 1e-4, (entries, float(err))

    step([("a", 0, 10), ("b", 0, 12)], end=["b"])       # portions: the state carries over between them
    step([("a", 10, 11)])
    step([("a", 11, 30), ("c", 0, 2)])                  # request c gets the slot request b gave back: it must start from zero
    step([("a", 30, 37), ("c", 2, 29)], end=["a", "c"])
    rep.manager.check()


def test_a_model_without_any_paged_cache():
    """Every layer's mixer keeps a state of fixed size and nothing in pages (the shape of a recurrent architecture): no group
    of pages exists, requests still get slots, steps and the scheduler run as for any model."""
    from nanospec_amd import Engine, EngineConfig, SamplingParams
    from nanospec_amd.config.spec import LayerCall, ModelSpec, RMSNormSpec, SwiGLUSpec
    from nanospec_amd.engine.replay import Replayer
    from nanospec_amd.parts import DecoderModel, register
    from nanospec_amd.weights import DictSource, random_tensors

    register("mixer", "prefix_mean", PrefixMean)
    hidden, vocab = 40, 53
    norm = RMSNormSpec(hidden, 1e-5)
    layers = tuple(llama_block(f"model.layers.{i}.", norm, PrefixMeanSpec(hidden), norm, SwiGLUSpec(hidden, 56)) for i in range(2))
    spec = ModelSpec(vocab, hidden, "model.embed_tokens.weight", layers, (LayerCall(0), LayerCall(1)), norm, "model.norm.weight",
                     "lm_head.weight", False)
    net = DecoderModel(spec)
    w = random_tensors(net.wanted(), seed=2)
    w = {k: v * (6.0 if k.endswith("proj.weight") or k.endswith("mean.weight") else 1.0) for k, v in w.items()}
    model = net.load(DictSource(w), torch.float32, DEV)
    assert [type(n).__name__ for n in model.cache_needs] == ["StateNeed", "StateNeed"]

    def plain(tokens):
        x = w["model.embed_tokens.weight"][torch.tensor(tokens)]
        t = len(tokens)
        for i in range(2):
            p = f"model.layers.{i}."
            h = pl.rms_norm(x, w[p + "input_layernorm.weight"], 1e-5)
            x = x + (torch.cumsum(h, 0) / torch.arange(1, t + 1)[:, None]) @ w[p + "prefix_mean.weight"].T
            h = pl.rms_norm(x, w[p + "post_attention_layernorm.weight"], 1e-5)
            x = x + pl.swiglu(h, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
        return pl.rms_norm(x, w["model.norm.weight"], 1e-5) @ w["lm_head.weight"].T

    g = torch.Generator().manual_seed(1)
    seqs = {r: torch.randint(0, vocab, (n,), generator=g).tolist() for r, n in (("a", 33), ("b", 9))}
    refs = {r: plain(t) for r, t in seqs.items()}
    rep = Replayer(model, 128, page_size=4)
    assert not rep.manager.groups and len(rep.storage.states) == 2
    for entries, end in (([("a", 0, 20), ("b", 0, 3)], []), ([("a", 20, 21), ("b", 3, 9)], ["b"]), ([("a", 21, 33)], ["a"])):
        out = rep.step([{"id": r, "tokens": seqs[r][s:e], "want": list(range(e - s))} for r, s, e in entries], end)
        want = torch.cat([refs[r][s:e] for r, s, e in entries])
        assert ((out.cpu() - want).abs().amax(-1) / want.abs().amax(-1)).max() < 1e-4, entries
    rep.manager.check()
    # through the scheduler: greedy tokens equal the plain implementation's, whole sequence recomputed per token
    eng = Engine(model, EngineConfig(num_blocks=8, block_size=4, max_step_tokens=16, prefill_chunk=8))
    prompts = [seqs["a"][:11], seqs["b"][:4]]
    reqs = [eng.add(p, SamplingParams(max_tokens=6)) for p in prompts]
    while eng.has_work:
        eng.step()
    for p, r in zip(prompts, reqs):
        seq = list(p)
        for _ in range(6):
            seq.append(int(plain(seq)[-1].argmax()))
        assert r.out_tokens == seq[len(p):]


# ------------------------------------------------------- a toy feed-forward with routing and a toy position encoding


@dataclass(frozen=True)
class HarmonicRotationSpec:
    """Rotation of the first ``rotary_dim`` channels of a head by angle position / (j + 1) for pair j."""

    kind: ClassVar[str] = "harmonic"
    rotary_dim: int


class HarmonicRotation:
    graph_safe = True
    max_positions = None

    def __init__(self, spec, prefix=""):
        self.rotary_dim, self.inv_freq = spec.rotary_dim, None

    def wanted(self):
        return {}

    def load(self, get, dtype, device):
        self.inv_freq = (1.0 / torch.arange(1, self.rotary_dim // 2 + 1, dtype=torch.float32)).to(device)


@dataclass(frozen=True)
class TopOneExpertsSpec:
    """Each token goes through the one expert (a SwiGLU) its router row likes best, weighted by that expert's share of
    the soft-max over the router's 32-bit logits."""

    kind: ClassVar[str] = "top_one"
    hidden: int
    inner: int
    experts: int


class TopOneExperts:
    graph_safe = False

    def __init__(self, spec, prefix):
        self.spec, self.prefix = spec, prefix

    def wanted(self):
        s, p = self.spec, self.prefix
        out = {p + "router.weight": ((s.experts, s.hidden), "linear")}
        for e in range(s.experts):
            out[f"{p}experts.{e}.gate.weight"] = ((s.inner, s.hidden), "linear")
            out[f"{p}experts.{e}.up.weight"] = ((s.inner, s.hidden), "linear")
            out[f"{p}experts.{e}.down.weight"] = ((s.hidden, s.inner), "linear")
        return out

    def load(self, get, dtype, device):
        from nanospec_amd.parts.linear import GatedWeights, LinearWeight

        p = self.prefix
        self.router = get(p + "router.weight").to(device=device, dtype=torch.float32)
        on = lambda name: get(name).to(device=device, dtype=dtype).contiguous()
        self.gated = [GatedWeights(on(f"{p}experts.{e}.gate.weight"), on(f"{p}experts.{e}.up.weight")) for e in range(self.spec.experts)]
        self.down = [LinearWeight(on(f"{p}experts.{e}.down.weight")) for e in range(self.spec.experts)]

    def forward(self, ctx, x, out=None):
        share = torch.softmax(x.float() @ self.router.T, dim=-1)
        top, choice = share.max(-1)
        res = torch.zeros_like(x)
        for e in range(self.spec.experts):
            rows = (choice == e).nonzero().flatten()
            if rows.numel():
                xe = x[rows].contiguous()
                y = self.down[e](self.gated[e](ctx, xe, torch.empty((rows.numel(), self.spec.inner), dtype=x.dtype, device=x.device)))
                res[rows] = (y.float() * top[rows, None]).to(x.dtype)
        return res if out is None else out.copy_(res)


def test_toy_routed_feed_forward_and_toy_position_in_one_layer_only():
    import math

    from nanospec_amd.config.spec import AttentionSpec, LayerCall, ModelSpec, PreNormBlockSpec, RMSNormSpec, RopeSpec, SwiGLUSpec
    from nanospec_amd.engine.replay import Replayer
    from nanospec_amd.parts import DecoderModel, register
    from nanospec_amd.weights import DictSource, random_tensors

    register("ffn", "top_one", TopOneExperts)
    register("position", "harmonic", HarmonicRotation)
    hidden, vocab, hd = 40, 61, 32
    norm = RMSNormSpec(hidden, 1e-5)
    layers = (llama_block("model.layers.0.", norm, AttentionSpec(hidden, 2, 2, hd, RopeSpec(hd, 1e4), 1 / math.sqrt(hd)), norm, SwiGLUSpec(hidden, 56)),
              llama_block("model.layers.1.", norm, AttentionSpec(hidden, 2, 1, hd, HarmonicRotationSpec(16), 0.25), norm, TopOneExpertsSpec(hidden, 24, 3)))
    spec = ModelSpec(vocab, hidden, "model.embed_tokens.weight", layers, (LayerCall(0), LayerCall(1)), norm, "model.norm.weight", "lm_head.weight", False)
    net = DecoderModel(spec)
    wanted = net.wanted()
    assert "model.layers.1.top_one.router.weight" in wanted and "model.layers.0.mlp.gate_proj.weight" in wanted
    w = random_tensors(wanted, seed=11)
    w = {k: v * (8.0 if "proj" in k or "experts" in k or "router" in k else 1.0) for k, v in w.items()}
    model = net.load(DictSource(w), torch.float32, DEV)

    def plain(tokens):
        t = len(tokens)
        x = w["model.embed_tokens.weight"][torch.tensor(tokens)]
        positions = torch.arange(t)
        tables = [pl.rotation_tables(positions, pl.inverse_frequencies(hd, 1e4, None)),
                  pl.rotation_tables(positions, 1.0 / torch.arange(1, 9, dtype=torch.float32))]
        for i, (heads, kvh, rot, scale) in enumerate(((2, 2, hd, 1 / math.sqrt(hd)), (2, 1, 16, 0.25))):
            p = f"model.layers.{i}."
            h = pl.rms_norm(x, w[p + "input_layernorm.weight"], 1e-5)
            cos, sin = tables[i]
            turn = lambda y: torch.cat([pl.rotate(y[..., :rot], cos, sin), y[..., rot:]], -1)
            q = turn(pl.linear(h, w[p + "self_attn.q_proj.weight"]).view(t, heads, hd))
            k = turn(pl.linear(h, w[p + "self_attn.k_proj.weight"]).view(t, kvh, hd))
            v = pl.linear(h, w[p + "self_attn.v_proj.weight"]).view(t, kvh, hd)
            a = pl.causal_attention(q * (scale * math.sqrt(hd)), k, v).reshape(t, -1)  # the plain function scales by 1/sqrt(d)
            x = x + pl.linear(a, w[p + "self_attn.o_proj.weight"])
            h = pl.rms_norm(x, w[p + "post_attention_layernorm.weight"], 1e-5)
            if i == 0:
                x = x + pl.swiglu(h, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
            else:
                share = torch.softmax(h @ w[p + "top_one.router.weight"].T, -1)
                top, choice = share.max(-1)
                y = torch.stack([pl.swiglu(h[j : j + 1], w[f"{p}top_one.experts.{e}.gate.weight"], w[f"{p}top_one.experts.{e}.up.weight"],
                                           w[f"{p}top_one.experts.{e}.down.weight"])[0] for j, e in enumerate(choice.tolist())])
                x = x + y * top[:, None]
        return pl.rms_norm(x, w["model.norm.weight"], 1e-5) @ w["lm_head.weight"].T

    g = torch.Generator().manual_seed(3)
    seqs = {r: torch.randint(0, vocab, (n,), generator=g).tolist() for r, n in (("a", 41), ("b", 19))}
    refs = {r: plain(t) for r, t in seqs.items()}
    rep = Replayer(model, 128, page_size=8)
    for entries in ([("a", 0, 17), ("b", 0, 2)], [("a", 17, 18), ("b", 2, 19)], [("a", 18, 41)]):
        out = rep.step([{"id": r, "tokens": seqs[r][s:e], "want": list(range(e - s))} for r, s, e in entries], [])
        want = torch.cat([refs[r][s:e] for r, s, e in entries])
        err = ((out.cpu() - want).abs().amax(-1) / want.abs().amax(-1)).max()
        assert err < 1e-4, (entries, float(err))


# ------------------------------------------------------- a toy norm


@dataclass(frozen=True)
class CentredNormSpec:
    """y = weight * (r - mean(r)) / sqrt(var(r) + eps) + bias over the channels of a row."""

    kind: ClassVar[str] = "centred"
    dim: int
    eps: float


class CentredNorm:
    """Takes what every norm of a pre-norm block takes: the stream, what is still to be added to it, the rows to give.
    It does not say ``links_products``, so the products around it neither fold its factor in nor hand it unadded ranges."""

    graph_safe = True

    def __init__(self, spec, name):
        self.spec, self.name, self.bias_name = spec, name, name.replace("weight", "bias")

    def wanted(self):
        return {self.name: ((self.spec.dim,), "norm"), self.bias_name: ((self.spec.dim,), "linear")}

    def load(self, get, dtype, device):
        self.weight = get(self.name).to(device=device, dtype=dtype)
        self.bias = get(self.bias_name).to(device=device, dtype=dtype)

    def forward(self, ctx, resid=None, x=None, rows=None, write_resid=False, out=None):
        assert x is None or isinstance(x, torch.Tensor), type(x)  # never a product's unadded ranges
        r = resid if x is None else (resid.float() + x.float()).to(resid.dtype)
        if write_resid:
            resid.copy_(r)
        if rows is not None:
            r = r[rows.long()]
        f = r.float()
        y = (f - f.mean(-1, keepdim=True)) * torch.rsqrt(f.var(-1, unbiased=False, keepdim=True) + self.spec.eps)
        y = (y * self.weight.float() + self.bias.float()).to(r.dtype)
        return y if out is None else out.copy_(y)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_toy_norm_in_one_layer_and_at_the_end(dtype):
    """A norm of another kind, registered from here: both norms of the second layer and the norm before the head.  The first
    layer keeps RMS norms, whose products fold the norm in where they can (few rows, bfloat16) and must stop doing so at
    the border to the other kind."""
    import math

    from nanospec_amd.config.spec import AttentionSpec, LayerCall, ModelSpec, RMSNormSpec, RopeSpec, SwiGLUSpec
    from nanospec_amd.engine.replay import Replayer
    from nanospec_amd.parts import DecoderModel, register
    from nanospec_amd.weights import DictSource, random_tensors

    register("norm", "centred", CentredNorm)
    hidden, vocab, hd, inner = 64, 83, 16, 88
    rms, centred = RMSNormSpec(hidden, 1e-5), CentredNormSpec(hidden, 1e-3)
    attn = AttentionSpec(hidden, 4, 2, hd, RopeSpec(hd, 1e4), 1 / math.sqrt(hd))
    layers = (llama_block("model.layers.0.", rms, attn, rms, SwiGLUSpec(hidden, inner)),
              llama_block("model.layers.1.", centred, attn, centred, SwiGLUSpec(hidden, inner)),
              llama_block("model.layers.2.", rms, attn, rms, SwiGLUSpec(hidden, inner)))
    spec = ModelSpec(vocab, hidden, "model.embed_tokens.weight", layers, (LayerCall(0), LayerCall(1), LayerCall(2)), centred,
                     "model.norm.weight", "lm_head.weight", False)
    net = DecoderModel(spec)
    wanted = net.wanted()
    assert "model.layers.1.input_layernorm.bias" in wanted and "model.norm.bias" in wanted and "model.layers.0.input_layernorm.bias" not in wanted
    w = random_tensors(wanted, seed=5)
    w = {k: (v * 6.0 if "proj" in k else v + (0.3 if k.endswith("bias") else 0.0)).to(dtype) for k, v in w.items()}
    model = net.load(DictSource(w), dtype, DEV)

    def centred_norm(x, name, eps):
        f = x.float()
        y = (f - f.mean(-1, keepdim=True)) * torch.rsqrt(f.var(-1, unbiased=False, keepdim=True) + eps)
        return (y * w[name].float() + w[name.replace("weight", "bias")].float()).to(x.dtype)

    def plain(tokens):
        t = len(tokens)
        x = w["model.embed_tokens.weight"][torch.tensor(tokens)]
        cos, sin = pl.rotation_tables(torch.arange(t), pl.inverse_frequencies(hd, 1e4, None))
        for i in range(3):
            p = f"model.layers.{i}."
            norm = (lambda y, name: centred_norm(y, name, 1e-3)) if i == 1 else (lambda y, name: pl.rms_norm(y, w[name], 1e-5))
            h = norm(x, p + "input_layernorm.weight")
            q = pl.rotate(pl.linear(h, w[p + "self_attn.q_proj.weight"]).view(t, 4, hd), cos, sin)
            k = pl.rotate(pl.linear(h, w[p + "self_attn.k_proj.weight"]).view(t, 2, hd), cos, sin)
            v = pl.linear(h, w[p + "self_attn.v_proj.weight"]).view(t, 2, hd)
            x = x + pl.linear(pl.causal_attention(q, k, v).reshape(t, -1), w[p + "self_attn.o_proj.weight"])
            h = norm(x, p + "post_attention_layernorm.weight")
            x = x + pl.swiglu(h, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
        return centred_norm(x, "model.norm.weight", 1e-3).float() @ w["lm_head.weight"].float().T

    g = torch.Generator().manual_seed(9)
    seqs = {r: torch.randint(0, vocab, (n,), generator=g).tolist() for r, n in (("a", 60), ("b", 23))}
    refs = {r: plain(t) for r, t in seqs.items()}
    rep = Replayer(model, 128, page_size=8)
    steps = [[("a", 0, 40), ("b", 0, 2)], [("a", 40, 41), ("b", 2, 22)]] + [[("a", 41 + i, 42 + i)] + ([("b", 22, 23)] if i == 0 else []) for i in range(19)]
    for entries in steps:
        out = rep.step([{"id": r, "tokens": seqs[r][s:e], "want": list(range(e - s))} for r, s, e in entries], [])
        want = torch.cat([refs[r][s:e] for r, s, e in entries])
        if dtype == torch.float32:
            err = ((out.cpu() - want).abs().amax(-1) / want.abs().amax(-1)).max()
            assert err < 1e-4, (entries, float(err))
        else:
            assert ulps_of_row_max(out.cpu(), want).max() <= 8, entries
    assert rep.runner.last_used_graph  # the single-token steps were captured with the toy norm inside


# ------------------------------------------------------- a toy block of another shape, and tensor names of another origin


@dataclass(frozen=True)
class ParallelBlockSpec:
    """x = x + mixer(norm(x)) + feed_forward(norm(x)): one norm whose output both parts read."""

    kind: ClassVar[str] = "parallel"
    prefix: str
    norm: object
    mixer: object
    ffn: object


class ParallelBlock:
    graph_safe = False  # the sum of the two parts is a torch operation

    def __init__(self, spec, prefix=None):
        from nanospec_amd.parts import build

        p = spec.prefix
        self.norm = build("norm", spec.norm, p + "ln.w")
        self.mixer = build("mixer", spec.mixer, p + "att.")
        self.ffn = build("ffn", spec.ffn, p + "ff.")
        self.parts = (self.norm, self.mixer, self.ffn)

    def wanted(self):
        out = {}
        for part in self.parts:
            out.update(part.wanted())
        return out

    def load(self, get, dtype, device):
        for part in self.parts:
            part.load(get, dtype, device)

    def cache_need(self):
        return self.mixer.cache_need()

    def max_positions(self):
        return self.mixer.max_positions()

    def forward(self, ctx, resid, delta, cache, owns_cache, delta_out):
        h = self.norm.forward(ctx, resid=resid, x=delta, write_resid=delta is not None)
        a = self.mixer.forward(ctx, h, cache, owns_cache)
        f = self.ffn.forward(ctx, h)
        delta_out.copy_((a.float() + f.float()).to(delta_out.dtype))
        return None


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_toy_block_and_other_tensor_names(dtype):
    """A block of another shape registered from here (one norm, mixer and feed-forward side by side, tensor names of its
    own) before a pre-norm block whose four names are not Llama's: nothing in the framework knows either set of names."""
    import math

    from nanospec_amd.config.spec import AttentionSpec, LayerCall, ModelSpec, PreNormBlockSpec, RMSNormSpec, RopeSpec, SwiGLUSpec
    from nanospec_amd.engine.replay import Replayer
    from nanospec_amd.parts import DecoderModel, register
    from nanospec_amd.weights import DictSource, random_tensors

    register("block", "parallel", ParallelBlock)
    hidden, vocab, hd = 64, 131, 16
    norm = RMSNormSpec(hidden, 1e-5)
    attn = AttentionSpec(hidden, 4, 2, hd, RopeSpec(hd, 1e4, max_positions=96), 1 / math.sqrt(hd))
    ffn = SwiGLUSpec(hidden, 96)
    layers = (ParallelBlockSpec("h.0.", norm, attn, ffn),
              PreNormBlockSpec("h.1.", norm, attn, norm, ffn, mixer_norm_name="ln_a.weight", mixer_prefix="mix.",
                               ffn_norm_name="ln_b.weight", ffn_prefix="feed."))
    spec = ModelSpec(vocab, hidden, "wte", layers, (LayerCall(0), LayerCall(1)), norm, "ln_f", "out_head", False)
    net = DecoderModel(spec)
    names = set(net.wanted())
    assert {"h.0.ln.w", "h.0.att.q_proj.weight", "h.0.ff.down_proj.weight", "h.1.ln_a.weight", "h.1.mix.o_proj.weight",
            "h.1.ln_b.weight", "h.1.feed.gate_proj.weight", "wte", "ln_f", "out_head"} <= names
    assert not any("layernorm" in n or "self_attn" in n or "mlp" in n for n in names)
    w = {k: (v * (5.0 if "proj" in k else 1.0)).to(dtype) for k, v in random_tensors(net.wanted(), seed=21).items()}
    model = net.load(DictSource(w), dtype, DEV)
    assert model.max_positions == 96

    def plain(tokens):
        t = len(tokens)
        x = w["wte"][torch.tensor(tokens)]
        cos, sin = pl.rotation_tables(torch.arange(t), pl.inverse_frequencies(hd, 1e4, None))

        def attention(h, p):
            q = pl.rotate(pl.linear(h, w[p + "q_proj.weight"]).view(t, 4, hd), cos, sin)
            k = pl.rotate(pl.linear(h, w[p + "k_proj.weight"]).view(t, 2, hd), cos, sin)
            v = pl.linear(h, w[p + "v_proj.weight"]).view(t, 2, hd)
            return pl.linear(pl.causal_attention(q, k, v).reshape(t, -1), w[p + "o_proj.weight"])

        feed = lambda h, p: pl.swiglu(h, w[p + "gate_proj.weight"], w[p + "up_proj.weight"], w[p + "down_proj.weight"])
        h = pl.rms_norm(x, w["h.0.ln.w"], 1e-5)
        x = pl.residual_add(x, (attention(h, "h.0.att.").float() + feed(h, "h.0.ff.").float()).to(dtype))
        x = pl.residual_add(x, attention(pl.rms_norm(x, w["h.1.ln_a.weight"], 1e-5), "h.1.mix."))
        x = pl.residual_add(x, feed(pl.rms_norm(x, w["h.1.ln_b.weight"], 1e-5), "h.1.feed."))
        return pl.rms_norm(x, w["ln_f"], 1e-5).float() @ w["out_head"].float().T

    g = torch.Generator().manual_seed(8)
    seqs = {r: torch.randint(0, vocab, (n,), generator=g).tolist() for r, n in (("a", 45), ("b", 23))}
    refs = {r: plain(t) for r, t in seqs.items()}
    rep = Replayer(model, 256, page_size=4)
    for entries in ([("a", 0, 20), ("b", 0, 3)], [("a", 20, 21), ("b", 3, 23)], [("a", 21, 45)]):
        out = rep.step([{"id": r, "tokens": seqs[r][s:e], "want": list(range(e - s))} for r, s, e in entries], [])
        want = torch.cat([refs[r][s:e] for r, s, e in entries])
        if dtype == torch.float32:
            err = ((out.cpu() - want).abs().amax(-1) / want.abs().amax(-1)).max()
            assert err < 1e-4, (entries, float(err))
        else:
            assert ulps_of_row_max(out.cpu(), want).max() <= 8, entries
    with pytest.raises(ValueError):  # the block's mixer bounds the positions, and the model asks the block
        rep.step([{"id": "c", "tokens": list(range(97)), "want": []}], [])


# ------------------------------------------------------- layers that keep a window of keys beside layers that keep all


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_windowed_layers_give_pages_back_while_requests_run(dtype):
    """One layer sees every earlier key, two see the last ten: two groups of pages.  The windowed group's pool holds far
    fewer pages than the requests have positions, so pages that a window has passed are given back while the request
    runs and handed out again, to the same request and to others; block tables then hold released entries, which the
    kernels must never follow.  Against plain attention over the whole sequences with the window as a mask."""
    import math

    from nanospec_amd.cache.manager import RELEASED, CacheManager
    from nanospec_amd.cache.storage import CacheStorage, plan_groups
    from nanospec_amd.config.spec import AttentionSpec, LayerCall, ModelSpec, RMSNormSpec, RopeSpec, SwiGLUSpec
    from nanospec_amd.engine.runner import ModelRunner, StepEntry
    from nanospec_amd.parts import DecoderModel
    from nanospec_amd.weights import DictSource, random_tensors

    hidden, vocab, hd, page, window = 64, 83, 16, 4, 10
    norm = RMSNormSpec(hidden, 1e-5)
    ffn = SwiGLUSpec(hidden, 96)
    full = AttentionSpec(hidden, 4, 2, hd, RopeSpec(hd, 1e4), 1 / math.sqrt(hd))
    near = AttentionSpec(hidden, 4, 1, hd, RopeSpec(hd, 1e4), 1 / math.sqrt(hd), window=window)
    layers = tuple(llama_block(f"model.layers.{i}.", norm, a, norm, ffn) for i, a in enumerate((full, near, near)))
    spec = ModelSpec(vocab, hidden, "model.embed_tokens.weight", layers, tuple(LayerCall(i) for i in range(3)), norm, "model.norm.weight",
                     "lm_head.weight", True)
    net = DecoderModel(spec)
    w = {k: (v * (5.0 if "proj" in k else 1.0)).to(dtype) for k, v in random_tensors(net.wanted(), seed=31, skip={"lm_head.weight"}).items()}
    model = net.load(DictSource(w), dtype, DEV)
    specs, _, _ = plan_groups(model.cache_needs)
    assert [(s.name, s.window) for s in specs] == [("kv2x16", 0), ("kv1x16w10", window)]
    lengths = {"a": 61, "b": 47, "c": 52}
    pages = [sum(-(-n // page) for n in lengths.values()) + 2, 14]  # all keys of all requests; 14 pages for the windows
    manager = CacheManager(specs, pages, page, 8)
    storage = CacheStorage(model, pages, page, 8, dtype, model.device)
    runner = ModelRunner(model, manager, storage, 8, max(pages))

    g = torch.Generator().manual_seed(12)
    seqs = {r: torch.randint(0, vocab, (n,), generator=g).tolist() for r, n in lengths.items()}

    def plain(tokens):
        t = len(tokens)
        x = w["model.embed_tokens.weight"][torch.tensor(tokens)]
        cos, sin = pl.rotation_tables(torch.arange(t), pl.inverse_frequencies(hd, 1e4, None))
        for i, (kvh, win) in enumerate(((2, 0), (1, window), (1, window))):
            p = f"model.layers.{i}."
            h = pl.rms_norm(x, w[p + "input_layernorm.weight"], 1e-5)
            q = pl.rotate(pl.linear(h, w[p + "self_attn.q_proj.weight"]).view(t, 4, hd), cos, sin)
            k = pl.rotate(pl.linear(h, w[p + "self_attn.k_proj.weight"]).view(t, kvh, hd), cos, sin)
            v = pl.linear(h, w[p + "self_attn.v_proj.weight"]).view(t, kvh, hd)
            if win:
                a = torch.cat([pl.causal_attention(q[j : j + 1], k[max(0, j - win + 1) : j + 1], v[max(0, j - win + 1) : j + 1],
                                                   first_query=min(j, win - 1)) for j in range(t)])
            else:
                a = pl.causal_attention(q, k, v)
            x = pl.residual_add(x, pl.linear(a.reshape(t, -1), w[p + "self_attn.o_proj.weight"]))
            h = pl.rms_norm(x, w[p + "post_attention_layernorm.weight"], 1e-5)
            x = pl.residual_add(x, pl.swiglu(h, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"]))
        return pl.rms_norm(x, w["model.norm.weight"], 1e-5).float() @ w["model.embed_tokens.weight"].float().T

    refs = {r: plain(t) for r, t in seqs.items()}
    at = {r: 0 for r in seqs}
    granted = {}  # page of the windowed group -> the (request, table index) pairs it has served
    released_seen = 0
    import random

    rng = random.Random(3)
    for r in seqs:
        runner.admit(r)
    step_no = 0
    while any(at[r] < lengths[r] for r in seqs):
        entries, places = [], []
        for r in seqs:
            left = lengths[r] - at[r]
            if not left or rng.random() < 0.15:
                continue
            n = 1 if rng.random() < 0.5 else min(left, rng.choice((2, 3, 4)))  # never more than a page beyond the window
            entries.append(StepEntry(r, seqs[r][at[r] : at[r] + n], list(range(n))))
            places += [(r, at[r] + i) for i in range(n)]
            at[r] += n
        if not entries:
            continue
        out = runner.step(entries).cpu()
        want = torch.stack([refs[r][p] for r, p in places])
        if dtype == torch.float32:
            err = ((out - want).abs().amax(-1) / want.abs().amax(-1)).max()
            assert err < 1e-4, (step_no, float(err))
        else:
            assert ulps_of_row_max(out, want).max() <= 8, step_no
        manager.check()
        for r in seqs:
            table = manager.get(r).tables[1]
            released_seen += sum(1 for p in table if p == RELEASED)
            assert manager.get(r).held[1] <= -(-window // page) + 2
            for i, p in enumerate(table):
                if p != RELEASED:
                    granted.setdefault(p, set()).add((r, i))
        step_no += 1
    assert released_seen > 100, "the windows were meant to give pages back"
    assert sum(1 for uses in granted.values() if len(uses) > 1) >= 10, "pages of the windowed group were meant to be used again"
    assert sum(lengths.values()) > 2 * pages[1] * page  # the windowed pool holds less than half of what was written through it
    for r in seqs:
        runner.release(r)
    manager.check()


# ------------------------------------------------------- a whole architecture that the framework has never heard of


@dataclass(frozen=True)
class ToyParallelConfig:
    """The configuration of an architecture defined here: blocks with one norm and mixer and feed-forward side by side,
    config.json keys and tensor names of its own."""

    vocab: int
    width: int
    depth: int
    n_head: int
    n_kv: int
    d_head: int
    d_ff: int
    eps: float
    n_ctx: int

    @classmethod
    def from_hf(cls, cfg, generation_cfg=None):
        return cls(cfg["vocab"], cfg["width"], cfg["depth"], cfg["n_head"], cfg["n_kv"], cfg["d_head"], cfg["d_ff"], cfg["eps"], cfg["n_ctx"])

    def to_hf(self):
        return dict(architectures=["ToyParallelLM"], model_type="toy_parallel", **self.__dict__)

    def model_spec(self):
        import math

        from nanospec_amd.config.spec import AttentionSpec, LayerCall, ModelSpec, RMSNormSpec, RopeSpec, SwiGLUSpec

        norm = RMSNormSpec(self.width, self.eps)
        attn = AttentionSpec(self.width, self.n_head, self.n_kv, self.d_head, RopeSpec(self.d_head, 1e4, max_positions=self.n_ctx),
                             1 / math.sqrt(self.d_head))
        layers = tuple(ParallelBlockSpec(f"h.{i}.", norm, attn, SwiGLUSpec(self.width, self.d_ff)) for i in range(self.depth))
        return ModelSpec(self.vocab, self.width, "wte", layers, tuple(LayerCall(i) for i in range(self.depth)), norm, "ln_f", "out_head", False)


def test_an_architecture_registered_from_outside_generates(tmp_path):
    """A typed configuration, a block class and one registry entry, all defined in this file: the framework writes a model
    folder with random weights for it, finds the architecture by config.json, loads it by tensor name, generates through
    the engine and the one-call entry point, and replays a trace; the tokens are the plain functions' greedy choice."""
    import json

    from nanospec_amd import SamplingParams, generate, load_model
    from nanospec_amd.config import load_config, register_architecture
    from nanospec_amd.engine.replay import Replayer
    from nanospec_amd.parts import register
    from nanospec_amd.weights import write_model_folder

    register("block", "parallel", ParallelBlock)
    register_architecture("ToyParallelLM", lambda cfg, gen=None: (lambda c: (c, c.model_spec()))(ToyParallelConfig.from_hf(cfg, gen)),
                          model_type="toy_parallel")
    config = ToyParallelConfig(vocab=131, width=64, depth=2, n_head=4, n_kv=2, d_head=16, d_ff=96, eps=1e-5, n_ctx=96)
    folder = write_model_folder(tmp_path / "toy", config, seed=9)
    assert json.loads((folder / "config.json").read_text())["architectures"] == ["ToyParallelLM"]
    loaded_cfg, spec = load_config(folder)
    assert loaded_cfg == config and spec.embed_name == "wte"
    w = pl.read_safetensors(folder / "model.safetensors")
    assert "h.1.att.k_proj.weight" in w and "h.0.ln.w" in w

    def plain(tokens):
        t = len(tokens)
        x = w["wte"][torch.tensor(tokens)]
        cos, sin = pl.rotation_tables(torch.arange(t), pl.inverse_frequencies(16, 1e4, None))
        for i in range(2):
            p = f"h.{i}."
            h = pl.rms_norm(x, w[p + "ln.w"], 1e-5)
            q = pl.rotate(pl.linear(h, w[p + "att.q_proj.weight"]).view(t, 4, 16), cos, sin)
            k = pl.rotate(pl.linear(h, w[p + "att.k_proj.weight"]).view(t, 2, 16), cos, sin)
            v = pl.linear(h, w[p + "att.v_proj.weight"]).view(t, 2, 16)
            a = pl.linear(pl.causal_attention(q, k, v).reshape(t, -1), w[p + "att.o_proj.weight"])
            f = pl.swiglu(h, w[p + "ff.gate_proj.weight"], w[p + "ff.up_proj.weight"], w[p + "ff.down_proj.weight"])
            x = x + (a + f)
        return pl.rms_norm(x, w["ln_f"], 1e-5) @ w["out_head"].T

    def plain_greedy(prompt, n):
        seq = list(prompt)
        for _ in range(n):
            seq.append(int(plain(seq)[-1].argmax()))
        return seq[len(prompt):]

    g = torch.Generator().manual_seed(2)
    prompts = [torch.randint(0, 131, (n,), generator=g).tolist() for n in (4, 19, 33)]
    want = [plain_greedy(p, 6) for p in prompts]
    assert generate(str(folder), prompts, SamplingParams(max_tokens=6), dtype="float32", block_size=4, max_step_tokens=24, prefill_chunk=16) == want
    model = load_model(folder, dtype="float32")
    assert model.max_positions == 96
    rep = Replayer(model, 128, page_size=4)
    out = rep.step([{"id": "a", "tokens": prompts[2][:20], "want": [19]}, {"id": "b", "tokens": prompts[1][:2], "want": []}], [])
    torch.testing.assert_close(out[0], plain(prompts[2][:20])[-1], rtol=1e-4, atol=1e-4)
    out = rep.step([{"id": "a", "tokens": prompts[2][20:], "want": [12]}, {"id": "b", "tokens": prompts[1][2:], "want": [16]}], ["a", "b"])
    torch.testing.assert_close(out, torch.stack([plain(prompts[2])[-1], plain(prompts[1])[-1]]), rtol=1e-4, atol=1e-4)


# ------------------------------------------- an architecture whose differences lie at the ends of the stack and in the rotation


def interleaved_rotation(x, positions, inv_freq, factor):
    """Channels 2j and 2j + 1 of x [T, heads, d] turn by angle position * inv_freq[j]; cosine and sine times ``factor``."""
    ang = torch.outer(positions.float(), inv_freq)
    c, s = ang.cos()[:, None, :] * factor, ang.sin()[:, None, :] * factor
    a, b = x.float()[..., 0::2], x.float()[..., 1::2]
    out = torch.empty(x.shape, dtype=torch.float32)
    out[..., 0::2] = a * c - b * s
    out[..., 1::2] = b * c + a * s
    return out.to(x.dtype)


def gain_law(shape, generator):
    """The initial law of a tensor that says so itself: uniform in [0.5, 1.5]."""
    return torch.rand(shape, generator=generator, device=generator.device) + 0.5


@dataclass(frozen=True)
class GainBiasFfnSpec:
    """down(silu(gate x) * up x) * gain + bias: a gain drawn by a law of its own and a bias that starts at zero."""

    kind: ClassVar[str] = "gain_bias_ffn"
    hidden: int
    inner: int


class GainBiasFfn:
    graph_safe = True  # the product's kernels, then two in-place operations on the output buffer

    def __init__(self, spec, prefix):
        from nanospec_amd.config.spec import SwiGLUSpec
        from nanospec_amd.parts import build

        self.spec, self.prefix = spec, prefix
        self.inner = build("ffn", SwiGLUSpec(spec.hidden, spec.inner), prefix)

    def wanted(self):
        return {**self.inner.wanted(), self.prefix + "gain": ((self.spec.hidden,), gain_law), self.prefix + "bias": ((self.spec.hidden,), "zeros")}

    def load(self, get, dtype, device):
        self.inner.load(get, dtype, device)
        self.gain = get(self.prefix + "gain").to(device=device, dtype=dtype)
        self.bias = get(self.prefix + "bias").to(device=device, dtype=dtype)

    def forward(self, ctx, x, out=None):
        out = self.inner.forward(ctx, x, out=out if out is not None else ctx.arena.take((x.shape[0], self.spec.hidden), x.dtype))
        return out.mul_(self.gain).add_(self.bias)


@dataclass(frozen=True)
class ToyScaledConfig:
    """Pre-norm blocks as the framework has them, and around them what the Llama decoder does not do: the embedding enters
    the stream scaled, the logits leave scaled and soft-capped, the rotation pairs neighbouring channels of a part of the
    head and scales cosine and sine, the feed-forward ends in a gain and a bias."""

    vocab: int
    width: int
    depth: int
    n_head: int
    n_kv: int
    d_head: int
    d_rot: int
    d_ff: int
    eps: float
    rot_factor: float
    emb_scale: float
    out_scale: float
    out_cap: float

    @classmethod
    def from_hf(cls, cfg, generation_cfg=None):
        return cls(**{k: cfg[k] for k in cls.__dataclass_fields__})

    def to_hf(self):
        return dict(architectures=["ToyScaledLM"], model_type="toy_scaled", **self.__dict__)

    def model_spec(self):
        import math

        from nanospec_amd.config.spec import AttentionSpec, LayerCall, ModelSpec, PreNormBlockSpec, RMSNormSpec, RopeSpec

        norm = RMSNormSpec(self.width, self.eps)
        rope = RopeSpec(self.d_rot, 1e4, interleaved=True, cos_sin_factor=self.rot_factor)
        attn = AttentionSpec(self.width, self.n_head, self.n_kv, self.d_head, rope, 1 / math.sqrt(self.d_head))
        layers = tuple(PreNormBlockSpec(f"blocks.{i}.", norm, attn, norm, GainBiasFfnSpec(self.width, self.d_ff), mixer_norm_name="n1", mixer_prefix="attn.",
                                        ffn_norm_name="n2", ffn_prefix="ffn.") for i in range(self.depth))
        return ModelSpec(self.vocab, self.width, "emb", layers, tuple(LayerCall(i) for i in range(self.depth)), norm, "n_out", "head", False,
                         embed_scale=self.emb_scale, logit_scale=self.out_scale, logit_softcap=self.out_cap)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_an_architecture_with_other_ends_and_another_rotation(tmp_path, dtype):
    """Registered from this file, nothing in the package changed: interleaved rotation of half a head with a factor on cosine
    and sine, an embedding scale, a logit scale and soft cap, a part whose tensors name their own initial laws.  The
    framework writes its folder, finds it by config.json, generates, and replays whole, in portions and token by token
    (in bfloat16 through the kernels that fuse the rotation into the q/k/v product, and through captured steps)."""
    from nanospec_amd import SamplingParams, generate, load_model
    from nanospec_amd.config import register_architecture
    from nanospec_amd.engine.replay import Replayer
    from nanospec_amd.parts import register
    from nanospec_amd.weights import write_model_folder

    register("ffn", "gain_bias_ffn", GainBiasFfn)
    register_architecture("ToyScaledLM", lambda cfg, gen=None: (lambda c: (c, c.model_spec()))(ToyScaledConfig.from_hf(cfg, gen)),
                          model_type="toy_scaled")
    c = ToyScaledConfig(vocab=211, width=1024, depth=2, n_head=4, n_kv=2, d_head=32, d_rot=16, d_ff=192, eps=1e-5, rot_factor=0.8,
                        emb_scale=7.5, out_scale=0.6, out_cap=3.0)
    folder = write_model_folder(tmp_path / "toy", c, seed=21, dtype=dtype)
    w = pl.read_safetensors(folder / "model.safetensors")
    for i in range(c.depth):
        gain, bias = w[f"blocks.{i}.ffn.gain"].float(), w[f"blocks.{i}.ffn.bias"].float()
        assert torch.count_nonzero(bias) == 0 and 0.5 <= gain.min() < gain.max() <= 1.5 and gain.std() > 0.2
        w[f"blocks.{i}.ffn.bias"] = (torch.randn(c.width, generator=torch.Generator().manual_seed(i)) * 0.05).to(dtype)  # a bias that shows
    from safetensors.torch import save_file

    save_file({k: v.contiguous() for k, v in w.items()}, str(folder / "model.safetensors"))
    inv = pl.inverse_frequencies(c.d_rot, 1e4, None)

    def plain(tokens):
        t = len(tokens)
        pos = torch.arange(t)
        x = (w["emb"][torch.tensor(tokens)].float() * c.emb_scale).to(dtype)
        turn = lambda y: torch.cat([interleaved_rotation(y[..., : c.d_rot], pos, inv, c.rot_factor), y[..., c.d_rot :]], -1)
        for i in range(c.depth):
            p = f"blocks.{i}."
            h = pl.rms_norm(x, w[p + "n1"], c.eps)
            q = turn(pl.linear(h, w[p + "attn.q_proj.weight"]).view(t, c.n_head, c.d_head))
            k = turn(pl.linear(h, w[p + "attn.k_proj.weight"]).view(t, c.n_kv, c.d_head))
            v = pl.linear(h, w[p + "attn.v_proj.weight"]).view(t, c.n_kv, c.d_head)
            x = pl.residual_add(x, pl.linear(pl.causal_attention(q, k, v).reshape(t, -1), w[p + "attn.o_proj.weight"]))
            h = pl.rms_norm(x, w[p + "n2"], c.eps)
            f = pl.swiglu(h, w[p + "ffn.gate_proj.weight"], w[p + "ffn.up_proj.weight"], w[p + "ffn.down_proj.weight"])
            f = (f * w[p + "ffn.gain"]) + w[p + "ffn.bias"]  # two roundings in the stream's precision, as the part does it
            x = pl.residual_add(x, f)
        z = pl.rms_norm(x, w["n_out"], c.eps).float() @ w["head"].float().T * c.out_scale
        return c.out_cap * torch.tanh(z / c.out_cap)

    def close(ours, ref, what):
        if dtype == torch.float32:
            err = ((ours - ref).abs().amax(-1) / ref.abs().amax(-1)).max()
            assert err < 1e-4, (what, float(err))
        else:
            assert ulps_of_row_max(ours, ref).max() <= 8, what

    g = torch.Generator().manual_seed(4)
    toks = torch.randint(0, c.vocab, (90,), generator=g).tolist()
    ref = plain(toks)
    assert ref.abs().max() < c.out_cap and ref.abs().max() > 0.5 * c.out_cap * 0.2  # the cap bounds the logits and is not idle
    model = load_model(folder, dtype=dtype)
    rep = Replayer(model, 256, page_size=8)
    out = rep.step([{"id": "whole", "tokens": toks, "want": list(range(90))}], ["whole"])
    close(out, ref, "whole")
    at = 0
    for n in (40, 20, 2, 9) + (1,) * 19:  # 17 to 128 rows, up to 16 rows, single tokens (captured steps)
        out = rep.step([{"id": "cut", "tokens": toks[at : at + n], "want": list(range(n))}], [])
        close(out, ref[at : at + n], f"tokens {at}:{at + n}")
        at += n
    assert at == 90 and rep.runner.last_used_graph
    if dtype == torch.float32:
        seq = list(toks[:12])
        for _ in range(5):
            seq.append(int(plain(seq)[-1].argmax()))
        assert generate(str(folder), [toks[:12]], SamplingParams(max_tokens=5), dtype="float32", block_size=8) == [seq[12:]]
