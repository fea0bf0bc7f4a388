"""What fixes the plain implementation beside the reference's text: special cases that reduce to a library routine,
invariants, and the vectors the reference's own tests hold.  Each is chosen so that a plausible mistake fails it.
CPU only."""

import math

import pytest
import torch
import torch.nn.functional as F

import plain_llama as pl


def test_rms_norm_against_float64_and_its_invariants():
    torch.manual_seed(0)
    x, w = torch.randn(5, 48) * 3, 1 + 0.1 * torch.randn(48)
    x64 = x.double()
    ref = x64 / torch.sqrt((x64 ** 2).mean(-1, keepdim=True) + 1e-6) * w.double()
    torch.testing.assert_close(pl.rms_norm(x, w, 1e-6).double(), ref, rtol=1e-6, atol=1e-6)
    unit = pl.rms_norm(x, torch.ones(48), 0.0)
    torch.testing.assert_close((unit ** 2).mean(-1), torch.ones(5))  # rows come out with RMS 1: the mean, not the sum
    torch.testing.assert_close(pl.rms_norm(7 * x, w, 0.0), pl.rms_norm(x, w, 0.0))  # scale invariance
    big_eps = pl.rms_norm(x, torch.ones(48), 1e6)
    assert big_eps.abs().max() < 0.02  # eps sits inside the square root, beside the mean


def test_rms_norm_casts_before_the_weight():
    """model/llama.py:95: in bfloat16 the normalised value is rounded BEFORE the multiplication by the weight."""
    x = torch.tensor([[1.0, 2.0, 3.0, 4.0]], dtype=torch.bfloat16)
    w = torch.tensor([1.5, 0.7, 1.1, 0.9], dtype=torch.bfloat16)
    h = x.float() * torch.rsqrt((x.float() ** 2).mean(-1, keepdim=True) + 1e-5)
    assert torch.equal(pl.rms_norm(x, w, 1e-5), w * h.to(torch.bfloat16))


def test_inverse_frequencies():
    inv = pl.inverse_frequencies(16, 10000.0, None)
    torch.testing.assert_close(inv, torch.tensor([10000.0 ** (-2 * j / 16) for j in range(8)]))
    assert inv[0] == 1.0 and torch.all(inv[1:] < inv[:-1])
    s = dict(factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=64)
    torch.testing.assert_close(pl.inverse_frequencies(32, 5e5, dict(s, factor=1.0)), pl.inverse_frequencies(32, 5e5, None))
    base, scaled = pl.inverse_frequencies(32, 5e5, None), pl.inverse_frequencies(32, 5e5, s)
    wavelen = 2 * math.pi / base
    high, low = wavelen < 64 / 4.0, wavelen > 64 / 1.0
    assert high.any() and low.any() and (~high & ~low).any()  # all three bands occur in this table
    torch.testing.assert_close(scaled[high], base[high])          # short waves untouched
    torch.testing.assert_close(scaled[low], base[low] / 8.0)      # long waves divided by the factor
    mid = ~high & ~low
    assert torch.all(scaled[mid] < base[mid]) and torch.all(scaled[mid] > base[mid] / 8.0)
    assert torch.all(scaled[1:] <= scaled[:-1])  # still monotone across the bands


def test_rotation_pairs_and_relative_positions():
    torch.manual_seed(1)
    d = 16
    inv = pl.inverse_frequencies(d, 10000.0, None)
    q, k = torch.randn(1, 1, d), torch.randn(1, 1, d)
    cos0, sin0 = pl.rotation_tables(torch.tensor([0]), inv)
    torch.testing.assert_close(pl.rotate(q, cos0, sin0), q)  # position 0 is the identity
    cos, sin = pl.rotation_tables(torch.tensor([5]), inv)
    r = pl.rotate(q, cos, sin)
    # the pair is (j, j + d/2), not (2j, 2j + 1): each such pair keeps its length
    torch.testing.assert_close(r[..., :8] ** 2 + r[..., 8:] ** 2, q[..., :8] ** 2 + q[..., 8:] ** 2)
    assert not torch.allclose(r[..., 0::2] ** 2 + r[..., 1::2] ** 2, q[..., 0::2] ** 2 + q[..., 1::2] ** 2)
    # the sign: a rotation by +angle (x1' = x1 cos - x2 sin)
    ang = 5 * inv[0]
    assert r[0, 0, 0] == pytest.approx(float(q[0, 0, 0] * torch.cos(ang) - q[0, 0, 8] * torch.sin(ang)), rel=1e-5)

    def dot(m, n):
        cm, sm = pl.rotation_tables(torch.tensor([m]), inv)
        cn, sn = pl.rotation_tables(torch.tensor([n]), inv)
        return float((pl.rotate(q, cm, sm) * pl.rotate(k, cn, sn)).sum())

    assert dot(9, 4) == pytest.approx(dot(25, 20), rel=1e-4, abs=1e-4)  # only the distance counts
    assert dot(9, 4) != pytest.approx(dot(4, 9), rel=1e-3)               # and its direction


def test_attention_reduces_to_the_library_routine():
    """The reference's three branches (model/attention.py:32-41): whole prompt = causal SDPA with grouped heads, one decode
    row = unmasked SDPA, a portion = explicit mask kpos <= qpos."""
    torch.manual_seed(2)
    heads, kvh, d, t = 6, 2, 8, 11
    q, k, v = torch.randn(t, heads, d), torch.randn(t, kvh, d), torch.randn(t, kvh, d)
    sdpa = lambda qq, mask=None, causal=False: F.scaled_dot_product_attention(
        qq.transpose(0, 1)[None], k.transpose(0, 1)[None], v.transpose(0, 1)[None], attn_mask=mask, is_causal=causal,
        enable_gqa=True)[0].transpose(0, 1)
    torch.testing.assert_close(pl.causal_attention(q, k, v), sdpa(q, causal=True), rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(pl.causal_attention(q[-1:], k, v, first_query=t - 1), sdpa(q[-1:]), rtol=1e-5, atol=1e-5)
    mask = torch.arange(t)[None, :] <= torch.arange(t - 4, t)[:, None]
    torch.testing.assert_close(pl.causal_attention(q[-4:], k, v, first_query=t - 4), sdpa(q[-4:], mask=mask), rtol=1e-5, atol=1e-5)
    # one head, no rotation, one key: the output is that key's value whatever the scores
    torch.testing.assert_close(pl.causal_attention(q[:1, :1], k[:1, :1], v[:1, :1]), v[:1, :1])
    # the scale: doubling d's worth of identical entries must not saturate differently than 1/sqrt(d) says
    qq, kk = torch.ones(1, 1, 4), torch.stack([torch.ones(1, 4), torch.zeros(1, 4)])
    vv = torch.tensor([[[1.0]], [[0.0]]]).expand(2, 1, 4).contiguous()
    p = pl.causal_attention(qq, kk, vv, first_query=1)[0, 0, 0]
    assert float(p) == pytest.approx(1 / (1 + math.exp(-4 / math.sqrt(4))), rel=1e-5)


def test_grouped_heads_share_consecutive_query_heads():
    """Query head h reads key/value head h // group (model/attention.py:33), not h % kv_heads."""
    torch.manual_seed(3)
    q, k, v = torch.randn(3, 4, 8), torch.randn(3, 2, 8), torch.randn(3, 2, 8)
    out = pl.causal_attention(q, k, v)
    for h in range(4):
        alone = pl.causal_attention(q[:, h : h + 1], k[:, h // 2 : h // 2 + 1], v[:, h // 2 : h // 2 + 1])
        torch.testing.assert_close(out[:, h : h + 1], alone)


def test_swiglu_and_linear():
    torch.manual_seed(4)
    x, g, u, dn = torch.randn(3, 10), torch.randn(7, 10), torch.randn(7, 10), torch.randn(10, 7)
    torch.testing.assert_close(pl.swiglu(x, g, u, dn), F.linear(F.silu(F.linear(x, g)) * F.linear(x, u), dn), rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(pl.linear(x, g), x @ g.T)


def test_whole_model_properties(tiny_folders):
    cfg, w = pl.read_config(tiny_folders["A"]), pl.read_weights(tiny_folders["A"], torch.float32)
    assert cfg["tied"] and w["lm_head.weight"] is w["model.embed_tokens.weight"]  # one storage (model/loader.py:65-66)
    toks = [3, 200, 17, 17, 42, 9]
    full = pl.logits_of_sequence(w, cfg, toks)
    assert full.shape == (6, 256)
    # causality: a prefix's logits do not depend on what follows
    torch.testing.assert_close(pl.logits_of_sequence(w, cfg, toks[:4]), full[:4], rtol=1e-5, atol=1e-6)
    cfgB, wB = pl.read_config(tiny_folders["B"]), pl.read_weights(tiny_folders["B"], torch.float32)
    assert not cfgB["tied"] and cfgB["scaling"]["factor"] == 8.0 and cfgB["kv_heads"] == 1 and cfgB["eps"] == 1e-6
    new, rows = pl.greedy_continuation(wB, cfgB, [5, 6, 7], 3)
    assert len(new) == 3 and new[0] == int(pl.logits_of_sequence(wB, cfgB, [5, 6, 7])[-1].argmax())


# ------------------------------------------------------------------ how the parts are put together
# No text but the reference's fixes the order of norms, sums and rotations, so each property below is one that only the
# right arrangement has: a plausible other arrangement (a norm after the sum, a branch that reads the raw stream, a value
# that is rotated, a last norm left out) fails at least one of them.


def _layer_setup(name, tiny_folders, t=9):
    cfg, w = pl.read_config(tiny_folders[name]), pl.read_weights(tiny_folders[name], torch.float32)
    torch.manual_seed(5)
    x = torch.randn(t, cfg["hidden"])
    inv = pl.inverse_frequencies(cfg["head_dim"], cfg["theta"], cfg["scaling"])
    return cfg, dict(w), x, inv


@pytest.mark.parametrize("name", ["A", "B"])
def test_layer_is_pre_norm_with_two_plain_sums(tiny_folders, name):
    cfg, w, x, inv = _layer_setup(name, tiny_folders)
    p = "model.layers.0."
    cos, sin = pl.rotation_tables(torch.arange(x.shape[0]), inv)
    out = pl.decoder_layer(x, w, p, cfg, cos, sin)
    # (1) the norms sit in front of the parts, inside the branches: with both norm weights zero each part sees zeros and
    #     returns zeros (no biases), and the layer is the identity.  A norm behind a sum would give zeros.
    w0 = dict(w)
    w0[p + "input_layernorm.weight"] = torch.zeros_like(w[p + "input_layernorm.weight"])
    w0[p + "post_attention_layernorm.weight"] = torch.zeros_like(w[p + "post_attention_layernorm.weight"])
    assert torch.equal(pl.decoder_layer(x, w0, p, cfg, cos, sin), x)
    # (2) each branch is added once, unscaled: without the feed-forward (down = 0) the layer's change of the stream is
    #     linear in the output projection, and it vanishes with it
    wd = dict(w)
    wd[p + "mlp.down_proj.weight"] = torch.zeros_like(w[p + "mlp.down_proj.weight"])
    inc = pl.decoder_layer(x, wd, p, cfg, cos, sin) - x
    wd2 = dict(wd)
    wd2[p + "self_attn.o_proj.weight"] = 2 * w[p + "self_attn.o_proj.weight"]
    torch.testing.assert_close(pl.decoder_layer(x, wd2, p, cfg, cos, sin) - x, 2 * inc, rtol=1e-5, atol=1e-6)
    wd2[p + "self_attn.o_proj.weight"] = torch.zeros_like(w[p + "self_attn.o_proj.weight"])
    assert torch.equal(pl.decoder_layer(x, wd2, p, cfg, cos, sin), x)
    # (3) the branches read the NORMED stream: scaling the stream leaves the attention branch's output as it was (eps is
    #     tiny beside these values), so the change of the stream stays the same while the stream is seven times larger
    torch.testing.assert_close(pl.decoder_layer(7 * x, wd, p, cfg, cos, sin) - 7 * x, inc, rtol=1e-3, atol=1e-5)
    # (4) the feed-forward reads the stream AFTER the attention's sum: it equals the feed-forward alone applied to it
    mid = x + inc
    wa = dict(w)
    wa[p + "self_attn.o_proj.weight"] = torch.zeros_like(w[p + "self_attn.o_proj.weight"])
    torch.testing.assert_close(out, pl.decoder_layer(mid, wa, p, cfg, cos, sin), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("name", ["A", "B"])
def test_layer_rotates_queries_and_keys_but_not_values(tiny_folders, name):
    """Only distances count: with every position shifted by the same amount the layer's output is the same.  That holds
    if queries and keys are turned alike and values are not; a rotated value, or a rotation of one of q and k only,
    changes the output with the shift."""
    cfg, w, x, inv = _layer_setup(name, tiny_folders)
    p = "model.layers.0."
    t = x.shape[0]
    base = pl.decoder_layer(x, w, p, cfg, *pl.rotation_tables(torch.arange(t), inv))
    far = pl.decoder_layer(x, w, p, cfg, *pl.rotation_tables(torch.arange(t) + 41, inv))
    torch.testing.assert_close(far, base, rtol=1e-4, atol=1e-5)
    # and the rotation is there at all: reversing the order of the positions changes the output
    back = pl.decoder_layer(x, w, p, cfg, *pl.rotation_tables(torch.arange(t - 1, -1, -1), inv))
    assert not torch.allclose(back, base, rtol=1e-3, atol=1e-4)


@pytest.mark.parametrize("name", ["A", "B"])
def test_model_without_branches_is_last_norm_and_head(tiny_folders, name):
    """With every output and down projection zero the layers pass the embedding through, and the logits must be the
    library's RMS norm of the embedding rows times the head: the last norm is applied, once, with the model's eps, and
    the head is the tied table or the head of its own."""
    cfg, w = pl.read_config(tiny_folders[name]), dict(pl.read_weights(tiny_folders[name], torch.float32))
    for k in list(w):
        if k.endswith("o_proj.weight") or k.endswith("down_proj.weight"):
            w[k] = torch.zeros_like(w[k])
    toks = [3, 99, 17, 17, 42]
    emb = w["model.embed_tokens.weight"][torch.tensor(toks)]
    normed = F.rms_norm(emb, (cfg["hidden"],), w["model.norm.weight"], cfg["eps"])
    head = w["model.embed_tokens.weight"] if cfg["tied"] else w["lm_head.weight"]
    got = pl.logits_of_sequence(w, cfg, toks)
    torch.testing.assert_close(got, normed @ head.T, rtol=1e-5, atol=1e-6)
    w2 = dict(w)
    w2["model.norm.weight"] = 2 * w["model.norm.weight"]
    torch.testing.assert_close(pl.logits_of_sequence(w2, cfg, toks), 2 * got, rtol=1e-5, atol=1e-6)
    assert torch.equal(got[2], got[3])  # equal tokens, nothing mixes positions: equal rows


def test_layers_run_in_order_and_each_once(tiny_folders):
    """Swapping two layers' weights changes the logits; and the model is the layers applied in turn to the embedding."""
    cfg, w = pl.read_config(tiny_folders["B"]), pl.read_weights(tiny_folders["B"], torch.float32)
    toks = [5, 600, 7, 123, 9, 9, 31]
    full = pl.logits_of_sequence(w, cfg, toks)
    x = w["model.embed_tokens.weight"][torch.tensor(toks)]
    cos, sin = pl.rotation_tables(torch.arange(len(toks)), pl.inverse_frequencies(cfg["head_dim"], cfg["theta"], cfg["scaling"]))
    for i in range(cfg["layers"]):
        x = pl.decoder_layer(x, w, f"model.layers.{i}.", cfg, cos, sin)
    torch.testing.assert_close(full, pl.rms_norm(x, w["model.norm.weight"], cfg["eps"]) @ w["lm_head.weight"].T)
    swapped = {k.replace("layers.0.", "layers.X.").replace("layers.1.", "layers.0.").replace("layers.X.", "layers.1."): v for k, v in w.items()}
    assert not torch.allclose(pl.logits_of_sequence(swapped, cfg, toks), full, rtol=1e-3, atol=1e-4)


def test_processed_logprobs_vectors():
    """The vectors of the reference's tests/test_sampling.py:94-104."""
    torch.manual_seed(0)
    z = torch.randn(4, 50)
    torch.testing.assert_close(pl.processed_logprobs(z[0], 1.0, 0, 1.0), z[0].log_softmax(-1))
    torch.testing.assert_close(pl.processed_logprobs(z[3], 0.0, 0, 1.0), z[3].log_softmax(-1))  # greedy rows: scaled by 1
    lp = pl.processed_logprobs(z[1], 0.7, 5, 1.0)
    top5 = (z[1] / 0.7).topk(5)
    assert int((lp > -math.inf).sum()) == 5
    torch.testing.assert_close(lp[top5.indices], top5.values.log_softmax(-1))
    lp = pl.processed_logprobs(z[2], 1.0, 0, 0.8)
    srt = z[2].softmax(-1).sort(descending=True)
    keep = (srt.values.cumsum(-1) - srt.values) <= 0.8
    assert set((lp > -math.inf).nonzero().flatten().tolist()) == set(srt.indices[keep].tolist())


def test_draw_token():
    lp = torch.log(torch.tensor([0.0, 0.2, 0.0, 0.5, 0.3]))
    assert pl.draw_token(lp, 0.0) == 1       # u -> 0 gives the first token with probability > 0
    assert pl.draw_token(lp, 0.19) == 1 and pl.draw_token(lp, 0.21) == 3 and pl.draw_token(lp, 0.71) == 4
    assert pl.draw_token(lp, 1.0) == 4       # clamped to the last index
