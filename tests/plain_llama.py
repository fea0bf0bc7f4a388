"""A plain, slow Llama 3 dense decoder: whole sequences, no cache, one function per part.

This file is the oracle of the test-suite.  It shares no code with ``nanospec_amd``: it reads
``config.json`` and ``model.safetensors`` by itself, and every function is written from the
formula that the reference implementation computes (cited as ``file:line`` of
ved1beta/nanospec).  Everything runs on the CPU with torch tensor arithmetic only.

``dtype`` is the storage precision of weights and of the values that pass from one part to
the next.  In ``torch.float32`` nothing is rounded anywhere.  In ``torch.bfloat16`` weights
and the outputs of the parts are rounded to bfloat16 while the inside of each part (norm
statistics, rotation angles, soft-max, accumulation of dot products, the residual sum) is
computed in 32-bit and rounded once, which is what a kernel with 32-bit accumulators does.
"""

from __future__ import annotations

import json
import math
import struct
from pathlib import Path

import torch

# --------------------------------------------------------------------------- files


def read_config(folder) -> dict:
    """config.json as the sizes and constants this file needs.

    Keys and defaults as parsed by the reference, model/llama.py:39-78: ``num_key_value_heads``
    defaults to the number of heads (:69), ``head_dim`` to ``hidden_size // heads`` (:70),
    ``rms_norm_eps`` to 1e-5 (:71), ``rope_theta`` to 10000 (:48); the rope dictionary is
    either ``rope_parameters`` or ``rope_scaling`` and its kind either ``rope_type`` or
    ``type`` (:47-55)."""
    raw = json.loads((Path(folder) / "config.json").read_text())
    heads = raw["num_attention_heads"]
    rope = dict(raw.get("rope_parameters") or raw.get("rope_scaling") or {})
    theta = float(rope.pop("rope_theta", raw.get("rope_theta", 10000.0)))
    kind = rope.pop("rope_type", rope.pop("type", "default"))
    return {
        "vocab": raw["vocab_size"],
        "hidden": raw["hidden_size"],
        "inter": raw["intermediate_size"],
        "layers": raw["num_hidden_layers"],
        "heads": heads,
        "kv_heads": raw.get("num_key_value_heads", heads),
        "head_dim": raw.get("head_dim") or raw["hidden_size"] // heads,
        "eps": raw.get("rms_norm_eps", 1e-5),
        "theta": theta,
        "scaling": rope if kind == "llama3" else None,
        "tied": bool(raw.get("tie_word_embeddings", False)),
    }


_ST_DTYPES = {"F32": torch.float32, "BF16": torch.bfloat16, "F16": torch.float16, "I32": torch.int32, "I64": torch.int64}


def read_safetensors(path) -> dict[str, torch.Tensor]:
    """The safetensors container: 8 bytes little-endian header length, a JSON header with
    dtype / shape / byte offsets per tensor name, then the raw bytes."""
    blob = Path(path).read_bytes()
    (n,) = struct.unpack("<Q", blob[:8])
    header = json.loads(blob[8 : 8 + n])
    base = 8 + n
    out = {}
    for name, info in header.items():
        if name == "__metadata__":
            continue
        lo, hi = info["data_offsets"]
        flat = torch.frombuffer(bytearray(blob[base + lo : base + hi]), dtype=_ST_DTYPES[info["dtype"]])
        out[name] = flat.reshape(info["shape"]).clone()
    return out


def read_weights(folder, dtype) -> dict[str, torch.Tensor]:
    """Every tensor of the folder cast to ``dtype`` (model/loader.py:56-60); a missing
    ``lm_head.weight`` means the head is the embedding table (model/loader.py:62-66)."""
    w = {k: v.to(dtype) for k, v in read_safetensors(Path(folder) / "model.safetensors").items()}
    if "lm_head.weight" not in w:
        w["lm_head.weight"] = w["model.embed_tokens.weight"]
    return w


# --------------------------------------------------------------------------- parts


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """model/llama.py:92-95: in 32-bit ``h = x * rsqrt(mean(x^2) + eps)``; h is cast back to the
    dtype of x BEFORE it is multiplied by the weight."""
    h = x.float()
    h = h * torch.rsqrt((h * h).mean(dim=-1, keepdim=True) + eps)
    return weight * h.to(x.dtype)


def inverse_frequencies(head_dim: int, theta: float, scaling: dict | None) -> torch.Tensor:
    """model/llama.py:98-118.  ``1 / theta^(2j/d)`` for j < d/2 (:101-102); with llama3 scaling
    a frequency whose wavelength is longer than ``P/low`` is divided by ``factor`` (:114), one
    between ``P/high`` and ``P/low`` is blended (:115-118), shorter ones stay."""
    j = torch.arange(0, head_dim, 2, dtype=torch.int64).float()
    inv = 1.0 / (theta ** (j / head_dim))
    if scaling is None:
        return inv
    factor, low, high = scaling["factor"], scaling["low_freq_factor"], scaling["high_freq_factor"]
    span = scaling["original_max_position_embeddings"]
    wavelen = 2 * math.pi / inv
    out = torch.where(wavelen > span / low, inv / factor, inv)
    blend = (span / wavelen - low) / (high - low)
    mixed = (1 - blend) * out / factor + blend * out
    medium = ~(wavelen < span / high) & ~(wavelen > span / low)
    return torch.where(medium, mixed, out)


def rotation_tables(positions: torch.Tensor, inv_freq: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """model/llama.py:133-136: angle[p, j] = p * inv_freq[j] in 32-bit, the half table repeated
    twice along the last axis; cos and sin of it.  [T, head_dim] each, 32-bit."""
    ang = torch.outer(positions.float(), inv_freq)
    ang = torch.cat((ang, ang), dim=-1)
    return ang.cos(), ang.sin()


def rotate(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """model/llama.py:150-158: element j is paired with element j + d/2 (half-split, not
    interleaved): ``x*cos + cat(-x[d/2:], x[:d/2])*sin``.  x: [T, heads, d]; cos, sin: [T, d].
    Computed in 32-bit from 32-bit angles and rounded once to the dtype of x."""
    half = x.shape[-1] // 2
    xf = x.float()
    swapped = torch.cat((-xf[..., half:], xf[..., :half]), dim=-1)
    return (xf * cos[:, None, :] + swapped * sin[:, None, :]).to(x.dtype)


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, first_query: int = 0) -> torch.Tensor:
    """model/attention.py:22-43.  q: [Tq, heads, d], k and v: [Tk, kv_heads, d].  Query row i is the
    token at position ``first_query + i`` and sees keys 0..first_query+i (the reference's
    explicit mask ``kpos <= qpos``, :38-41; with Tq == Tk it is the plain causal mask, :37).  Scores
    are scaled by 1/sqrt(d), the default of the library routine the reference calls (:33-41).
    Query head h reads key/value head ``h // (heads / kv_heads)`` (``enable_gqa``, :33)."""
    tq, heads, d = q.shape
    tk, kv_heads, _ = k.shape
    group = heads // kv_heads
    kf = k.float().repeat_interleave(group, dim=1)  # [Tk, heads, d]
    vf = v.float().repeat_interleave(group, dim=1)
    scores = torch.einsum("qhd,khd->hqk", q.float(), kf) / math.sqrt(d)
    qpos = torch.arange(first_query, first_query + tq)[:, None]
    kpos = torch.arange(tk)[None, :]
    scores = scores.masked_fill(~(kpos <= qpos), float("-inf"))
    probs = torch.softmax(scores, dim=-1)
    return torch.einsum("hqk,khd->qhd", probs, vf).to(q.dtype)


def linear(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """``x @ W^T`` without bias (model/llama.py:168-171,190-192); W is [out, in].  The sum is
    accumulated in 32-bit and rounded once."""
    return (x.float() @ weight.float().T).to(x.dtype)


def swiglu(x: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor) -> torch.Tensor:
    """model/llama.py:195: ``down(silu(gate(x)) * up(x))`` with silu(g) = g * sigmoid(g).  The
    product silu(g)*u is formed in 32-bit from the two 32-bit sums and rounded once."""
    g = x.float() @ gate.float().T
    u = x.float() @ up.float().T
    act = (g * torch.sigmoid(g) * u).to(x.dtype)
    return linear(act, down)


def residual_add(x: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
    """model/llama.py:207-208: the stream plus the part's output, summed in 32-bit."""
    return (x.float() + y.float()).to(x.dtype)


# --------------------------------------------------------------------------- the model


def decoder_layer(x, w, prefix, cfg, cos, sin):
    """model/llama.py:206-208: ``x + attn(norm1(x))`` then ``x + mlp(norm2(x))``; inside the
    attention (:175-184) q, k, v projections, rotation of q and k (v untouched), soft-max
    attention, output projection."""
    t = x.shape[0]
    h = rms_norm(x, w[prefix + "input_layernorm.weight"], cfg["eps"])
    q = linear(h, w[prefix + "self_attn.q_proj.weight"]).view(t, cfg["heads"], cfg["head_dim"])
    k = linear(h, w[prefix + "self_attn.k_proj.weight"]).view(t, cfg["kv_heads"], cfg["head_dim"])
    v = linear(h, w[prefix + "self_attn.v_proj.weight"]).view(t, cfg["kv_heads"], cfg["head_dim"])
    q, k = rotate(q, cos, sin), rotate(k, cos, sin)
    a = causal_attention(q, k, v).reshape(t, -1)
    x = residual_add(x, linear(a, w[prefix + "self_attn.o_proj.weight"]))
    h = rms_norm(x, w[prefix + "post_attention_layernorm.weight"], cfg["eps"])
    m = swiglu(h, w[prefix + "mlp.gate_proj.weight"], w[prefix + "mlp.up_proj.weight"], w[prefix + "mlp.down_proj.weight"])
    return residual_add(x, m)


def logits_of_sequence(w: dict, cfg: dict, tokens: list[int], dtype=torch.float32) -> torch.Tensor:
    """Logits at every position of one whole sequence, [T, vocab] in 32-bit.  model/llama.py:221-232
    (embedding row, the layers, the last norm) and :286 (the head), engine/engine.py:382 (logits are
    taken to 32-bit)."""
    ids = torch.tensor(tokens, dtype=torch.int64)
    x = w["model.embed_tokens.weight"][ids].to(dtype)
    inv = inverse_frequencies(cfg["head_dim"], cfg["theta"], cfg["scaling"])
    cos, sin = rotation_tables(torch.arange(len(tokens)), inv)
    for i in range(cfg["layers"]):
        x = decoder_layer(x, w, f"model.layers.{i}.", cfg, cos, sin)
    x = rms_norm(x, w["model.norm.weight"], cfg["eps"])
    return x.float() @ w["lm_head.weight"].float().T


def greedy_continuation(w: dict, cfg: dict, prompt: list[int], n_new: int, dtype=torch.float32) -> tuple[list[int], torch.Tensor]:
    """tests/decode.py:12-39 without a cache: the arg-max of the last position's logits is appended
    and the whole sequence is run again.  -> (new tokens, the logits each was chosen from)."""
    seq, rows = list(prompt), []
    for _ in range(n_new):
        row = logits_of_sequence(w, cfg, seq, dtype)[-1]
        rows.append(row)
        seq.append(int(row.argmax()))
    return seq[len(prompt) :], torch.stack(rows)


# --------------------------------------------------------------------------- sampling


def processed_logprobs(z: torch.Tensor, temperature: float, top_k: int, top_p: float) -> torch.Tensor:
    """spec/sampling.py:24-35 for one row of 32-bit logits.  Divide by the temperature (a
    temperature of 0 divides by 1, :28); sort descending; keep the tokens whose EXCLUSIVE cumulative
    probability is <= top_p (:31) and, if top_k > 0, only the first top_k (:32); log-soft-max of
    what is kept, -inf elsewhere (:33-35)."""
    z = z.float() / (temperature if temperature > 0 else 1.0)
    if top_k > 0 or top_p < 1.0:
        order = torch.argsort(z, descending=True, stable=True)
        p = torch.softmax(z[order], dim=-1)
        keep = (torch.cumsum(p, -1) - p) <= top_p
        if top_k > 0:
            keep &= torch.arange(z.numel()) < top_k
        masked = torch.full_like(z, float("-inf"))
        masked[order[keep]] = z[order[keep]]
        z = masked
    return torch.log_softmax(z, dim=-1)


def draw_token(logprobs: torch.Tensor, u: float) -> int:
    """spec/sampling.py:38-42 with no proposal mass: cumulative sum of exp(logprobs) in vocabulary
    order; the first index whose cumulative value exceeds ``u * total`` (searchsorted right),
    clamped to the last index."""
    cdf = torch.cumsum(logprobs.exp(), -1)
    idx = int(torch.searchsorted(cdf, torch.tensor([u * float(cdf[-1])], dtype=cdf.dtype), right=True))
    return min(idx, logprobs.numel() - 1)
