"""Configurations at the edges of what the kernels take: head sizes in steps of 16 up to 256 (and one that is no multiple of
16), widths and feed-forward sizes that are no multiple of 8 or of anything, vocabularies that are no power of two,
one head, seven heads, ten query heads to a key/value head.  Every one must give the plain implementation's logits, in
32-bit and in bfloat16, decoded token by token and in a mixed schedule, or be refused with a clear error: never a wrong
result."""

from __future__ import annotations

import pytest
import torch

import plain_llama as pl
import traces
from tiny import random_tokens, ulps_of_row_max

pytestmark = pytest.mark.gpu


def cfg(**kw):
    base = dict(architectures=["LlamaForCausalLM"], model_type="llama", rms_norm_eps=1e-5, rope_theta=10000.0,
                max_position_embeddings=512, tie_word_embeddings=False)
    base.update(kw)
    return base


CONFIGS = {
    # a width that is no multiple of 8 (no matrix-core product takes it), as many key/value heads as heads, head size 48
    "width100_heads5x48": cfg(vocab_size=257, hidden_size=100, intermediate_size=90, num_hidden_layers=1, num_attention_heads=5,
                              num_key_value_heads=5, head_dim=48),
    "mqa_3x80_tied": cfg(vocab_size=511, hidden_size=72, intermediate_size=200, num_hidden_layers=2, num_attention_heads=3,
                         num_key_value_heads=1, head_dim=80, tie_word_embeddings=True),
    "head256": cfg(vocab_size=300, hidden_size=128, intermediate_size=384, num_hidden_layers=1, num_attention_heads=2,
                   num_key_value_heads=1, head_dim=256),
    "width33_heads7x16": cfg(vocab_size=129, hidden_size=33, intermediate_size=47, num_hidden_layers=1, num_attention_heads=7,
                             num_key_value_heads=7, head_dim=16),
    "mqa_5x144_eps1e-6": cfg(vocab_size=777, hidden_size=144, intermediate_size=300, num_hidden_layers=2, num_attention_heads=5,
                             num_key_value_heads=1, head_dim=144, rms_norm_eps=1e-6),
    "heads12over4x96": cfg(vocab_size=1001, hidden_size=200, intermediate_size=344, num_hidden_layers=2, num_attention_heads=12,
                           num_key_value_heads=4, head_dim=96),
    "group_of_ten": cfg(vocab_size=640, hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=20,
                        num_key_value_heads=2, head_dim=32),
    # a head size that is no multiple of 16: the matrix-core attention does not take it, the plain kernel does
    "head24": cfg(vocab_size=90, hidden_size=96, intermediate_size=136, num_hidden_layers=1, num_attention_heads=4,
                  num_key_value_heads=2, head_dim=24),
    "llama3_scaling_16x64": cfg(vocab_size=4099, hidden_size=1024, intermediate_size=2816, num_hidden_layers=2, num_attention_heads=16,
                                num_key_value_heads=16, head_dim=64, rope_theta=500000.0,
                                rope_scaling=dict(rope_type="llama3", factor=4.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                                  original_max_position_embeddings=32)),
}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    from nanospec_amd.config import LlamaConfig
    from nanospec_amd.weights import write_model_folder

    base = tmp_path_factory.mktemp("sizes")
    return {name: write_model_folder(base / name, LlamaConfig.from_hf(c), 7, torch.float32) for name, c in CONFIGS.items()}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("name", list(CONFIGS))
def test_odd_sizes_match_plain(folders, name, dtype):
    from nanospec_amd.engine.replay import Replayer
    from nanospec_amd.loader import load_model

    folder = folders[name]
    vocab = CONFIGS[name]["vocab_size"]
    seqs = {f"r{i}": random_tokens(n, vocab, 10 * i + n) for i, n in enumerate((3, 40, 77, 130))}
    pcfg, w = pl.read_config(folder), pl.read_weights(folder, dtype)
    ref = {rid: pl.logits_of_sequence(w, pcfg, t, dtype) for rid, t in seqs.items()}
    model = load_model(folder, dtype=dtype)
    mixed_steps, mixed_where, peak = traces.mixed(seqs, seed=5)
    for what, (steps, where), room in (("tail", traces.tail_decoded(seqs), 512), ("mixed", (mixed_steps, mixed_where), peak)):
        rep = Replayer(model, room, page_size=16)
        for step, wh in zip(steps, where):
            out = rep.step(step["entries"], step["end"])
            if not wh:
                continue
            want = torch.stack([ref[rid][p] for rid, p in wh])
            assert torch.isfinite(out).all()
            if dtype == torch.float32:
                err = ((out - want).abs().amax(-1) / want.abs().amax(-1)).max().item()
                assert err <= 1e-4, f"{name} {what} step {step['step']}: {err:.2e} of the row's largest logit"
            else:
                u = ulps_of_row_max(out, want).max().item()
                assert u <= 8, f"{name} {what} step {step['step']}: {u:.2f} bf16 ulps of the row's largest logit"
        rep.manager.check()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_a_head_size_beyond_the_kernels_is_refused(tmp_path, dtype):
    """Heads of 272 channels: no attention kernel takes them.  The step raises with the reason; nothing is computed elsewhere."""
    from nanospec_amd.config import LlamaConfig
    from nanospec_amd.engine.replay import Replayer
    from nanospec_amd.kernels.ops import KernelRefused
    from nanospec_amd.loader import load_model
    from nanospec_amd.weights import write_model_folder

    c = cfg(vocab_size=50, hidden_size=64, intermediate_size=96, num_hidden_layers=1, num_attention_heads=1, num_key_value_heads=1, head_dim=272)
    folder = write_model_folder(tmp_path / "wide_head", LlamaConfig.from_hf(c), 1, torch.float32)
    rep = Replayer(load_model(folder, dtype=dtype), 64, page_size=16)
    with pytest.raises(KernelRefused, match="256"):
        rep.step([{"id": "a", "tokens": [1, 2, 3], "want": [2]}], [])
