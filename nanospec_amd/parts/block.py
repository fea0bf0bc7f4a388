"""The pre-norm residual block (reference: model/llama.py:198-208):
    x = x + mixer(norm1(x));  x = x + feed_forward(norm2(x)).

The stream is carried as ``resid`` plus a ``delta`` that has not been added yet, so that every sum is
done inside the norm kernel that follows it (the reference's fused form, model/llama.py:240-254)."""

from __future__ import annotations

from . import registry

_MIXER_PREFIX = {"attention": "self_attn."}
_FFN_PREFIX = {"swiglu": "mlp."}


class PreNormBlock:
    def __init__(self, spec, prefix: str | None = None) -> None:
        p = spec.prefix if prefix is None else prefix
        self.spec = spec
        self.mixer_norm = registry.build("norm", spec.mixer_norm, p + "input_layernorm.weight")
        self.mixer = registry.build("mixer", spec.mixer, p + _MIXER_PREFIX.get(spec.mixer.kind, spec.mixer.kind + "."))
        self.ffn_norm = registry.build("norm", spec.ffn_norm, p + "post_attention_layernorm.weight")
        self.ffn = registry.build("ffn", spec.ffn, p + _FFN_PREFIX.get(spec.ffn.kind, spec.ffn.kind + "."))
        self.parts = (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn)

    @property
    def graph_safe(self) -> bool:
        return all(getattr(p, "graph_safe", False) for p in self.parts)

    def wanted(self) -> dict:
        out = {}
        for p in self.parts:
            out.update(p.wanted())
        return out

    def load(self, get, dtype, device) -> None:
        for p in self.parts:
            p.load(get, dtype, device)

    def cache_need(self):
        return self.mixer.cache_need()

    def forward(self, ctx, resid, delta, cache, owns_cache, delta_out) -> None:
        mark = ctx.arena.mark()
        h = self.mixer_norm.forward(ctx, resid=resid, x=delta, write_resid=delta is not None,
                                    out=ctx.arena.take(resid.shape, resid.dtype))
        a = self.mixer.forward(ctx, h, cache, owns_cache, out=ctx.arena.take(resid.shape, resid.dtype))
        h2 = self.ffn_norm.forward(ctx, resid=resid, x=a, write_resid=True, out=h)
        self.ffn.forward(ctx, h2, out=delta_out)
        ctx.arena.release(mark)


registry.register("block", "prenorm", PreNormBlock)
