"""The Gulidra decoder described with parts (config.json "architecture": "Gulidra").

Token rows times a scale plus learned position vectors; every layer adds its sublayers' outputs through an RMS norm
and a constant factor (the sublayers read the residual itself); a layer's mixer is a differential attention whose
projections pass a short causal convolution (optionally reading the keys and values of an earlier layer) or a linear
attention with a decay per head and a matrix of state; its feed-forward is a gated unit, routed experts (some of them
identities), or none; final norm and head.  Tensor names: `embed`, `pos`, `l<i>.norm1|norm2`, `l<i>.mix.q|k|v|g|o`
(+ `.conv`, `.norm`), `l<i>.mix.lq1|lk1|lq2|lk2`, `l<i>.mix.norm`, `l<i>.mlp.gate|up|down`,
`l<i>.mlp.router|correction`, `l<i>.mlp.e<j>.gate|up|down`, `final.norm`, `head`."""
from __future__ import annotations

from ..config.gulidra import GulidraAttention, GulidraConfig, GulidraDense
from ..parts.spec import BlockSpec, ModelSpec, PartSpec, PlanEntry
from . import ARCHITECTURES, Architecture


def gulidra_spec(cfg: GulidraConfig) -> ModelSpec:
    D = cfg.width
    blocks, plan = [], []
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        if isinstance(m, GulidraAttention):
            mixer = PartSpec("differential_attention", dict(
                hidden_size=D, num_heads=m.heads, num_kv_heads=m.kv_heads, key_dim=m.dim, value_dim=m.vdim,
                scale=m.scale, diff=m.diff, conv_taps=m.conv, norm_eps=cfg.eps, head_gate=True,
                shares_kv=m.kv_from is not None), "mix.")
            cache_of = m.kv_from
        else:
            mixer = PartSpec("decay_linear_attention", dict(
                hidden_size=D, num_heads=m.heads, key_dim=m.dim, value_dim=m.vdim, decay=m.decay, norm_eps=cfg.eps,
                activation="silu", gate=True), "mix.")
            cache_of = None
        parts = {"mixer": mixer,
                 "mixer_norm": PartSpec("rmsnorm", dict(size=D, eps=cfg.eps, name="norm1")),
                 "scale": PartSpec("scaled", dict(mult=cfg.residual_mult))}
        f = layer.mlp
        if f is not None:
            parts["ffn_norm"] = PartSpec("rmsnorm", dict(size=D, eps=cfg.eps, name="norm2"))
            if isinstance(f, GulidraDense):
                parts["ffn"] = PartSpec("swiglu", dict(hidden_size=D, intermediate_size=f.ff,
                                                       names=dict(gate="gate", up="up", down="down")), "mlp.")
            else:
                parts["ffn"] = PartSpec("routed_experts", dict(
                    hidden_size=D, intermediate_size=f.ff, experts=f.experts, identity=f.identity, top=f.top,
                    correction=True, renormalize=False), "mlp.")
        blocks.append(BlockSpec(arrangement="sublayer_norm", weight_prefix=f"l{i}.", parts=parts))
        plan.append(PlanEntry(i, cache_of=cache_of))
    return ModelSpec(
        hidden_size=D,
        vocab_size=cfg.vocab,
        max_positions=cfg.max_positions,
        embedding=PartSpec("token_table_positions", dict(vocab_size=cfg.vocab, hidden_size=D,
                                                         max_positions=cfg.max_positions, scale=cfg.embedding_scale,
                                                         table_name="embed", positions_name="pos")),
        blocks=blocks,
        plan=plan,
        final_norm=PartSpec("rmsnorm", dict(size=D, eps=cfg.eps, name="final.norm")),
        head=PartSpec("linear", dict(vocab_size=cfg.vocab, hidden_size=D, name="head")),
    )


ARCHITECTURES.register("Gulidra", Architecture("gulidra", GulidraConfig.from_dict, gulidra_spec))
