"""The Risizen decoder described with parts (config.json "architecture": "Risizen").

Token rows through an RMS norm into S residual streams; every layer reads the streams with learned weights, runs an
attention whose projections pass a short causal convolution (unit-norm q and k, no rotation, a mask of chunks counted
from position 0, a softmax with a sink, keys and values of different sizes, optionally the keys and values of an
earlier layer) and a clamped gated feed-forward, and writes each output back into all streams; the sum of the streams
goes through the final norm and a head whose logits are scaled.  Tensor names: `embed`, `embed.norm`,
`l<i>.norm1|norm2`, `l<i>.mix.q|k|v|o` (+ `.b`, `.conv`), `l<i>.mlp.gate|up|down`, `l<i>.hc1|hc2.in|out|mix`,
`final.norm`, `head`."""
from __future__ import annotations

from ..config.risizen import DEFAULT_MAX_POSITIONS, RisizenConfig
from ..parts.spec import BlockSpec, ModelSpec, PartSpec, PlanEntry
from . import ARCHITECTURES, Architecture


def risizen_spec(cfg: RisizenConfig) -> ModelSpec:
    D, S = cfg.width, cfg.streams
    blocks, plan = [], []
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        link = dict(streams=S, optional_weights=not cfg.has_stream_weights)
        parts = {
            "mixer_norm": PartSpec("rmsnorm", dict(size=D, eps=cfg.eps, name="norm1")),
            "mixer": PartSpec("conv_attention", dict(
                hidden_size=D, num_heads=m.heads, num_kv_heads=m.kv_heads, key_dim=m.dim, value_dim=m.vdim,
                scale=m.scale, conv_taps=m.conv, unit_norm=True, norm_eps=cfg.eps, bias=True,
                mask="chunk" if m.chunk else "causal", mask_size=m.chunk or 0, sink=True,
                shares_kv=m.kv_from is not None), "mix."),
            "mixer_link": PartSpec("hyper", link, "hc1."),
        }
        if layer.mlp is not None:
            parts["ffn_norm"] = PartSpec("rmsnorm", dict(size=D, eps=cfg.eps, name="norm2"))
            parts["ffn"] = PartSpec("clamped_glu", dict(hidden_size=D, intermediate_size=layer.mlp.ff,
                                                        limit=layer.mlp.limit, alpha=1.702), "mlp.")
            parts["ffn_link"] = PartSpec("hyper", link, "hc2.")
        blocks.append(BlockSpec(arrangement="hyper_pre_norm", weight_prefix=f"l{i}.", parts=parts))
        plan.append(PlanEntry(i, cache_of=m.kv_from))
    return ModelSpec(
        hidden_size=D,
        vocab_size=cfg.vocab,
        max_positions=DEFAULT_MAX_POSITIONS,
        embedding=PartSpec("token_table_norm", dict(vocab_size=cfg.vocab, hidden_size=D, eps=cfg.eps, streams=S,
                                                    table_name="embed", norm_name="embed.norm")),
        blocks=blocks,
        plan=plan,
        final_norm=PartSpec("rmsnorm", dict(size=D, eps=cfg.eps, name="final.norm")),
        head=PartSpec("linear", dict(vocab_size=cfg.vocab, hidden_size=D, scale=cfg.logit_scale, name="head")),
        streams=S,
    )


ARCHITECTURES.register("Risizen", Architecture("risizen", RisizenConfig.from_dict, risizen_spec))
