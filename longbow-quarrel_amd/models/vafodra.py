"""The Vafodra decoder as a `ModelSpec`.

Every layer is a parallel block: one Dynamic Tanh norm whose output the mixer and the feed-forward both read,
x += residual_mult * (mixer + feed-forward).  A "parallel" layer's mixer is two mixers side by side (attention
over a sliding window that keeps the first tokens, with a sink and a gate per head, beside a Mamba-2 layer); a
"delta" layer's mixer is the gated delta rule.  The feed-forward is a gated linear unit with relu.  A layer that
names another layer's weights is one more run of that layer in the schedule, with a cache of its own.  The
embedding is scaled; the model's norm and an output head of its own follow the last layer.

Tensor names: `embed`, `head`, `final.norm`, and for layer i `l<i>.norm1`, `l<i>.mix.*`, `l<i>.mlp.*`; a
norm's bias and alpha are `<norm>.b` and `<norm>.alpha`.
"""
from __future__ import annotations

from ..config.vafodra import VafodraConfig, VafodraLayer
from ..model import ModelSpec, Run, token_table
from ..parts.base import PartSpec
from ..registry import register_architecture


def _mixer(cfg: VafodraConfig, layer: VafodraLayer, prefix: str) -> PartSpec:
    if layer.type == "delta":
        m = layer.delta
        return PartSpec("gated_delta", {
            "width": cfg.width, "heads": m.heads, "kv_heads": m.kv_heads, "key_dim": m.dim, "value_dim": m.vdim,
            "conv": m.conv, "eps": cfg.norm_eps, "prefix": prefix})
    a, s = layer.left, layer.right
    left = PartSpec("sink_window_attention", {
        "width": cfg.width, "heads": a.heads, "kv_heads": a.kv_heads, "key_dim": a.dim, "value_dim": a.vdim,
        "scale": a.scale, "window": a.window, "keep_first": a.keep_first, "sink": True, "head_gate": True,
        "prefix": prefix + ".left"})
    right = PartSpec("mamba2", {
        "width": cfg.width, "heads": s.heads, "head_dim": s.vdim, "state": s.state, "groups": s.groups,
        "conv": s.conv, "norm_groups": s.norm_groups, "eps": cfg.norm_eps, "prefix": prefix + ".right"})
    return PartSpec("side_by_side", {"width": cfg.width, "eps": cfg.norm_eps, "sides": (left, right),
                                     "out_names": (prefix + ".left.out", prefix + ".right.out")})


def vafodra_spec(cfg: VafodraConfig) -> ModelSpec:
    blocks, block_of = [], {}
    for i, layer in enumerate(cfg.layers):
        if layer.weights_of is not None:
            continue
        p = f"l{i}"
        block_of[i] = len(blocks)
        blocks.append(PartSpec("parallel", {
            "mixer": _mixer(cfg, layer, p + ".mix"),
            "feed_forward": None if layer.ff is None else PartSpec("glu", {
                "width": cfg.width, "inner": layer.ff, "prefix": p + ".mlp", "activation": "relu"}),
            "norm": PartSpec("dynamic_tanh", {"width": cfg.width, "name": p + ".norm1"}),
            "scale": cfg.residual_mult,
        }))
    schedule = tuple(Run(block_of[i if layer.weights_of is None else layer.weights_of])
                     for i, layer in enumerate(cfg.layers))
    return ModelSpec(
        vocab_size=cfg.vocab,
        width=cfg.width,
        embedding=token_table("embed", cfg.vocab, cfg.width, scale=cfg.embedding_scale),
        layers=tuple(blocks),
        schedule=schedule,
        final_norm=PartSpec("dynamic_tanh", {"width": cfg.width, "name": "final.norm"}),
        head_name="head",
        tie_head=False,
        max_positions=None,  # nothing in the design depends on a longest sequence
    )


register_architecture("Vafodra", VafodraConfig, vafodra_spec)
