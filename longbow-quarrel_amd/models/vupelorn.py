"""The Vupelorn decoder as a `ModelSpec`.

Every layer normalises what its sublayers return, not what they read: x += norm1(mixer(x)); x += norm2(ffn(x)).
A "gla" layer's mixer is gated linear attention; a "latent_attention" layer's is attention through a cached latent
with half-split rotary pairs under YaRN scaling, a "latent_attention_2" layer's the same with interleaved pairs and
plain frequencies, optionally reading the latent rows that an earlier layer cached (`kv_from`: that layer's run of
the schedule lends its cache).  The feed-forward is a mixture of experts whose router weights multiply the experts'
inputs.  The embedding adds a hashed bigram row; the model's norm is an RMS norm and the head is the embedding.

Tensor names: `embed`, `bigram`, `final.norm`, and for layer i `l<i>.norm1`, `l<i>.norm2`, `l<i>.mix.*`,
`l<i>.mlp.router`, `l<i>.mlp.e<j>.gate|up|down`.
"""
from __future__ import annotations

from ..config.base import ConfigError
from ..config.vupelorn import VupelornConfig, VupelornLayer
from ..model import ModelSpec, Run, token_table
from ..parts.base import PartSpec
from ..registry import register_architecture


def _mixer(cfg: VupelornConfig, layer: VupelornLayer, i: int) -> PartSpec:
    prefix = f"l{i}.mix"
    if layer.gla is not None:
        m = layer.gla
        if m.decay_rank is None:
            raise ConfigError(f"layers[{i}].mixer: the decay's rank is in no key; a model file's tensor shapes give "
                              "it (or state 'decay_rank')")
        return PartSpec("gated_linear_attention", {
            "width": cfg.width, "heads": m.heads, "key_dim": m.dim, "value_dim": m.vdim, "decay_rank": m.decay_rank,
            "tau": m.tau, "eps": cfg.norm_eps, "prefix": prefix})
    m = layer.latent
    scaling = None
    if m.rot.scaling is not None:
        sc = m.rot.scaling
        scaling = {"rope_type": "yarn", "factor": sc.factor, "original": sc.original, "fast": sc.fast, "slow": sc.slow}
    return PartSpec("latent_attention", {
        "width": cfg.width, "heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "value_dim": m.vdim,
        "kv_rank": m.kv_rank, "q_rank": m.q_rank, "scale": m.scale, "eps": cfg.norm_eps, "rot_base": m.rot.base,
        "rot_dims": m.rot.dims, "rot_scaling": scaling,
        "pairing": "interleaved" if layer.type == "latent_attention_2" else "half",
        "own_kv": m.kv_from is None, "prefix": prefix})


def vupelorn_spec(cfg: VupelornConfig) -> ModelSpec:
    blocks, schedule = [], []
    for i, layer in enumerate(cfg.layers):
        ffn = None
        ffn_norm = PartSpec("rmsnorm", {"width": cfg.width, "eps": cfg.norm_eps, "name": f"l{i}.norm2"})
        if layer.mlp is not None:
            e = layer.mlp
            ffn = PartSpec("moe", {"width": cfg.width, "experts": e.experts, "top": e.top, "inner": e.ff,
                                   "limit": e.limit, "prefix": f"l{i}.mlp", "weight_input": True})
        blocks.append(PartSpec("output_norm", {
            "mixer": _mixer(cfg, layer, i),
            "mixer_norm": PartSpec("rmsnorm", {"width": cfg.width, "eps": cfg.norm_eps, "name": f"l{i}.norm1"}),
            "feed_forward": ffn, "ffn_norm": ffn_norm}))
        # layers and runs of the schedule count alike here: a layer that reads another's latent reads that run's cache
        schedule.append(Run(i, cache_of=None if layer.latent is None else layer.latent.kv_from))
    if cfg.bigram is None:
        embedding = token_table("embed", cfg.vocab, cfg.width)
    else:
        b = cfg.bigram
        embedding = PartSpec("token_bigram_table", {
            "name": "embed", "vocab_size": cfg.vocab, "width": cfg.width, "bigram_name": "bigram",
            "buckets": b.buckets, "mul_prev": b.mul_prev, "mul_cur": b.mul_cur})
    return ModelSpec(
        vocab_size=cfg.vocab, width=cfg.width, embedding=embedding, layers=tuple(blocks), schedule=tuple(schedule),
        final_norm=PartSpec("rmsnorm", {"width": cfg.width, "eps": cfg.norm_eps, "name": "final.norm"}),
        head_name=None, tie_head=True,
        max_positions=None,  # nothing in the design depends on a longest sequence
    )


register_architecture("Vupelorn", VupelornConfig, vupelorn_spec)
