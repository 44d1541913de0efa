"""Attention whose keys and values are made from a cached latent (DeepSeek-AI: "DeepSeek-V2: A Strong, Economical,
and Efficient Mixture-of-Experts Language Model", its multi-head latent attention).

Per position the cache holds one row: the latent c = rmsnorm(first `kv_rank` rows of Wdkv h) and one rotated key
part of `rot_dim` entries that all heads share (the last rows of Wdkv h, rotated, not normed).  Queries go through
a latent as well: cq = rmsnorm(Wdq h), q = Wuq cq, head by head [`dim` unrotated | `rot_dim` rotated].  Head n's
unrotated key is Wuk_n c and its value Wuv_n c; score = (q_unrot . k_unrot + q_rot . k_rot) * scale, causal, an
ordinary softmax; the heads' results, concatenated, go through Wo.

Keys and values are never made per head.  With a_n = Wuk_n^T q_unrot (a vector of `kv_rank` entries),
q_unrot . (Wuk_n c) = a_n . c, and sum_t p_t (Wuv_n c_t) = Wuv_n (sum_t p_t c_t): every head asks the one cached
row [c | k_rot] with the query [a_n | q_rot] and gets a weighted mean of latents, which Wuv_n then lifts.  That is
attention with one key/value head whose value is the front of its key, and runs on the library's paged attention
kernel for keys and values of different sizes (scores, probabilities and sums in 32-bit).

The rotation takes the first `rot_dims` entries of the rotated part (the rest pass), in half-split pairs
(i, i + rot_dims / 2) or interleaved pairs (2 i, 2 i + 1); angles are position times a frequency table made once in
float64 (`rope.rotary_frequencies`, which knows the scalings), cos and sin times `rope.rotary_magnitude`.

A layer may read the rows that another run of the schedule cached (`own_kv=False`; the schedule's `cache_of` names
the run): it then has no Wdkv and uses its own Wuk, Wuv, queries and output projection.
"""
from __future__ import annotations

from typing import Dict, List, Mapping, Optional

import torch

from .base import (MIXERS, VECTOR32, BuildEnv, KVNeed, LayerCache, Mixer, StepContext, TensorSpec, product_weight,
                   project)
from .rope import rotary_frequencies, rotary_magnitude
from .sink_attention import split_scratch


def _round8(n: int) -> int:
    return (n + 7) // 8 * 8


@MIXERS.register("latent_attention")
class LatentAttention(Mixer):
    graph_safe = True
    takes_out = True

    def __init__(self, width: int, heads: int, dim: int, rot_dim: int, value_dim: int, kv_rank: int, q_rank: int,
                 scale: float, eps: float, rot_base: float, prefix: str, rot_dims: Optional[int] = None,
                 rot_scaling: Optional[Mapping] = None, pairing: str = "half", own_kv: bool = True,
                 names: Optional[Mapping[str, str]] = None) -> None:
        if pairing not in ("half", "interleaved"):
            raise ValueError(f"rotary pairing {pairing!r} is not known (known: 'half', 'interleaved')")
        self.width, self.heads, self.dim, self.rot_dim = int(width), int(heads), int(dim), int(rot_dim)
        self.value_dim, self.kv_rank, self.q_rank = int(value_dim), int(kv_rank), int(q_rank)
        self.scale, self.eps, self.pairing, self.own_kv = float(scale), float(eps), pairing, bool(own_kv)
        self.rot_dims = self.rot_dim if rot_dims is None else int(rot_dims)
        if self.rot_dims % 2 or not 2 <= self.rot_dims <= self.rot_dim:
            raise ValueError(f"{self.rot_dims} rotated entries do not fit a rotated part of {self.rot_dim}")
        self.freq_table = rotary_frequencies(self.rot_dims, float(rot_base), dict(rot_scaling) if rot_scaling else None)
        self.magnitude = rotary_magnitude(rot_scaling)
        self.key_dim = self.kv_rank + self.rot_dim  # a cached row, and a head's query after the fold
        n = {"dq": "dq", "dq_norm": "dq.norm", "uq": "uq", "dkv": "dkv", "dkv_norm": "dkv.norm", "uk": "uk", "uv": "uv",
             "o": "o"}
        n.update(names or {})
        self.names: Dict[str, str] = {key: f"{prefix}.{val}" for key, val in n.items()}

    def tensor_specs(self) -> List[TensorSpec]:
        nm, H = self.names, self.heads
        specs = [
            TensorSpec(nm["dq"], (self.q_rank, self.width)),
            TensorSpec(nm["dq_norm"], (self.q_rank,), kind=VECTOR32, init="around_one"),
            TensorSpec(nm["uq"], (H * (self.dim + self.rot_dim), self.q_rank)),
        ]
        if self.own_kv:
            specs += [TensorSpec(nm["dkv"], (self.kv_rank + self.rot_dim, self.width)),
                      TensorSpec(nm["dkv_norm"], (self.kv_rank,), kind=VECTOR32, init="around_one")]
        return specs + [
            TensorSpec(nm["uk"], (H * self.dim, self.kv_rank)),
            TensorSpec(nm["uv"], (H * self.value_dim, self.kv_rank)),
            TensorSpec(nm["o"], (self.width, H * self.value_dim)),
        ]

    def bind(self, tensors: Mapping[str, torch.Tensor], env: BuildEnv) -> None:
        super().bind(tensors, env)
        nm, H = self.names, self.heads
        down = [tensors[nm["dq"]]] + ([tensors[nm["dkv"]]] if self.own_kv else [])
        if len({m.dtype for m in down}) != 1:
            raise ValueError(f"{nm['dq']}: the projections of one input are stored in different dtypes")
        self.w_down = product_weight(env, torch.cat(down, dim=0))  # [dq | dkv]
        self.q_norm_w = tensors[nm["dq_norm"]].contiguous()
        self.kv_norm_w = tensors[nm["dkv_norm"]].contiguous() if self.own_kv else None
        uq = tensors[nm["uq"]].reshape(H, self.dim + self.rot_dim, self.q_rank)
        # the heads' unrotated rows first, then their rotated rows: two products, each with the result it feeds
        self.w_uq_plain = product_weight(env, uq[:, : self.dim].reshape(H * self.dim, self.q_rank).contiguous())
        self.w_uq_rot = product_weight(env, uq[:, self.dim :].reshape(H * self.rot_dim, self.q_rank).contiguous())
        # head n's Wuk_n^T [kv_rank, dim]: the weight of the product that folds the key's lift into the query
        self.w_uk_t = tensors[nm["uk"]].reshape(H, self.dim, self.kv_rank).transpose(1, 2).contiguous()
        self.w_uv = tensors[nm["uv"]].reshape(H, self.value_dim, self.kv_rank).contiguous()
        self.w_o = product_weight(env, tensors[nm["o"]])
        self.freqs = torch.tensor(self.freq_table, dtype=torch.float64, device=env.device)

    def cache_need(self) -> Optional[KVNeed]:
        # one row a position: [c | rotated key part] for the scores, c again (the kernel's value layout) for the sums
        return KVNeed(1, self.key_dim, 0, self.kv_rank) if self.own_kv else None

    def forward(self, h: torch.Tensor, ctx: StepContext, cache: Optional[LayerCache],
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
        if cache is None or cache.k is None:
            raise RuntimeError("latent attention needs a cache of latent rows")
        if self.own_kv != bool(cache.write):
            raise RuntimeError("a layer with a latent of its own writes its cache, a layer without one reads another's")
        kn = ctx.kernels
        rows, H = h.shape[0], self.heads
        qr, r, rd, kd = self.q_rank, self.kv_rank, self.rot_dim, self.key_dim
        inter = self.pairing == "interleaved"
        n_down = qr + (kd if self.own_kv else 0)
        down = ctx.ws.alloc((rows, _round8(n_down)), torch.float32)[:, :n_down]
        project(kn, ctx, h, self.w_down, down)
        cq = ctx.ws.alloc((rows, _round8(qr)), ctx.dtype)[:, :qr]
        kn.rmsnorm_cols(down[:, :qr], self.q_norm_w, self.eps, cq)
        if self.own_kv:
            row = ctx.ws.alloc((rows, _round8(kd)), ctx.dtype)[:, :kd]
            kn.rmsnorm_cols(down[:, qr : qr + r], self.kv_norm_w, self.eps, row[:, :r])
            kn.rotary(down[:, qr + r :], row[:, r:], 1, rd, rd, self.rot_dims, inter, self.freqs, self.magnitude,
                      ctx.row_pos)
            kn.kv_store(row, row[:, :r], 1, kd, r, ctx.row_pos, ctx.row_seq, ctx.seq_slot, cache.block_table,
                        cache.k, cache.v, cache.block_size)
        q_plain = ctx.ws.alloc((rows, H * self.dim), ctx.dtype)
        project(kn, ctx, cq, self.w_uq_plain, q_plain)
        q_rot = ctx.ws.alloc((rows, H * rd), torch.float32)
        project(kn, ctx, cq, self.w_uq_rot, q_rot)
        q = ctx.ws.alloc((rows, H * kd), ctx.dtype)  # head n: [Wuk_n^T q_unrot | q_rot rotated]
        kn.linear_heads(q_plain, self.w_uk_t, q, H, kd)
        kn.rotary(q_rot, q[:, r:], H, rd, kd, self.rot_dims, inter, self.freqs, self.magnitude, ctx.row_pos)
        mean = ctx.ws.alloc((rows, H * r), ctx.dtype)  # every head's weighted mean of latents
        kn.sink_attention(q, mean, H, 1, kd, r, ctx.row_pos, ctx.row_seq, ctx.seq_slot, cache.block_table, cache.k,
                          cache.v, cache.block_size, self.scale, window=0, keep_first=0, sink=False, gate=None,
                          decode=ctx.decode, **split_scratch(ctx, q.dtype, H, 1, kd, r, cache.block_size, 0, 0))
        att = ctx.ws.alloc((rows, H * self.value_dim), ctx.dtype)
        kn.linear_heads(mean, self.w_uv, att, H, self.value_dim)
        if out is None:
            out = ctx.ws.alloc((rows, self.width), torch.float32)
        project(kn, ctx, att, self.w_o, out)
        return out
