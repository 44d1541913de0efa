"""The Vupelorn decoder, written plainly: float64, whole sequences, no cache, one function per mechanism.

It shares nothing with the library: it takes a configuration as the dict that config.json holds and the
tensors as a dict name -> torch tensor, and walks a sequence from its first token.  `rounding=True` rounds the
activations to bfloat16 where a bfloat16 run of the library holds them in 16 bits (the inputs of matrix
products), so that a comparison with such a run is not dominated by that rounding.

Notation: h is a sublayer's input [T, width]; W x means a weight stored [out, in] applied to a column x.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F = torch.float64


def rb(x: torch.Tensor, rounding: bool) -> torch.Tensor:
    """The bfloat16 rounding of x (kept as float64) where a bfloat16 run holds the value in 16 bits."""
    return x.to(torch.bfloat16).to(F) if rounding else x


def lin(w: torch.Tensor, x: torch.Tensor, rounding: bool = False) -> torch.Tensor:
    return rb(x, rounding) @ w.to(F).t()


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


# ---- embedding ---------------------------------------------------------------------------------------------
def bigram_rows(tokens: List[int], buckets: int, mul_prev: int, mul_cur: int) -> List[int]:
    """Row of the bigram table for every token: a hash of (previous, current); the extra last row for the first."""
    rows = []
    for i, t in enumerate(tokens):
        rows.append(buckets if i == 0 else (tokens[i - 1] * mul_prev + t * mul_cur) % buckets)
    return rows


def embedding(cfg: dict, w: Dict[str, torch.Tensor], tokens: List[int]) -> torch.Tensor:
    x = w["embed"].to(F)[tokens]
    bg = (cfg.get("embedding") or {}).get("bigram")
    if bg:
        x = x + w["bigram"].to(F)[bigram_rows(tokens, bg["buckets"], bg["mul_prev"], bg["mul_cur"])]
    return x


# ---- gated linear attention ----------------------------------------------------------------------------------
def gla(m: dict, p: str, w: Dict[str, torch.Tensor], h: torch.Tensor, eps: float, rounding: bool) -> torch.Tensor:
    T = h.shape[0]
    H, dk, dv, tau = m["heads"], m["dim"], m["vdim"], float(m["tau"])
    q = lin(w[p + "q"], h, rounding).reshape(T, H, dk) * dk ** -0.5
    k = lin(w[p + "k"], h, rounding).reshape(T, H, dk)
    v = lin(w[p + "v"], h, rounding).reshape(T, H, dv)
    z = lin(w[p + "a2"], lin(w[p + "a1"], h, rounding), rounding) + w[p + "a2.b"].to(F)
    alpha = torch.sigmoid(z).pow(1.0 / tau).reshape(T, H, dk)
    S = torch.zeros(H, dk, dv, dtype=F)
    o = torch.zeros(T, H, dv, dtype=F)
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hkv,hk->hv", S, q[t])
    o = rms(o, eps) * w[p + "norm"].to(F)
    g = lin(w[p + "g"], h, rounding)
    y = o.reshape(T, H * dv) * (g * torch.sigmoid(g))
    return lin(w[p + "o"], y, rounding)


# ---- rotary positions ------------------------------------------------------------------------------------------
def rotary_table(rot: dict, positions: torch.Tensor):
    """cos and sin [T, dims / 2] of the angles p f_i, with the YaRN change of the frequencies where `scaling` is
    given (then both are also multiplied by 0.1 ln(factor) + 1)."""
    dims, base = int(rot["dims"]), float(rot["base"])
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F)
    mag = 1.0
    sc = rot.get("scaling")
    if sc:
        factor, orig = float(sc["factor"]), float(sc["original"])

        def dim_of(turns: float) -> float:
            return dims * math.log(orig / (2 * math.pi * turns)) / (2 * math.log(base))

        lo = max(math.floor(dim_of(float(sc["fast"]))), 0)
        hi = min(math.ceil(dim_of(float(sc["slow"]))), dims - 1)
        ramp = torch.clamp((torch.arange(half, dtype=F) - lo) / max(hi - lo, 0.001), 0, 1)
        f = f / factor * ramp + f * (1 - ramp)
        mag = 0.1 * math.log(factor) + 1
    ang = positions.to(F)[:, None] * f[None, :]
    return torch.cos(ang) * mag, torch.sin(ang) * mag


def rotate(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, dims: int, interleaved: bool) -> torch.Tensor:
    """x [T, ..., n]: the first `dims` entries of the last axis are rotated, the rest pass."""
    half = dims // 2
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    c, s = cos.reshape(shape), sin.reshape(shape)
    out = x.clone()
    if interleaved:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = u * c - v * s
        out[..., 1:dims:2] = v * c + u * s
    else:
        u, v = x[..., :half], x[..., half:dims]
        out[..., :half] = u * c - v * s
        out[..., half:dims] = v * c + u * s
    return out


# ---- latent attention --------------------------------------------------------------------------------------------
def latent_kv(m: dict, p: str, w: Dict[str, torch.Tensor], h: torch.Tensor, eps: float, interleaved: bool,
              rounding: bool):
    """What a layer with a down-projection of its own leaves for the keys and values: the normed latent c
    [T, kv_rank] and the rotated key part [T, rot_dim] that all heads share."""
    T = h.shape[0]
    r = m["kv_rank"]
    d = lin(w[p + "dkv"], h, rounding)
    c = rms(d[:, :r], eps) * w[p + "dkv.norm"].to(F)
    cos, sin = rotary_table(m["rot"], torch.arange(T))
    kr = rotate(d[:, r:], cos, sin, int(m["rot"]["dims"]), interleaved)
    return rb(c, rounding), rb(kr, rounding)


def latent_attention(m: dict, p: str, w: Dict[str, torch.Tensor], h: torch.Tensor, eps: float, interleaved: bool,
                     rounding: bool, shared=None) -> torch.Tensor:
    T = h.shape[0]
    H, dn, dr, dv, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    c, kr = shared if shared is not None else latent_kv(m, p, w, h, eps, interleaved, rounding)
    cq = rms(lin(w[p + "dq"], h, rounding), eps) * w[p + "dq.norm"].to(F)
    q = lin(w[p + "uq"], cq, rounding).reshape(T, H, dn + dr)
    cos, sin = rotary_table(m["rot"], torch.arange(T))
    q_rot = rotate(q[..., dn:], cos, sin, int(m["rot"]["dims"]), interleaved)
    k_nope = lin(w[p + "uk"], c).reshape(T, H, dn)
    val = lin(w[p + "uv"], c).reshape(T, H, dv)
    s = torch.einsum("thd,uhd->htu", q[..., :dn], k_nope) + torch.einsum("thd,ud->htu", q_rot, kr)
    s = s * float(m["scale"])
    mask = torch.ones(T, T, dtype=torch.bool).tril()
    s = s.masked_fill(~mask, float("-inf"))
    pr = torch.softmax(s, dim=-1)
    o = torch.einsum("htu,uhv->thv", pr, val).reshape(T, H * dv)
    return lin(w[p + "o"], o, rounding)


# ---- mixture of experts -----------------------------------------------------------------------------------------
def expert(e: str, w: Dict[str, torch.Tensor], h: torch.Tensor, limit: float, rounding: bool) -> torch.Tensor:
    g = torch.clamp(lin(w[e + "gate"], h, rounding), max=limit)
    u = torch.clamp(lin(w[e + "up"], h, rounding), -limit, limit)
    y = g * torch.sigmoid(1.702 * g) * (u + 1)
    return lin(w[e + "down"], y, rounding)


def moe(mlp: dict, p: str, w: Dict[str, torch.Tensor], h: torch.Tensor, rounding: bool) -> torch.Tensor:
    n, top = mlp["router"]["experts"], mlp["router"]["top"]
    limit = float(mlp["expert"]["limit"])
    score = torch.sigmoid(lin(w[p + "router"], h, rounding))
    out = torch.zeros(h.shape[0], w[p + "e0.down"].shape[0], dtype=F)
    for t in range(h.shape[0]):
        chosen = sorted(range(n), key=lambda e: (-float(score[t, e]), e))[:top]
        for e in chosen:
            out[t] += expert(f"{p}e{e}.", w, (score[t, e] * h[t])[None], limit, rounding)[0]
    return out


# ---- the model ------------------------------------------------------------------------------------------------------
def forward(cfg: dict, w: Dict[str, torch.Tensor], tokens: List[int], rounding: bool = False,
            layers_out: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of a whole sequence; `layers_out` collects the residual stream after every layer."""
    eps = float(cfg["norm"]["eps"])
    x = embedding(cfg, w, list(tokens))
    kept = {}
    for i, layer in enumerate(cfg["layers"]):
        p, m, kind = f"l{i}.mix.", layer["mixer"], layer["type"]
        if kind == "gla":
            y = gla(m, p, w, x, eps, rounding)
        elif kind in ("latent_attention", "latent_attention_2"):
            inter = kind == "latent_attention_2"
            src = m.get("kv_from")
            if src is None:
                kept[i] = latent_kv(m, p, w, x, eps, inter, rounding)
            y = latent_attention(m, p, w, x, eps, inter, rounding, shared=kept[i if src is None else src])
        else:
            raise ValueError(kind)
        x = x + rms(y, eps) * w[f"l{i}.norm1"].to(F)
        if layer.get("mlp") is not None:
            x = x + rms(moe(layer["mlp"], f"l{i}.mlp.", w, x, rounding), eps) * w[f"l{i}.norm2"].to(F)
        if layers_out is not None:
            layers_out.append(x.clone())
    return lin(w["embed"], rms(x, eps) * w["final.norm"].to(F), rounding)
