"""Plain CPU statement of the Kudirax decoder (TEST INFRASTRUCTURE ONLY, like oracle/model.py).

One function per mechanism, fp32 torch on the host, no cache and no batching: a sequence is always
recomputed whole, so nothing here can share a fault with the engine's pools, kernels or scheduler.
Weights arrive as a dict of tensors under the checkpoint's own names (`embed`, `l<i>.mix.q`,
`l<i>.norm1.b`, ..., `final.norm`, `head`); the configuration is the checkpoint's config.json as a
dict.

Notation: T tokens, H query heads, G key/value heads, D the query/key size, E the value size.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch


def layer_norm(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float) -> torch.Tensor:
    """(x - mean) / sqrt(var + eps) * w + b with the biased variance."""
    x = x.float()
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w.float() + b.float()


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis, no weight."""
    x = x.float()
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def soft_cap(s: torch.Tensor, cap: float) -> torch.Tensor:
    return cap * torch.tanh(s / cap) if cap else s


def visible(T: int, chunk: Optional[int]) -> torch.Tensor:
    """[T, T] bool: query i sees key j when j <= i and both lie in the same block of `chunk` positions counted from 0
    (no chunk: plain causal)."""
    i = torch.arange(T).view(T, 1)
    j = torch.arange(T).view(1, T)
    m = j <= i
    if chunk:
        m = m & (torch.div(i, chunk, rounding_mode="floor") == torch.div(j, chunk, rounding_mode="floor"))
    return m


def sink_softmax(s: torch.Tensor, mask: torch.Tensor, sink: Optional[torch.Tensor]) -> torch.Tensor:
    """Softmax over the visible keys whose denominator also holds exp(sink) of the head.  s [H, T, T], sink [H]."""
    s = s.masked_fill(~mask, float("-inf"))
    if sink is None:
        return torch.softmax(s, -1)
    col = sink.float().view(-1, 1, 1).expand(s.shape[0], s.shape[1], 1)
    p = torch.softmax(torch.cat([s, col], -1), -1)
    return p[..., :-1]


def local_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, cap: float, chunk: Optional[int],
                    sink: Optional[torch.Tensor]) -> torch.Tensor:
    """One whole sequence: q [T, H, D], k [T, G, D], v [T, G, E] -> [T, H, E].  Query head h reads key/value head
    h // (H / G); capped scores; block-local causal mask; sink in the denominator."""
    T, H = q.shape[0], q.shape[1]
    rep = H // k.shape[1]
    kk = k.float().repeat_interleave(rep, 1)
    vv = v.float().repeat_interleave(rep, 1)
    s = soft_cap(torch.einsum("ihd,jhd->hij", q.float(), kk) * scale, cap)
    p = sink_softmax(s, visible(T, chunk), sink)
    return torch.einsum("hij,jhe->ihe", p, vv)


def attention_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], pre: str, m: dict, eps: float,
                    v_first: Optional[torch.Tensor]):
    """One sequence h [T, width] through the attention mixer whose tensors start with `pre`.
    Returns (output [T, width], the values that went into the attention [T, G, E])."""
    T = h.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    h = h.float()
    q = (h @ w[pre + "q"].float().T).view(T, H, D)
    k = (h @ w[pre + "k"].float().T).view(T, G, D)
    v = (h @ w[pre + "v"].float().T).view(T, G, E)
    q, k = unit_rms(q, eps), unit_rms(k, eps)
    if v_first is not None:
        lam = w[pre + "vmix"].float()
        v = (1.0 - lam) * v + lam * v_first
    o = local_attention(q, k, v, m["scale"], m.get("softcap") or 0.0, (m.get("mask") or {}).get("size"),
                        w.get(pre + "sink")).reshape(T, H * E)
    o = o * torch.sigmoid(h @ w[pre + "g"].float().T)
    return o @ w[pre + "o"].float().T, v


def dense_ff(h: torch.Tensor, w: Dict[str, torch.Tensor], pre: str) -> torch.Tensor:
    h = h.float()
    u = torch.relu(h @ w[pre + "up"].float().T + w[pre + "up.b"].float()) ** 2
    return u @ w[pre + "down"].float().T + w[pre + "down.b"].float()


def forward(cfg: dict, w: Dict[str, torch.Tensor], tokens: List[int], return_layers: bool = False):
    """Logits [T, vocab] of one sequence (and the residual stream after every layer when asked)."""
    eps = cfg["norm"]["eps"]
    x = w["embed"].float()[torch.tensor(tokens, dtype=torch.long)]
    v_first, seen = None, []
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        if layer["type"] != "attention":
            raise ValueError(layer["type"])
        m = layer["mixer"]
        mixes = bool(m.get("v_mix"))
        y, v = attention_mixer(x, w, p + "mix.", m, eps, v_first if mixes else None)
        if mixes and v_first is None:
            v_first = v
        x = x + layer_norm(y, w[p + "norm1"], w[p + "norm1.b"], eps)
        if layer.get("mlp"):
            if layer["mlp"]["kind"] != "dense":
                raise ValueError(layer["mlp"]["kind"])
            x = x + layer_norm(dense_ff(x, w, p + "mlp."), w[p + "norm2"], w[p + "norm2.b"], eps)
        seen.append(x.clone())
    logits = layer_norm(x, w["final.norm"], w["final.norm.b"], eps) @ w["head"].float().T
    return (logits, torch.stack(seen)) if return_layers else logits


def random_weights(cfg: dict, seed: int = 0, std: float = 0.05) -> Dict[str, torch.Tensor]:
    """bfloat16 tensors under the checkpoint's names for a configuration (tests build their own small ones)."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def mat(o, i, s=None):
        return (torch.randn(o, i, generator=g) * (s if s is not None else 1.0 / math.sqrt(i))).to(torch.bfloat16)

    def vec(n, s=std, base=0.0):
        return (base + torch.randn(n, generator=g) * s).to(torch.bfloat16)

    w = {"embed": mat(cfg["vocab"], W, 1.0), "head": mat(cfg["vocab"], W),
         "final.norm": vec(W, 0.1, 1.0), "final.norm.b": vec(W, 0.1)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        w[p + "mix.q"], w[p + "mix.k"], w[p + "mix.v"] = mat(H * D, W), mat(G * D, W), mat(G * E, W)
        w[p + "mix.g"], w[p + "mix.o"] = mat(H * E, W), mat(W, H * E)
        w[p + "mix.sink"] = vec(H, 1.0)
        w[p + "mix.vmix"] = (torch.rand((), generator=g) * 0.6 + 0.2).to(torch.bfloat16)
        w[p + "norm1"], w[p + "norm1.b"] = vec(W, 0.1, 1.0), vec(W, 0.1)
        w[p + "norm2"], w[p + "norm2.b"] = vec(W, 0.1, 1.0), vec(W, 0.1)
        if layer.get("mlp"):
            F = layer["mlp"]["ff"]
            w[p + "mlp.up"], w[p + "mlp.up.b"] = mat(F, W), vec(F, 0.1)
            w[p + "mlp.down"], w[p + "mlp.down.b"] = mat(W, F), vec(W, 0.1)
    return w
