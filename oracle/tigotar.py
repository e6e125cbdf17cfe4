"""Plain CPU statement of the Tigotar decoder (TEST INFRASTRUCTURE ONLY, like oracle/model.py).

One function per mechanism, fp32 torch on the host, no cache, no state pool and no batching: a sequence is always
recomputed whole and the recurrence is a Python loop over its tokens, so nothing here can share a fault with the
engine's pools, kernels or scheduler.  Weights arrive as a dict of tensors under the checkpoint's own names (`embed`,
`embed.norm.alpha`, `loop.in`, `l<i>.mix.left.q`, `l<i>.mlp.e<j>.up`, ..., `final.norm`, `head`); the configuration is
the checkpoint's config.json as a dict.

Notation: T tokens, W the model width, H query heads, G key/value heads, D the query/key size, E the value size, R the
width of the recurrence, X experts of which each token takes K.
"""
from __future__ import annotations

import math
from typing import Dict, List

import torch


def dyn_tanh(x: torch.Tensor, w: Dict[str, torch.Tensor], name: str) -> torch.Tensor:
    """tanh(alpha x) * weight + bias: an element-wise squashing in the place of a norm (no statistics of the row)."""
    return torch.tanh(w[name + ".alpha"].float() * x.float()) * w[name].float() + w[name + ".b"].float()


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    x = x.float()
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rotate_pairs(x: torch.Tensor, base: float, dims: int) -> torch.Tensor:
    """x [T, heads, D]; the first `dims` elements of every head are dims / 2 neighbouring pairs (2i, 2i + 1); pair i of the
    token at position p turns by the angle p * base^(-2i / dims).  Elements from `dims` on are left as they are."""
    T = x.shape[0]
    x = x.float().clone()
    i = torch.arange(dims // 2, dtype=torch.float32)
    ang = torch.arange(T, dtype=torch.float32).view(T, 1) * base ** (-2.0 * i / dims)
    c, s = torch.cos(ang).view(T, 1, -1), torch.sin(ang).view(T, 1, -1)
    a, b = x[..., 0:dims:2].clone(), x[..., 1:dims:2].clone()
    x[..., 0:dims:2] = a * c - b * s
    x[..., 1:dims:2] = b * c + a * s
    return x


def window_mask(T: int, size: int, keep_first: int) -> torch.Tensor:
    """[T, T] bool: query i sees key j <= i when it is one of the last `size` positions (i - j < size) or one of the first
    `keep_first` of the sequence."""
    i = torch.arange(T).view(T, 1)
    j = torch.arange(T).view(1, T)
    return (j <= i) & ((i - j < size) | (j < keep_first))


def sigmoid_attention(q, k, v, scale: float, head_bias: torch.Tensor, mask: torch.Tensor) -> torch.Tensor:
    """q [T, H, D], k [T, G, D], v [T, G, E] -> [T, H, E].  Every visible key weighs sigmoid(scale q.k + bias of the head);
    the weights of a row are NOT normalised."""
    H, G = q.shape[1], k.shape[1]
    kk = k.float().repeat_interleave(H // G, 1)
    vv = v.float().repeat_interleave(H // G, 1)
    s = torch.einsum("ihd,jhd->hij", q.float(), kk) * scale + head_bias.float().view(H, 1, 1)
    p = torch.sigmoid(s) * mask
    return torch.einsum("hij,jhe->ihe", p, vv)


def window_attention_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], pre: str, m: dict, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    h = h.float()

    def proj(n):
        return h @ w[pre + n].float().T + w[pre + n + ".b"].float()

    q, k, v = proj("q").view(T, H, D), proj("k").view(T, G, D), proj("v").view(T, G, E)
    rot = m["rot"]
    q, k = rotate_pairs(q, rot["base"], rot["dims"]), rotate_pairs(k, rot["base"], rot["dims"])
    v = unit_rms(v, eps)
    mask = window_mask(T, m["mask"]["size"], m["mask"]["keep_first"])
    o = sigmoid_attention(q, k, v, m["scale"], w[pre + "pb"], mask)
    return o.reshape(T, H * E) @ w[pre + "o"].float().T


def min_gru_states(z_lin: torch.Tensor, u: torch.Tensor) -> torch.Tensor:
    """[T, R] pre-activations of the gate and of the candidate -> the states S_1 .. S_T from S_0 = 0:
    z = sigmoid(z_lin), c = u + 1/2 where u >= 0 else sigmoid(u), S_t = (1 - z_t) S_(t-1) + z_t c_t."""
    z = torch.sigmoid(z_lin.float())
    u = u.float()
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    S = torch.zeros(z.shape[1])
    states = []
    for t in range(z.shape[0]):
        S = (1.0 - z[t]) * S + z[t] * cand[t]
        states.append(S)
    return torch.stack(states) if states else torch.zeros(0, z.shape[1])


def min_gru_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], pre: str) -> torch.Tensor:
    """Gate and candidate read token t alone; the branch gives W_o (S_t * silu(W_g h_t))."""
    h = h.float()
    S = min_gru_states(h @ w[pre + "z"].float().T + w[pre + "z.b"].float(), h @ w[pre + "x"].float().T + w[pre + "x.b"].float())
    g = h @ w[pre + "g"].float().T
    return (S * torch.nn.functional.silu(g)) @ w[pre + "o"].float().T


def parallel_mixer(h, w, pre: str, m: dict, eps: float) -> torch.Tensor:
    return m["left_scale"] * window_attention_mixer(h, w, pre + "left.", m["left"], eps) \
        + m["right_scale"] * min_gru_mixer(h, w, pre + "right.")


def expert_mixture(h: torch.Tensor, w: Dict[str, torch.Tensor], pre: str, mlp: dict) -> torch.Tensor:
    """softmax over all X router logits, the K largest kept and divided by their sum; experts are down(relu(up h)^2)."""
    h = h.float()
    X, K = mlp["router"]["experts"], mlp["router"]["top"]
    s = torch.softmax(h @ w[pre + "router"].float().T, -1)
    top, idx = torch.topk(s, K, dim=-1)
    top = top / (top.sum(-1, keepdim=True) + 1e-20)
    out = torch.zeros_like(h)
    for e in range(X):
        y = torch.relu(h @ w[f"{pre}e{e}.up"].float().T) ** 2 @ w[f"{pre}e{e}.down"].float().T
        out = out + y * (top * (idx == e)).sum(-1, keepdim=True)
    return out


def layer_runs(cfg: dict) -> List[tuple]:
    """The order in which layers run: (layer index, number of the pass through the repeated span, first of its pass)."""
    n = len(cfg["layers"])
    loop = cfg.get("loop") or {"start": 0, "stop": 0, "times": 1}
    a, b, times = loop["start"], loop["stop"], loop["times"]
    runs = [(i, -1, False) for i in range(a)]
    for t in range(times):
        runs += [(i, t, i == a) for i in range(a, b)]
    return runs + [(i, -1, False) for i in range(b, n)]


def forward(cfg: dict, w: Dict[str, torch.Tensor], tokens: List[int], return_layers: bool = False):
    """Logits [T, vocab] of one sequence (and the residual stream after every layer run when asked)."""
    eps = cfg["norm"]["eps"]
    x0 = dyn_tanh(w["embed"].float()[torch.tensor(tokens, dtype=torch.long)], w, "embed.norm")
    x, seen = x0, []
    for i, t, first in layer_runs(cfg):
        if first:
            x = torch.cat([x, x0], -1) @ w["loop.in"].float().T + w["loop.step"].float()[t]
        layer, p = cfg["layers"][i], f"l{i}."
        if layer["type"] != "parallel":
            raise ValueError(layer["type"])
        y = parallel_mixer(dyn_tanh(x, w, p + "norm1"), w, p + "mix.", layer["mixer"], eps)
        x = x + dyn_tanh(y, w, p + "norm1b")
        if layer.get("mlp"):
            if layer["mlp"]["kind"] != "moe":
                raise ValueError(layer["mlp"]["kind"])
            y = expert_mixture(dyn_tanh(x, w, p + "norm2"), w, p + "mlp.", layer["mlp"])
            x = x + dyn_tanh(y, w, p + "norm2b")
        seen.append(x.clone())
    logits = dyn_tanh(x, w, "final.norm") @ w["head"].float().T * cfg["logit_scale"]
    return (logits, torch.stack(seen)) if return_layers else logits


def random_weights(cfg: dict, seed: int = 0) -> Dict[str, torch.Tensor]:
    """bfloat16 tensors under the checkpoint's names for a configuration (tests build their own small ones)."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def mat(o, i, s=None):
        return (torch.randn(o, i, generator=g) * (s if s is not None else 1.0 / math.sqrt(i))).to(torch.bfloat16)

    def vec(n, s=0.05, base=0.0):
        return (base + torch.randn(n, generator=g) * s).to(torch.bfloat16)

    w: Dict[str, torch.Tensor] = {"embed": mat(cfg["vocab"], W, 1.0), "head": mat(cfg["vocab"], W)}

    def norm(name, alpha=0.7):
        w[name], w[name + ".b"] = vec(W, 0.1, 1.0), vec(W, 0.1)
        w[name + ".alpha"] = (alpha + 0.3 * torch.rand((), generator=g)).to(torch.bfloat16)

    norm("embed.norm")
    norm("final.norm")
    loop = cfg.get("loop")
    if loop:
        w["loop.in"] = mat(W, 2 * W, 1.0 / math.sqrt(W))
        w["loop.step"] = vec(loop["times"] * W, 0.3).view(loop["times"], W)
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        for n in ("norm1", "norm1b", "norm2", "norm2b"):
            norm(p + n)
        a, r = m["left"], m["right"]["width"]
        H, G, D, E = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
        for n, rows in (("q", H * D), ("k", G * D), ("v", G * E)):
            w[p + "mix.left." + n], w[p + "mix.left." + n + ".b"] = mat(rows, W), vec(rows, 0.2)
        w[p + "mix.left.pb"] = vec(H, 1.0, -2.0)
        w[p + "mix.left.o"] = mat(W, H * E)
        for n in ("z", "x"):
            w[p + "mix.right." + n], w[p + "mix.right." + n + ".b"] = mat(r, W), vec(r, 0.5)
        w[p + "mix.right.g"], w[p + "mix.right.o"] = mat(r, W), mat(W, r)
        if layer.get("mlp"):
            F, X = layer["mlp"]["expert"]["ff"], layer["mlp"]["router"]["experts"]
            w[p + "mlp.router"] = mat(X, W, 2.0 / math.sqrt(W))
            for e in range(X):
                w[f"{p}mlp.e{e}.up"], w[f"{p}mlp.e{e}.down"] = mat(F, W), mat(W, F)
    return w
