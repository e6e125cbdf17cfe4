"""Kudirax: a post-norm decoder whose attention is local to blocks of positions and carries a sink term.

Per layer, on an fp32 residual stream x (a sublayer's input is x unnormalised; the norm is applied to what it RETURNS):
    x <- x + LayerNorm1(mixer(x));   x <- x + LayerNorm2(ff(x))   (a layer may have no ff)
mixer: q, k, v and an output gate from ONE merged GEMM; q and k scaled per head to unit RMS (no weight, no
rotation: positions enter only through the mask); v optionally blended with the values the first blending layer made for
the same token; attention over the keys of the query's own block of `chunk` positions (counted from the start of the
sequence) up to the query, scores scale * q.k capped by cap * tanh(. / cap), one extra term exp(sink[head]) in the softmax
denominator; heads * sigmoid(gate) -> output GEMM.  ff: down(relu(up(x) + b)^2) + b.  Final LayerNorm, vocabulary head.

Launches per layer: GEMM(q|k|v|gate), unit-norm + blend + KV-pool store, attention (+ gate), GEMM(o), LayerNorm + residual
add, GEMM(up), bias + squared ReLU, GEMM(down), (down's bias +) LayerNorm + residual add.  The GEMMs carry no bias -- the
biases ride in the elementwise kernels behind them -- so decode batches take the framework's weight-streaming kernel and
prefill batches its tuned library solutions like every other model's.  Every layer has its own head counts and sizes: the
KV pool holds one region per layer (mem_cache/memory_pool.py).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

import torch
import torch.nn.functional as F
from torch import nn

from semi_pd_amd import ops
from semi_pd_amd.distributed import get_tensor_model_parallel_world_size
from semi_pd_amd.layers.attention_backend import RadixAttention
from semi_pd_amd.layers.basic import (ColumnParallelLinear, LayerNorm, LogitsProcessor, MergedColumnParallelLinear,
                                      ParallelLMHead, RowParallelLinear, VocabParallelEmbedding, dense_linear)


@dataclass
class KudiraxMixerConfig:
    heads: int
    kv_heads: int
    dim: int                      # query / key size per head
    vdim: int                     # value size per head
    scale: float
    softcap: float = 0.0          # 0: scores are not capped
    chunk: int = 0                # positions per block of the mask; 0: every earlier position is visible
    v_mix: bool = False


@dataclass
class KudiraxLayerConfig:
    mixer: KudiraxMixerConfig
    ff: int = 0                   # 0: the layer has no feed-forward


@dataclass
class KudiraxConfig:
    vocab_size: int = 32000
    hidden_size: int = 1024
    norm_eps: float = 1e-5
    layers: List[KudiraxLayerConfig] = field(default_factory=list)
    architectures: tuple = ("Kudirax",)
    supports_float32 = True       # every kernel of its path is templated on the element type (ServerArgs --dtype float32)

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "KudiraxConfig":
        """The checkpoint's config.json: vocab, width, norm.eps and one entry per layer (type, mixer sizes, mlp or null)."""
        layers = []
        for i, entry in enumerate(d["layers"]):
            if entry.get("type") != "attention":
                raise ValueError(f"Kudirax layer {i}: mixer type {entry.get('type')!r} is not supported (attention only)")
            m = entry["mixer"]
            mask = m.get("mask") or {}
            unknown = set(mask) - {"size"}
            if unknown:
                raise ValueError(f"Kudirax layer {i}: mask keys {sorted(unknown)} are not supported")
            mixer = KudiraxMixerConfig(heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])), dim=int(m["dim"]),
                                       vdim=int(m.get("vdim", m["dim"])), scale=float(m["scale"]),
                                       softcap=float(m.get("softcap") or 0.0), chunk=int(mask.get("size") or 0),
                                       v_mix=bool(m.get("v_mix", False)))
            if mixer.heads % mixer.kv_heads:
                raise ValueError(f"Kudirax layer {i}: {mixer.heads} heads over {mixer.kv_heads} key/value heads")
            mlp = entry.get("mlp")
            if mlp is not None and mlp.get("kind", "dense") != "dense":
                raise ValueError(f"Kudirax layer {i}: feed-forward kind {mlp.get('kind')!r} is not supported (dense only)")
            layers.append(KudiraxLayerConfig(mixer=mixer, ff=int(mlp["ff"]) if mlp is not None else 0))
        return cls(vocab_size=int(d["vocab"]), hidden_size=int(d["width"]), norm_eps=float(d["norm"]["eps"]), layers=layers)


def kudirax_uniform(vocab_size: int, hidden_size: int, num_layers: int, heads: int, kv_heads: int, dim: int, vdim: int, ff: int,
                    chunk: int, softcap: float = 30.0, v_mix: bool = True, norm_eps: float = 1e-5) -> KudiraxConfig:
    """A configuration whose layers are all alike (benchmarks, tests)."""
    mixer = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=dim ** -0.5, softcap=softcap, chunk=chunk, v_mix=v_mix)
    return KudiraxConfig(vocab_size=vocab_size, hidden_size=hidden_size, norm_eps=norm_eps,
                         layers=[KudiraxLayerConfig(KudiraxMixerConfig(**mixer), ff) for _ in range(num_layers)])


class KudiraxForwardState:
    """What one forward pass carries from layer to layer next to the residual stream: the values of the first blending
    layer (a column range of that layer's projection output, alive for the pass only -- nothing of it is cached)."""

    def __init__(self):
        self.v_first: Optional[torch.Tensor] = None


class KudiraxMixer(nn.Module):
    def __init__(self, hidden_size: int, m: KudiraxMixerConfig, eps: float, layer_id: int, dtype):
        super().__init__()
        self.m, self.eps = m, eps
        self.q_size, self.k_size = m.heads * m.dim, m.kv_heads * m.dim
        self.v_size, self.o_size = m.kv_heads * m.vdim, m.heads * m.vdim
        # rows of the merged weight: q | k | v | gate
        self.qkvg_proj = MergedColumnParallelLinear(hidden_size, [self.q_size, self.k_size, self.v_size, self.o_size],
                                                    params_dtype=dtype)
        self.o_proj = RowParallelLinear(self.o_size, hidden_size, params_dtype=dtype)
        self.sink = nn.Parameter(torch.zeros(m.heads, dtype=torch.float32), requires_grad=False)
        self.vmix = nn.Parameter(torch.zeros((), dtype=dtype), requires_grad=False)
        self.attn = RadixAttention(m.heads, m.dim, m.scale, m.kv_heads, layer_id, logit_cap=m.softcap, v_head_dim=m.vdim,
                                   chunk_size=m.chunk)

    def forward(self, h: torch.Tensor, forward_batch, state: KudiraxForwardState) -> torch.Tensor:
        m = self.m
        p = self.qkvg_proj(h)
        k_off, v_off, g_off = self.q_size, self.q_size + self.k_size, self.q_size + self.k_size + self.v_size
        v_first = None
        if m.v_mix:
            if state.v_first is None:
                state.v_first = p[:, v_off: v_off + self.v_size]       # this layer's own values, as projected
            else:
                v_first = state.v_first
        pool = forward_batch.token_to_kv_pool
        lid = self.attn.layer_id
        ops.unit_norm_and_store_kv(p, m.heads, m.kv_heads, m.dim, m.vdim, k_off, v_off, self.eps, pool.get_key_buffer(lid),
                                   pool.get_value_buffer(lid), forward_batch.out_cache_loc, v_first=v_first,
                                   mix=self.vmix if v_first is not None else None)
        o = forward_batch.attn_backend.forward_local(p[:, : self.q_size], self.attn, forward_batch,
                                                     gate=p[:, g_off: g_off + self.o_size], sink=self.sink)
        return self.o_proj(o)


class KudiraxFeedForward(nn.Module):
    def __init__(self, hidden_size: int, ff: int, dtype):
        super().__init__()
        self.up = ColumnParallelLinear(hidden_size, ff, bias=True, params_dtype=dtype)
        self.down = RowParallelLinear(ff, hidden_size, bias=True, params_dtype=dtype)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        """down(relu(up(h) + b_up)^2) WITHOUT down's bias: the LayerNorm kernel behind it adds it."""
        u = dense_linear(h, self.up.weight)
        ops.bias_relu_square_(u, self.up.bias)
        return dense_linear(u, self.down.weight)


class KudiraxDecoderLayer(nn.Module):
    def __init__(self, config: KudiraxConfig, layer_id: int, dtype):
        super().__init__()
        lc = config.layers[layer_id]
        W = config.hidden_size
        self.mix = KudiraxMixer(W, lc.mixer, config.norm_eps, layer_id, dtype)
        self.norm1 = LayerNorm(W, config.norm_eps, dtype)
        self.mlp = KudiraxFeedForward(W, lc.ff, dtype) if lc.ff else None
        self.norm2 = LayerNorm(W, config.norm_eps, dtype) if lc.ff else None

    def forward(self, h: torch.Tensor, x: torch.Tensor, forward_batch, state: KudiraxForwardState) -> torch.Tensor:
        """x: the fp32 stream (updated in place); h: x in the activation type.  Returns the new h."""
        h = self.norm1.forward_add(self.mix(h, forward_batch, state), x)
        if self.mlp is not None:
            h = self.norm2.forward_add(self.mlp(h), x, in_bias=self.mlp.down.bias)
        return h


class KudiraxForCausalLM(nn.Module):
    def __init__(self, config: KudiraxConfig, dtype=torch.bfloat16):
        super().__init__()
        if get_tensor_model_parallel_world_size() != 1:
            raise ValueError("Kudirax runs on one GPU per replica (tensor parallelism over its per-layer head counts is not "
                             "implemented)")
        if not config.layers:
            raise ValueError("Kudirax: the configuration lists no layers")
        self.config = config
        self.embed = VocabParallelEmbedding(config.vocab_size, config.hidden_size, params_dtype=dtype)
        self.layers = nn.ModuleList([KudiraxDecoderLayer(config, i, dtype) for i in range(len(config.layers))])
        self.final_norm = LayerNorm(config.hidden_size, config.norm_eps, dtype)
        self.head = ParallelLMHead(config.vocab_size, config.hidden_size, params_dtype=dtype)
        self.logits_processor = LogitsProcessor(config.vocab_size)
        self.layer_probe = None      # tests: a callable (layer index, fp32 stream) run after every layer
        for p in self.parameters():
            p.requires_grad_(False)

    @property
    def kv_geometry(self):
        ms = [lc.mixer for lc in self.config.layers]
        return dict(kind="mha", num_kv_heads=[m.kv_heads for m in ms], head_dim=[m.dim for m in ms],
                    v_head_dim=[m.vdim for m in ms], num_heads=[m.heads for m in ms], num_layers=len(ms))

    @torch.no_grad()
    def forward(self, input_ids, positions, forward_batch):
        h = self.embed(input_ids)
        x = h.float()                                   # the residual stream never leaves fp32
        state = KudiraxForwardState()
        for i, layer in enumerate(self.layers):
            h = layer(h, x, forward_batch, state)
            if self.layer_probe is not None:
                self.layer_probe(i, x)
        hidden = self.final_norm(x)
        return self.logits_processor(input_ids, hidden, self.head, forward_batch)
