"""Tigotar: a decoder whose mixer is an attention branch and a recurrent branch side by side, with a mixture of experts
behind it, squashed (not normalised) on both sides of every sublayer, and a span of layers that is run several times.

On an fp32 residual stream x, DynTanh(v) = tanh(alpha v) * w + b:
    x <- x + DynTanh_1b(mixer(DynTanh_1(x)));   x <- x + DynTanh_2b(experts(DynTanh_2(x)))   (a layer may have no experts)
mixer(h) = left_scale * attention(h) + right_scale * recurrence(h), both reading the same h:
  * attention: q, k, v with biases; neighbouring pairs of the first rot_dims elements of every q / k head rotated by the
    position; every value head scaled to unit RMS before it is cached; a query sees the last `window` positions and the
    first `keep_first` positions of its sequence; a visible key weighs sigmoid(scale q.k + bias of the head), and the
    weights are NOT normalised over the keys.
  * recurrence (minGRU): S_t = (1 - z_t) S_(t-1) + z_t c_t per channel, gate z and candidate c functions of token t alone,
    S in fp32 in the request's row of the state pool; the branch gives S_t * silu(g_t).
experts: softmax over all router logits (fp32), the top-k kept and renormalised, experts down(relu(up h)^2).
Layers [loop_start, loop_stop) run loop_times times with the same weights; every pass has KV-pool regions and state columns
of its own and starts with x <- W_in [x; x0] + step[pass], x0 the stream as the embedding (and its DynTanh) left it.

Launches per layer run: GEMM(q|k|v|z|x|g), bias + rotation + value norm + KV store, attention -> columns [0, H E) of the
output projection's input, recurrence -> its columns [H E, H E + R), GEMM([left o | right o]) (the two branch scales ride in
the kernels in front of it), DynTanh seam (stream += squash(y); next sublayer's input = squash(stream)), router GEMM (fp32),
top-k, expert GEMMs + activation + sum, DynTanh seam.  Biases ride in the elementwise kernels behind the GEMMs, so the GEMMs
are the framework's bias-free ones (weight streaming for decode batches, tuned library solutions for prompts).
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
from semi_pd_amd.layers.basic import (DynTanh, LogitsProcessor, MergedColumnParallelLinear, ParallelLMHead,
                                      RowParallelLinear, VocabParallelEmbedding)
from semi_pd_amd.layers.moe import UngatedMoE


@dataclass
class TigotarAttentionConfig:
    heads: int
    kv_heads: int
    dim: int                      # query / key size per head
    vdim: int                     # value size per head
    scale: float
    window: int                   # positions a query looks back over, itself included (0: every earlier position)
    keep_first: int               # positions at the start of the sequence that stay visible
    rot_dims: int                 # leading elements of a head that are rotated (0: none)
    rot_base: float


@dataclass
class TigotarMixerConfig:
    left: TigotarAttentionConfig
    right_width: int
    left_scale: float = 1.0
    right_scale: float = 1.0


@dataclass
class TigotarLayerConfig:
    mixer: TigotarMixerConfig
    experts: int = 0              # 0: the layer has no feed-forward
    top: int = 0
    ff: int = 0


@dataclass
class LayerRun:
    layer: int                    # which layer's weights
    run: int                      # number of the run: the id of its KV-pool region and of its state columns
    loop_pass: int                # pass through the repeated span (-1 outside it)
    enters_pass: bool             # the pass starts in front of this run


@dataclass
class TigotarConfig:
    vocab_size: int = 32000
    hidden_size: int = 1024
    norm_eps: float = 1e-6
    logit_scale: float = 1.0
    layers: List[TigotarLayerConfig] = field(default_factory=list)
    loop_start: int = 0
    loop_stop: int = 0            # start == stop: nothing is repeated
    loop_times: int = 1
    architectures: tuple = ("Tigotar",)
    supports_float32 = True       # every kernel of its path is templated on the element type (ServerArgs --dtype float32)

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @property
    def has_loop(self) -> bool:
        return self.loop_stop > self.loop_start

    def runs(self) -> List[LayerRun]:
        """Layer runs in execution order: layers in front of the span once, the span loop_times times, the rest once."""
        order = [(i, -1, False) for i in range(self.loop_start)]
        for t in range(self.loop_times if self.has_loop else 0):
            order += [(i, t, i == self.loop_start) for i in range(self.loop_start, self.loop_stop)]
        order += [(i, -1, False) for i in range(self.loop_stop if self.has_loop else self.loop_start, len(self.layers))]
        return [LayerRun(i, n, t, first) for n, (i, t, first) in enumerate(order)]

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "TigotarConfig":
        """The checkpoint's config.json: vocab, width, norm.eps, logit_scale, loop {start, stop, times} and one entry per
        layer (type, mixer {left {...}, right {width}, left_scale, right_scale}, mlp {kind, expert {ff}, router {experts,
        top}} or null)."""
        layers = []
        for i, entry in enumerate(d["layers"]):
            if entry.get("type") != "parallel":
                raise ValueError(f"Tigotar layer {i}: mixer type {entry.get('type')!r} is not supported (parallel only)")
            m = entry["mixer"]
            a = m["left"]
            mask, rot = a.get("mask") or {}, a.get("rot") or {}
            unknown = (set(mask) - {"size", "keep_first"}) | (set(rot) - {"base", "dims"})
            if unknown:
                raise ValueError(f"Tigotar layer {i}: keys {sorted(unknown)} are not supported")
            left = TigotarAttentionConfig(heads=int(a["heads"]), kv_heads=int(a.get("kv_heads", a["heads"])), dim=int(a["dim"]),
                                          vdim=int(a.get("vdim", a["dim"])), scale=float(a["scale"]),
                                          window=int(mask.get("size") or 0), keep_first=int(mask.get("keep_first") or 0),
                                          rot_dims=int(rot.get("dims") or 0), rot_base=float(rot.get("base") or 10000.0))
            if left.heads % left.kv_heads:
                raise ValueError(f"Tigotar layer {i}: {left.heads} heads over {left.kv_heads} key/value heads")
            if left.rot_dims % 2 or left.rot_dims > left.dim:
                raise ValueError(f"Tigotar layer {i}: {left.rot_dims} rotated elements of a head of {left.dim}")
            if left.keep_first and not left.window:
                left.keep_first = 0            # without a window every earlier position is visible anyway
            mixer = TigotarMixerConfig(left=left, right_width=int(m["right"]["width"]), left_scale=float(m.get("left_scale", 1.0)),
                                       right_scale=float(m.get("right_scale", 1.0)))
            mlp = entry.get("mlp")
            if mlp is None:
                layers.append(TigotarLayerConfig(mixer=mixer))
                continue
            if mlp.get("kind") != "moe":
                raise ValueError(f"Tigotar layer {i}: feed-forward kind {mlp.get('kind')!r} is not supported (moe only)")
            lc = TigotarLayerConfig(mixer=mixer, experts=int(mlp["router"]["experts"]), top=int(mlp["router"]["top"]),
                                    ff=int(mlp["expert"]["ff"]))
            if not 0 < lc.top <= lc.experts:
                raise ValueError(f"Tigotar layer {i}: top {lc.top} of {lc.experts} experts")
            layers.append(lc)
        loop = d.get("loop") or {}
        start, stop, times = int(loop.get("start", 0)), int(loop.get("stop", 0)), int(loop.get("times", 1))
        if not (0 <= start <= stop <= len(layers)) or times < 1:
            raise ValueError(f"Tigotar: loop {loop} does not fit {len(layers)} layers")
        return cls(vocab_size=int(d["vocab"]), hidden_size=int(d["width"]), norm_eps=float(d["norm"]["eps"]),
                   logit_scale=float(d.get("logit_scale", 1.0)), layers=layers, loop_start=start, loop_stop=stop,
                   loop_times=times)


def tigotar_uniform(vocab_size: int, hidden_size: int, num_layers: int, heads: int, kv_heads: int, dim: int, vdim: int,
                    right_width: int, experts: int, top: int, ff: int, window: int, keep_first: int = 4,
                    loop: Optional[tuple] = None, rot_dims: Optional[int] = None, norm_eps: float = 1e-6) -> TigotarConfig:
    """A configuration whose layers are all alike (benchmarks, tests).  loop: (start, stop, times)."""
    left = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=dim ** -0.5, window=window, keep_first=keep_first,
                rot_dims=dim if rot_dims is None else rot_dims, rot_base=10000.0)
    start, stop, times = loop or (0, 0, 1)
    return TigotarConfig(vocab_size=vocab_size, hidden_size=hidden_size, norm_eps=norm_eps, loop_start=start, loop_stop=stop,
                         loop_times=times, layers=[TigotarLayerConfig(TigotarMixerConfig(TigotarAttentionConfig(**left),
                                                                                         right_width), experts, top, ff)
                                                   for _ in range(num_layers)])


class TigotarMixer(nn.Module):
    def __init__(self, hidden_size: int, mc: TigotarMixerConfig, eps: float, run_ids: List[int], dtype):
        super().__init__()
        a = mc.left
        self.mc, self.eps = mc, eps
        self.q_size, self.k_size, self.v_size = a.heads * a.dim, a.kv_heads * a.dim, a.kv_heads * a.vdim
        self.o_size, self.r_size = a.heads * a.vdim, mc.right_width
        # rows of the merged weight: q | k | v of the attention branch, z | x | g of the recurrent one
        self.in_proj = MergedColumnParallelLinear(hidden_size, [self.q_size, self.k_size, self.v_size, self.r_size, self.r_size,
                                                                self.r_size], params_dtype=dtype)
        # columns of the merged output weight: the attention heads, then the recurrent channels
        self.out_proj = RowParallelLinear(self.o_size + self.r_size, hidden_size, params_dtype=dtype)
        for name, n in (("bias_q", self.q_size), ("bias_k", self.k_size), ("bias_v", self.v_size), ("bias_z", self.r_size),
                        ("bias_x", self.r_size)):
            setattr(self, name, nn.Parameter(torch.zeros(n, dtype=dtype), requires_grad=False))
        self.head_bias = nn.Parameter(torch.zeros(a.heads, dtype=torch.float32), requires_grad=False)
        i = torch.arange(a.rot_dims // 2, dtype=torch.float32)
        self.register_buffer("inv_freq", a.rot_base ** (-2.0 * i / max(a.rot_dims, 1)), persistent=False)
        # one descriptor per run of this layer: a run has a KV-pool region and state columns of its own
        self.attn = {r: RadixAttention(a.heads, a.dim, a.scale, a.kv_heads, r, v_head_dim=a.vdim, window=a.window,
                                       keep_first=a.keep_first, sigmoid_weights=True) for r in run_ids}

    def forward(self, h: torch.Tensor, forward_batch, run: int) -> torch.Tensor:
        a, mc = self.mc.left, self.mc
        p = self.in_proj(h)
        k_off = self.q_size
        v_off = k_off + self.k_size
        z_off = v_off + self.v_size
        x_off, g_off = z_off + self.r_size, z_off + 2 * self.r_size
        pool = forward_batch.token_to_kv_pool
        ops.bias_rope_vnorm_kv_store(p, a.heads, a.kv_heads, a.dim, a.vdim, k_off, v_off, self.bias_q, self.bias_k, self.bias_v,
                                     forward_batch.positions, self.inv_freq if a.rot_dims else None, a.rot_dims, self.eps,
                                     pool.get_key_buffer(run), pool.get_value_buffer(run), forward_batch.out_cache_loc)
        both = torch.empty((p.shape[0], self.o_size + self.r_size), dtype=p.dtype, device=p.device)
        forward_batch.attn_backend.forward_window(p[:, : self.q_size], self.attn[run], forward_batch, out=both[:, : self.o_size],
                                                  head_bias=self.head_bias, out_scale=mc.left_scale)
        if forward_batch.forward_mode.is_decode():
            q_start = q_len = None
            max_q = 1
        else:
            q_start, q_len = forward_batch.extend_start_loc, forward_batch.extend_seq_lens
            max_q = max(forward_batch.extend_seq_lens_cpu)
        ops.min_gru(p, z_off, x_off, g_off, self.r_size, self.bias_z, self.bias_x, both[:, self.o_size:],
                    forward_batch.state_pool.get_state_buffer(run), forward_batch.state_indices, forward_batch.seq_lens,
                    q_start, q_len, max_q, out_scale=mc.right_scale)
        return self.out_proj(both)


class TigotarDecoderLayer(nn.Module):
    def __init__(self, config: TigotarConfig, layer_id: int, run_ids: List[int], dtype):
        super().__init__()
        lc = config.layers[layer_id]
        W = config.hidden_size
        self.mix = TigotarMixer(W, lc.mixer, config.norm_eps, run_ids, dtype)
        self.norm1, self.norm1b = DynTanh(W, dtype), DynTanh(W, dtype)
        self.mlp = UngatedMoE(lc.experts, lc.top, W, lc.ff, "relu2", params_dtype=dtype) if lc.experts else None
        self.norm2 = DynTanh(W, dtype) if lc.experts else None
        self.norm2b = DynTanh(W, dtype) if lc.experts else None

    def forward(self, x: torch.Tensor, h: Optional[torch.Tensor], forward_batch, run: int,
                next_norm: Optional[DynTanh]) -> Optional[torch.Tensor]:
        """x: the fp32 stream (updated in place); h: norm1(x) in the activation type when the previous seam made it.
        Returns next_norm(x) in the activation type (None without next_norm)."""
        if h is None:
            h = self.norm1.read_stream(x)
        y = self.mix(h, forward_batch, run)
        if self.mlp is None:
            return self.norm1b.seam(y, x, next_norm, want_out=next_norm is not None)
        h = self.norm1b.seam(y, x, self.norm2)
        return self.norm2b.seam(self.mlp(h), x, next_norm, want_out=next_norm is not None)


class TigotarForCausalLM(nn.Module):
    def __init__(self, config: TigotarConfig, dtype=torch.bfloat16):
        super().__init__()
        if get_tensor_model_parallel_world_size() != 1:
            raise ValueError("Tigotar runs on one GPU per replica (tensor parallelism over its per-layer head counts and its "
                             "recurrent channels is not implemented)")
        if not config.layers:
            raise ValueError("Tigotar: the configuration lists no layers")
        self.config = config
        self.runs = config.runs()
        W = config.hidden_size
        self.embed = VocabParallelEmbedding(config.vocab_size, W, params_dtype=dtype)
        self.embed_norm = DynTanh(W, dtype)
        by_layer: Dict[int, List[int]] = {}
        for r in self.runs:
            by_layer.setdefault(r.layer, []).append(r.run)
        self.layers = nn.ModuleList([TigotarDecoderLayer(config, i, by_layer.get(i, []), dtype) for i in range(len(config.layers))])
        if config.has_loop:
            self.loop_in = RowParallelLinear(2 * W, W, params_dtype=dtype)       # columns: the stream, then the embedding output
            self.loop_step = nn.Parameter(torch.zeros(config.loop_times, W, dtype=torch.float32), requires_grad=False)
        self.final_norm = DynTanh(W, dtype)
        self.head = ParallelLMHead(config.vocab_size, W, params_dtype=dtype)
        self.logits_processor = LogitsProcessor(config.vocab_size, logit_scale=config.logit_scale)
        self.layer_probe = None      # tests: a callable (run index, fp32 stream) run after every layer run
        self._mm_f32_out = None      # whether torch.mm takes 16-bit operands with an fp32 result on this build
        for p in self.parameters():
            p.requires_grad_(False)

    def post_load_weights(self):
        for layer in self.layers:
            if layer.mlp is not None:
                layer.mlp.post_load_weights()

    @property
    def kv_geometry(self):
        ms = [self.config.layers[r.layer].mixer.left for r in self.runs]
        return dict(kind="mha", num_kv_heads=[m.kv_heads for m in ms], head_dim=[m.dim for m in ms],
                    v_head_dim=[m.vdim for m in ms], num_heads=[m.heads for m in ms], num_layers=len(ms))

    @property
    def state_geometry(self) -> List[int]:
        """Width of the recurrent state of every layer run (the state pool gives each a column range)."""
        return [self.config.layers[r.layer].mixer.right_width for r in self.runs]

    def _enter_pass(self, x: torch.Tensor, x0: torch.Tensor, t: int) -> torch.Tensor:
        """x <- W_in [x; x0] + step[t] as a new fp32 stream: operands in the activation type, fp32 accumulation, and the
        result is NOT rounded to the activation type on its way into the stream."""
        w = self.loop_in.weight
        both = torch.cat([x, x0], -1).to(w.dtype)
        if w.dtype == torch.float32:
            y = F.linear(both, w)
        else:
            if self._mm_f32_out is None:
                try:
                    torch.mm(both[:1], w.t(), out_dtype=torch.float32)
                    self._mm_f32_out = True
                except (TypeError, RuntimeError):
                    self._mm_f32_out = False
                    self._loop_in_f32 = w.float()
            y = torch.mm(both, w.t(), out_dtype=torch.float32) if self._mm_f32_out else F.linear(both.float(), self._loop_in_f32)
        return y.add_(self.loop_step[t])

    @torch.no_grad()
    def forward(self, input_ids, positions, forward_batch):
        e = self.embed(input_ids)
        x0 = torch.empty(e.shape, dtype=torch.float32, device=e.device)
        self.embed_norm.forward_stream(e, x0)
        x = x0.clone() if self.config.has_loop else x0          # the stream is updated in place; passes re-read x0
        h = None
        for n, r in enumerate(self.runs):
            if r.enters_pass:
                x = self._enter_pass(x, x0, r.loop_pass)
                h = None
            nxt = self.runs[n + 1] if n + 1 < len(self.runs) else None
            next_norm = self.final_norm if nxt is None else (None if nxt.enters_pass else self.layers[nxt.layer].norm1)
            h = self.layers[r.layer](x, h, forward_batch, r.run, next_norm)
            if self.layer_probe is not None:
                self.layer_probe(r.run, x)
        if h is None:      # (no layer runs at all: only reachable with an empty layer list, refused above)
            h = self.final_norm.read_stream(x)
        return self.logits_processor(input_ids, h, self.head, forward_batch)
