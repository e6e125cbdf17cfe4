"""Kudirax on the GPU against the plain host statement of its mechanisms (oracle/kudirax.py).

Op level: unit norm + blend + pool store, block-local attention with a sink (one-wave-per-row form in fp32 / bf16, the
matrix-core prompt and decode forms in bf16 / f16), LayerNorm + residual, squared ReLU -- each alone, with pool slots in
random order and inputs built so that one key just inside or just outside a block's edge, or far back, dominates.
Model level: small configurations of this file's own (layers of different head counts and sizes, a layer without
feed-forward, the first blending layer not the first layer, a vocabulary that needs padding) through the replay
scheduler: whole prompts, token-by-token decoding through the captured graphs, portions down to two tokens, batches of
unequal requests, rows and slots that are given back and used again; and greedy generation through the Engine.
"""
import json
import os

import pytest
import torch

from oracle import kudirax as K

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


# ----------------------------------------------------------------------------------------------- op level
def _attention_case(H, G, D, E, chunk, cap, dtype, form, reqs, seed=0, with_sink=True, with_gate=True, decode=False,
                    standout=None):
    """reqs: [(prefix, extend)].  Sequences are laid out in the pools through a random slot order; returns what the
    kernel and the oracle make of the same rounded inputs."""
    from semi_pd_amd import ops
    g = torch.Generator().manual_seed(seed)
    total = sum(p + e for p, e in reqs)
    n_slots = total + 7
    perm = (torch.randperm(n_slots - 1, generator=g) + 1)[:total]
    kp = torch.zeros(n_slots, G, D, dtype=dtype)
    vp = torch.zeros(n_slots, G, E, dtype=dtype)
    max_len = max(p + e for p, e in reqs)
    r2t = torch.zeros(len(reqs) + 3, max_len + 4, dtype=torch.int32)
    rows = torch.randperm(len(reqs) + 3, generator=g)[: len(reqs)]
    scale = D ** -0.5
    sink = torch.randn(H, generator=g) if with_sink else None
    q_all, gate_all, want, at = [], [], [], 0
    for b, (pre, ext) in enumerate(reqs):
        n = pre + ext
        q = torch.randn(n, H, D, generator=g)
        k = torch.randn(n, G, D, generator=g)
        v = torch.randn(n, G, E, generator=g)
        if standout is not None:
            # the query at `qi` points along one direction; key `kj` points the same way, strongly, and carries values that
            # cannot be missed if it is wrongly seen -- or wrongly left out
            for queries, keys in standout(pre, ext):
                d = torch.randn(D, generator=g)
                d = d / d.norm() * D ** 0.5
                for qi in queries:
                    q[qi] = d
                for kj, strength, val in keys:
                    k[kj] = strength * d
                    v[kj] = val
        q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
        slots = perm[at: at + n]
        at += n
        kp[slots], vp[slots] = k, v
        r2t[rows[b], :n] = slots.int()
        gate = torch.randn(n, H * E, generator=g).to(dtype)
        ref = K.local_attention(q, k, v, scale, cap, chunk or None, sink).reshape(n, H * E)
        if with_gate:
            ref = ref * torch.sigmoid(gate.float())
        want.append(ref[pre:])
        q_all.append(q[pre:].reshape(ext, H * D))
        gate_all.append(gate[pre:])
    q_cat, gate_cat = torch.cat(q_all).to(DEV), torch.cat(gate_all).to(DEV)
    out = torch.empty(q_cat.shape[0], H * E, dtype=dtype, device=DEV)
    ext_lens = [e for _, e in reqs]
    starts = [sum(ext_lens[:i]) for i in range(len(reqs))]
    if decode:
        assert all(e == 1 for e in ext_lens)
        q_start = q_len = None
    else:
        q_start = torch.tensor(starts, dtype=torch.int32, device=DEV)
        q_len = torch.tensor(ext_lens, dtype=torch.int32, device=DEV)
    ops.local_attention_fwd(q_cat, out, kp.to(DEV), vp.to(DEV), r2t.to(DEV), rows.to(DEV), torch.tensor(
        [p + e for p, e in reqs], dtype=torch.int64, device=DEV), q_start, q_len, max(ext_lens), scale, cap, chunk,
        sink.to(DEV) if sink is not None else None, gate_cat if with_gate else None, form=form)
    return out.float().cpu(), torch.cat(want)


REQS = [(0, 1), (0, 70), (63, 2), (64, 65), (100, 1), (5, 130), (31, 3)]
TOL = {torch.float32: dict(rtol=2e-5, atol=2e-5), torch.bfloat16: dict(rtol=3e-2, atol=3e-2),
       torch.float16: dict(rtol=4e-3, atol=4e-3)}


@pytest.mark.parametrize("chunk", [0, 1, 5, 32, 33, 64, 1000])
@pytest.mark.parametrize("dtype,form", [(torch.float32, 1), (torch.bfloat16, 1), (torch.bfloat16, 2), (torch.float16, 2)])
def test_attention_every_block_size(chunk, dtype, form):
    got, want = _attention_case(4, 2, 64, 32, chunk, 12.0, dtype, form, REQS, seed=chunk)
    torch.testing.assert_close(got, want, **TOL[dtype])


@pytest.mark.parametrize("H,G,D,E", [(4, 4, 96, 64), (8, 2, 128, 128), (2, 1, 256, 256), (3, 1, 32, 16), (32, 1, 64, 32),
                                     (6, 3, 160, 80), (40, 2, 32, 48)])
@pytest.mark.parametrize("dtype,form", [(torch.bfloat16, 2), (torch.float32, 1)])
def test_attention_head_counts_and_sizes(H, G, D, E, dtype, form):
    """Sizes in every template range of the matrix-core forms (<= 128, above), groups of one, of 16 and more q heads."""
    for decode in (False, True):
        reqs = [(70, 1), (0, 1), (129, 1), (33, 1)] if decode else [(0, 40), (70, 30), (16, 1)]
        got, want = _attention_case(H, G, D, E, 48, 20.0, dtype, form, reqs, seed=H + D, decode=decode)
        torch.testing.assert_close(got, want, **TOL[dtype])


@pytest.mark.parametrize("D,E", [(40, 24), (100, 7), (512, 8)])
def test_attention_sizes_only_the_row_form_takes(D, E):
    from semi_pd_amd import ops
    assert not ops.local_attention_mfma_supported(4, 2, D, E, torch.bfloat16)
    for dtype in (torch.bfloat16, torch.float32):
        got, want = _attention_case(4, 2, D, E, 16, 8.0, dtype, 0, [(0, 35), (20, 1), (17, 9)], seed=D)
        torch.testing.assert_close(got, want, **TOL[dtype])


@pytest.mark.parametrize("dtype,form", [(torch.float32, 1), (torch.bfloat16, 1), (torch.bfloat16, 2)])
@pytest.mark.parametrize("decode", [False, True])
def test_attention_edges_of_a_block_stand_out(dtype, form, decode):
    """For queries at the start, the end and the middle of a block: the key just OUTSIDE the block (the position before the
    block's first) matches the query far better than any other and carries large values; the block's first key matches
    well and carries its own.  A mask that is one position off moves the result by orders of magnitude."""
    chunk = 24

    def standout(pre, ext):
        qi = pre + ext - 1
        lo = (qi // chunk) * chunk
        keys = [(lo, 3.0, -3.0)] if lo < qi else []
        if lo > 0:
            keys.append((lo - 1, 6.0, 200.0))
        return [([qi], keys)]

    reqs = [(p, 1) for p in (23, 24, 25, 47, 48, 71, 100, 0)] if decode else [(0, 24), (0, 25), (0, 49), (40, 9), (47, 2), (20, 77)]
    got, want = _attention_case(2, 1, 32, 32, chunk, 0.0, dtype, form, reqs, seed=3, standout=standout, decode=decode)
    last = torch.tensor([e for _, e in reqs]).cumsum(0) - 1
    assert want[last].abs().max() < 50      # the outside key's values are nowhere in the truth of the rows it was built for
    torch.testing.assert_close(got, want, **TOL[dtype])


@pytest.mark.parametrize("dtype,form", [(torch.float32, 1), (torch.bfloat16, 2)])
def test_attention_far_key_and_sink(dtype, form):
    """No blocks: a key hundreds of positions back dominates the last queries; with and without the sink term (a large
    positive sink takes most of the weight away, so leaving it out shows)."""
    def standout(pre, ext):
        return [([pre + ext - 1, pre + ext - 2], [(3, 4.0, 5.0)])]

    for with_sink in (True, False):
        got, want = _attention_case(2, 2, 64, 32, 0, 30.0, dtype, form, [(0, 700), (650, 2)], seed=9, standout=standout,
                                    with_sink=with_sink, with_gate=False)
        torch.testing.assert_close(got, want, **TOL[dtype])
        assert want[-1].abs().mean() > 0.5


@pytest.mark.parametrize("decode", [False, True])
def test_attention_more_keys_than_the_slot_copy_holds(decode):
    """Over 2048 visible keys (no blocks, and blocks of 2304): the matrix-core forms then read the slots from the table
    instead of their copy in LDS; the key at position 5 dominates the last query."""
    def standout(pre, ext):
        return [([pre + ext - 1], [(5, 4.0, 3.0)])]

    for chunk in (0, 2304):
        reqs = [(2499, 1), (2100, 1), (40, 1)] if decode else [(0, 2300), (2290, 3)]
        got, want = _attention_case(2, 1, 32, 16, chunk, 25.0, torch.bfloat16, 2, reqs, seed=4, standout=standout, decode=decode)
        torch.testing.assert_close(got, want, **TOL[torch.bfloat16])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,D,E", [(4, 2, 64, 32), (3, 3, 40, 24), (2, 1, 96, 200)])
def test_unit_norm_blend_and_store(dtype, H, G, D, E):
    from semi_pd_amd import ops
    g = torch.Generator().manual_seed(H * D)
    T, eps = 37, 1e-5
    cols = H * D + G * D + G * E + 16
    qkv = (torch.randn(T, cols, generator=g) * 3).to(dtype)
    v0 = torch.randn(T, G * E, generator=g).to(dtype)
    mix = torch.tensor(0.3125, dtype=dtype)
    loc = (torch.randperm(60, generator=g) + 1)[:T]
    for blend in (False, True):
        kp = torch.zeros(64, G, D, dtype=dtype, device=DEV)
        vp = torch.zeros(64, G, E, dtype=dtype, device=DEV)
        x = qkv.clone().to(DEV)
        ops.unit_norm_and_store_kv(x, H, G, D, E, H * D, H * D + G * D, eps, kp, vp, loc.to(DEV),
                                   v_first=v0.to(DEV) if blend else None, mix=mix.to(DEV) if blend else None)
        q_ref = K.unit_rms(qkv[:, : H * D].view(T, H, D), eps).reshape(T, H * D)
        k_ref = K.unit_rms(qkv[:, H * D: H * D + G * D].view(T, G, D), eps)
        v_ref = qkv[:, H * D + G * D: H * D + G * D + G * E].float()
        if blend:
            v_ref = (1 - mix.float()) * v_ref + mix.float() * v0.float()
        tol = TOL[dtype]
        torch.testing.assert_close(x[:, : H * D].float().cpu(), q_ref, **tol)
        torch.testing.assert_close(kp[loc.to(DEV)].float().cpu(), k_ref, **tol)
        torch.testing.assert_close(vp[loc.to(DEV)].float().cpu().reshape(T, G * E), v_ref, **tol)
        assert torch.equal(x[:, H * D:].cpu(), qkv[:, H * D:])            # k, v and what follows stay as projected
        untouched = torch.ones(64, dtype=torch.bool)
        untouched[loc] = False
        assert kp.cpu()[untouched].abs().sum() == 0 and vp.cpu()[untouched].abs().sum() == 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [48, 192, 1000])
def test_layernorm_residual_and_squared_relu(dtype, width):
    from semi_pd_amd import ops
    g = torch.Generator().manual_seed(width)
    T, eps = 19, 1e-5
    y = (torch.randn(T, width, generator=g) * 4 + 1).to(dtype)
    w, b, ib = [(torch.randn(width, generator=g) * s + o).to(dtype) for s, o in ((0.2, 1.0), (0.3, 0.0), (0.5, 0.0))]
    res = torch.randn(T, width, generator=g) * 5
    tol = TOL[dtype]
    out = ops.layernorm(y.to(DEV), w.to(DEV), b.to(DEV), eps)
    torch.testing.assert_close(out.float().cpu(), K.layer_norm(y, w, b, eps), **tol)
    r = res.clone().to(DEV)
    out = ops.layernorm(y.to(DEV), w.to(DEV), b.to(DEV), eps, residual=r, in_bias=ib.to(DEV))
    want = res + K.layer_norm(y.float() + ib.float(), w, b, eps)
    torch.testing.assert_close(r.cpu(), want, rtol=2e-5, atol=2e-5)       # the stream stays fp32 whatever the type
    torch.testing.assert_close(out.float().cpu(), want, **tol)
    out = ops.layernorm(res.to(DEV), w.to(DEV), b.to(DEV), eps)          # fp32 rows in, activation type out
    torch.testing.assert_close(out.float().cpu(), K.layer_norm(res, w, b, eps), **tol)
    u = y.clone().to(DEV)
    ops.bias_relu_square_(u, ib.to(DEV))
    torch.testing.assert_close(u.float().cpu(), torch.relu(y.float() + ib.float()) ** 2, **tol)


# ----------------------------------------------------------------------------------------------- model level
def _mixer(heads, kv_heads, dim, vdim, chunk, softcap, v_mix, scale=None):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": chunk}, "softcap": softcap,
            "scale": scale if scale is not None else dim ** -0.5, "v_mix": v_mix}


CONFIGS = {
    # layers of their own geometry; the first blending layer is layer 1; a layer without feed-forward; sizes that only the
    # row form takes next to sizes of the matrix-core forms; a vocabulary that is padded
    "mixed": {"architecture": "Kudirax", "vocab": 300, "width": 128, "norm": {"eps": 1e-5}, "layers": [
        {"type": "attention", "mixer": _mixer(4, 2, 64, 32, 16, 15.0, False), "mlp": {"kind": "dense", "ff": 256}},
        {"type": "attention", "mixer": _mixer(4, 2, 64, 32, 48, 25.0, True), "mlp": None},
        {"type": "attention", "mixer": _mixer(8, 2, 40, 32, 5, 10.0, True, scale=0.21), "mlp": {"kind": "dense", "ff": 192}},
        {"type": "attention", "mixer": _mixer(2, 2, 32, 32, 64, 30.0, True), "mlp": {"kind": "dense", "ff": 128}}]},
    # one head, a block of one position, equal sizes, a single layer that does not blend
    "minimal": {"architecture": "Kudirax", "vocab": 64, "width": 64, "norm": {"eps": 1e-6}, "layers": [
        {"type": "attention", "mixer": _mixer(1, 1, 64, 64, 1, 5.0, False), "mlp": {"kind": "dense", "ff": 64}},
        {"type": "attention", "mixer": _mixer(1, 1, 64, 64, 7, 5.0, True), "mlp": {"kind": "dense", "ff": 64}}]},
    # nothing a multiple of 8: width, vocabulary, head sizes, feed-forward; no layer blends; a block longer than any prompt here
    "awkward": {"architecture": "Kudirax", "vocab": 301, "width": 100, "norm": {"eps": 1e-4}, "layers": [
        {"type": "attention", "mixer": _mixer(3, 1, 24, 20, 3, 7.0, False), "mlp": {"kind": "dense", "ff": 130}},
        {"type": "attention", "mixer": _mixer(5, 5, 12, 36, 500, 50.0, False, scale=0.4), "mlp": None},
        {"type": "attention", "mixer": _mixer(2, 1, 50, 6, 11, 3.0, False), "mlp": {"kind": "dense", "ff": 36}}]},
}


def _write_checkpoint(path, cfg, seed):
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    w = K.random_weights(cfg, seed)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in w.items()}, os.path.join(path, "model.safetensors"))
    return w


def _scheduler(path, dtype, max_tokens, max_requests=4, graphs=True):
    from semi_pd_amd.entrypoints.engine import _build_runner
    from semi_pd_amd.managers.replay_scheduler import ReplayScheduler
    from semi_pd_amd.semi_pd.utils import InstanceRole
    from semi_pd_amd.server_args import ServerArgs
    sa = ServerArgs(model_path=path, load_format="auto", dtype=dtype, context_length=max_tokens, max_total_tokens=max_tokens,
                    max_running_requests=max_requests, cuda_graph_max_bs=max_requests, disable_cuda_graph=not graphs,
                    skip_tokenizer_init=True)
    mr = _build_runner(sa, 0, 0, InstanceRole.OTHER, 29650, max_total_tokens=max_tokens)
    mr.init_attention_backend()
    mr.init_cuda_graphs()
    return ReplayScheduler(sa, mr)


def _tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def _run_schedule(sched, prompts, schedule):
    """schedule: steps of [(request name, token count)]; every position's logits are asked for.  Returns name -> [T, vocab]."""
    at = {n: 0 for n in prompts}
    got = {n: [] for n in prompts}
    for step in schedule:
        entries, end = [], []
        for name, count in step:
            lo, hi = at[name], at[name] + count
            entries.append({"id": name, "tokens": prompts[name][lo:hi], "want": list(range(count))})
            at[name] = hi
            if hi == len(prompts[name]):
                end.append(name)
        logits = sched.replay_step(entries, end).cpu()
        k = 0
        for name, count in step:
            got[name].append(logits[k: k + count])
            k += count
    assert all(at[n] == len(prompts[n]) for n in prompts)
    return {n: torch.cat(v) for n, v in got.items()}


def _rel_err(got, want):
    d = (got - want) - (got - want).mean(-1, keepdim=True)
    return (d.pow(2).mean(-1).sqrt() / want.std(-1)).max().item()


LIMIT = {"float32": 5e-5, "bfloat16": 6e-2}


@pytest.fixture(scope="module", params=["float32", "bfloat16"])
def mixed_model(request, tmp_path_factory):
    path = str(tmp_path_factory.mktemp("kudirax_mixed"))
    cfg = CONFIGS["mixed"]
    w = _write_checkpoint(path, cfg, seed=11)
    # a pool far smaller than the tokens that pass through it: slots and rows come back and are used again all the time
    sched = _scheduler(path, request.param, max_tokens=448)
    lens = {"a": 150, "b": 1, "c": 97, "d": 2, "e": 64, "f": 131}
    prompts = {n: _tokens(k, cfg["vocab"], seed=ord(n)) for n, k in lens.items()}
    truth = {n: K.forward(cfg, w, t) for n, t in prompts.items()}
    return request.param, sched, prompts, truth


def test_whole_prompts_match_the_plain_model(mixed_model):
    dtype, sched, prompts, truth = mixed_model
    got = _run_schedule(sched, prompts, [[(n, len(t))] for n, t in prompts.items()])
    for n in prompts:
        assert _rel_err(got[n], truth[n]) < LIMIT[dtype], n
    assert sched.token_to_kv_pool_allocator.available_size() == 448 and sched.req_to_token_pool.available_size() == 5


def test_decoding_token_by_token_matches_the_prompt_pass(mixed_model):
    """Ten tokens as a prompt, then one token per step through the captured decode graphs: past several edges of every
    layer's blocks (5, 16, 48, 64), 140 steps long."""
    dtype, sched, prompts, truth = mixed_model
    for n in ("a", "f", "d"):
        T = len(prompts[n])
        first = min(10, T - 1)
        got = _run_schedule(sched, {n: prompts[n]}, [[(n, first)]] + [[(n, 1)] for _ in range(T - first)])
        assert _rel_err(got[n], truth[n]) < LIMIT[dtype], n
    assert sched.stats["decode_steps"] > 0


def test_portions_of_every_size_down_to_two(mixed_model):
    dtype, sched, prompts, truth = mixed_model
    sizes = [2, 3, 5, 16, 31, 2, 48, 7, 64, 1, 2]
    for n in ("a", "c", "f"):
        T, sched_steps, at, i = len(prompts[n]), [], 0, 0
        while at < T:
            k = min(sizes[i % len(sizes)], T - at)
            sched_steps.append([(n, k)])
            at, i = at + k, i + 1
        got = _run_schedule(sched, {n: prompts[n]}, sched_steps)
        assert _rel_err(got[n], truth[n]) < LIMIT[dtype], n


def test_unequal_requests_side_by_side_with_reuse(mixed_model):
    """Up to four live requests: portions of some next to single tokens of others, requests that sit a step out, requests
    that end while others go on, new ones taking their rows and slots."""
    dtype, sched, prompts, truth = mixed_model
    schedule = [
        [("a", 16), ("b", 1), ("c", 3)],
        [("a", 49), ("c", 16)],
        [("a", 1), ("c", 2), ("d", 1)],
        [("a", 1), ("c", 30), ("d", 1), ("e", 33)],
        [("c", 1), ("e", 1), ("f", 100)],              # a sits out; b and d are gone, their rows are e's and f's now
        [("a", 1), ("c", 1), ("e", 1), ("f", 1)],      # four single tokens: a decode batch
        [("a", 1), ("c", 1), ("e", 1), ("f", 1)],
        [("a", 70), ("c", 2), ("e", 28), ("f", 29)],
        [("a", 11), ("c", 41)],
    ]
    got = _run_schedule(sched, prompts, schedule)
    for n in prompts:
        assert _rel_err(got[n], truth[n]) < LIMIT[dtype], n
    assert sched.token_to_kv_pool_allocator.available_size() == 448 and not sched.live


def test_logits_do_not_depend_on_the_cut_or_the_neighbours(mixed_model):
    """The same request alone and whole, and in a batch cut into portions: equal up to rounding (fp32: ~1e-6)."""
    dtype, sched, prompts, truth = mixed_model
    alone = _run_schedule(sched, {"c": prompts["c"]}, [[("c", 97)]])["c"]
    mixed = _run_schedule(sched, {k: prompts[k] for k in "ce"}, [[("c", 40), ("e", 3)], [("c", 1), ("e", 60)], [("c", 56), ("e", 1)]])["c"]
    assert _rel_err(mixed, alone) < (2e-5 if dtype == "float32" else 5e-2)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_minimal_sizes(dtype, tmp_path):
    """Heads, groups and block sizes of one; key and value sizes equal; a layer list where nothing blends first."""
    cfg = CONFIGS["minimal"]
    w = _write_checkpoint(str(tmp_path), cfg, seed=5)
    sched = _scheduler(str(tmp_path), dtype, max_tokens=128, graphs=False)
    prompts = {"x": _tokens(40, 64, 1), "y": _tokens(9, 64, 2)}
    got = _run_schedule(sched, prompts, [[("x", 7), ("y", 2)], [("x", 1), ("y", 1)], [("x", 1), ("y", 1)], [("x", 31), ("y", 5)]])
    for n, t in prompts.items():
        assert _rel_err(got[n], K.forward(cfg, w, t)) < LIMIT[dtype], n


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_awkward_sizes(dtype, tmp_path):
    """Sizes that no vector path takes (width 100, value size 20, a vocabulary of 301): every kernel's plain form, the
    library GEMMs at odd shapes, the decode graphs."""
    cfg = CONFIGS["awkward"]
    w = _write_checkpoint(str(tmp_path), cfg, seed=8)
    sched = _scheduler(str(tmp_path), dtype, max_tokens=192)
    prompts = {"x": _tokens(70, 301, 3), "y": _tokens(23, 301, 4), "z": _tokens(1, 301, 5)}
    got = _run_schedule(sched, prompts, [[("x", 30), ("y", 2), ("z", 1)], [("x", 1), ("y", 1)], [("x", 1), ("y", 1)],
                                         [("x", 37), ("y", 19)], [("x", 1)]])
    for n, t in prompts.items():
        assert _rel_err(got[n], K.forward(cfg, w, t)) < LIMIT[dtype], n


def _check_generation(cfg, w, prompts, outs, steps):
    exact = 0
    for p, o in zip(prompts, outs):
        assert len(o) == steps
        logits = K.forward(cfg, w, p + o)
        for i, tok in enumerate(o):
            row = logits[len(p) + i - 1]
            assert row[tok] >= row.max() - 0.08 * row.std(), (len(p), i)
            exact += int(row.argmax().item() == tok)
    assert exact > 0.9 * steps * len(prompts)


def test_greedy_generation_through_the_engine(tmp_path):
    """Prompts of unequal length through Engine.generate (the unified scheduler: chunked prefill, decode graphs, sampler):
    every generated token is the plain model's argmax given the tokens before it, or within a small margin of it."""
    from semi_pd_amd.entrypoints.engine import Engine
    from semi_pd_amd.managers.io_struct import SamplingParams
    from semi_pd_amd.server_args import ServerArgs
    cfg = CONFIGS["mixed"]
    w = _write_checkpoint(str(tmp_path), cfg, seed=21)
    prompts = [_tokens(n, cfg["vocab"], seed=n) for n in (3, 70, 33, 1, 120)]
    sa = ServerArgs(model_path=str(tmp_path), load_format="auto", dtype="bfloat16", context_length=256, max_total_tokens=1024,
                    max_running_requests=8, cuda_graph_max_bs=8, chunked_prefill_size=64, skip_tokenizer_init=True)
    eng = Engine(sa)
    try:
        outs = eng.generate(prompts, SamplingParams(max_new_tokens=24, ignore_eos=True), timeout=300)
    finally:
        eng.shutdown()
    _check_generation(cfg, w, prompts, outs, 24)


def test_greedy_generation_through_the_semi_pd_engine(tmp_path):
    """The same through a prefill and a decode process on one GPU: the per-layer pool regions and every parameter (the fp32
    sinks, the blend weights) reach the prefill process through IPC handles; prompts are cut into 48-token portions there and
    decoded in the other process."""
    from semi_pd_amd.entrypoints.engine import Engine
    from semi_pd_amd.managers.io_struct import SamplingParams
    from semi_pd_amd.server_args import ServerArgs
    cfg = CONFIGS["mixed"]
    w = _write_checkpoint(str(tmp_path), cfg, seed=22)
    prompts = [_tokens(n, cfg["vocab"], seed=100 + n) for n in (5, 90, 47, 130)]
    sa = ServerArgs(model_path=str(tmp_path), load_format="auto", dtype="bfloat16", context_length=256, max_total_tokens=2048,
                    max_running_requests=8, cuda_graph_max_bs=8, chunked_prefill_size=48, skip_tokenizer_init=True,
                    enable_semi_pd=True, cu_mask_mode="env", prefill_cu_percent=50, decode_cu_percent=50, tune_prefill_gemm=False,
                    watchdog_timeout=120.0)
    eng = Engine(sa)
    try:
        outs = eng.generate(prompts, SamplingParams(max_new_tokens=16, ignore_eos=True), timeout=300)
    finally:
        eng.shutdown()
    _check_generation(cfg, w, prompts, outs, 16)
