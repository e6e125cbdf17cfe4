"""Tigotar on the GPU against the plain host statement of its mechanisms (oracle/tigotar.py).

Op level: DynTanh seams, bias + pair rotation + value norm + pool store, sliding-window attention with kept first positions
and sigmoid weights (one-wave-per-row form in fp32 / bf16, the matrix-core prompt and decode forms in bf16 / f16), the
minGRU recurrence over pooled state rows (row-walking and chunked forms), the ungated mixture of experts (grouped and
side-by-side forms) -- each alone, with pool slots in random order and inputs built so that one key just inside or just
outside the window, among the kept first positions or just behind them, or far back, dominates.
Model level: small configurations of this file's own (layers of different head counts and sizes, a layer without experts, a
repeated span, no repeated span, a partial rotation, sizes of one, sizes no vector path takes) through the replay
scheduler: whole prompts, token-by-token decoding through the captured graphs, portions down to two tokens, batches of
unequal requests, rows, slots and state rows that are given back and used again; and greedy generation through the Engine.
"""
import json
import os

import pytest
import torch

from oracle import tigotar as P

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = {torch.float32: dict(rtol=3e-5, atol=3e-5), torch.bfloat16: dict(rtol=3e-2, atol=3e-2),
       torch.float16: dict(rtol=4e-3, atol=4e-3)}


# ----------------------------------------------------------------------------------------------- DynTanh
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,width", [(1, 8), (5, 100), (37, 256), (3, 4104)])
def test_dyn_tanh_seam(dtype, rows, width):
    from semi_pd_amd import ops
    g = torch.Generator().manual_seed(width)
    w = {}
    for n in ("a", "b"):
        w[n], w[n + ".b"] = (1 + 0.2 * torch.randn(width, generator=g)).to(dtype), (0.3 * torch.randn(width, generator=g)).to(dtype)
        w[n + ".alpha"] = torch.tensor(0.4 if n == "a" else 1.3).to(dtype)
    prm = {n: tuple(w[k].to(DEV) for k in (n, n + ".b", n + ".alpha")) for n in ("a", "b")}
    y = (2 * torch.randn(rows, width, generator=g)).to(dtype)
    x = 3 * torch.randn(rows, width, generator=g)
    # squash(y) alone; start of a stream; stream += squash_a(y) and squash_b of the sum; squash of the stream alone
    torch.testing.assert_close(ops.dyn_tanh(y.to(DEV), prm["a"]).float().cpu(), P.dyn_tanh(y, w, "a").to(dtype).float(), **TOL[dtype])
    res = torch.full((rows, width), 7.0, device=DEV)
    assert ops.dyn_tanh(y.to(DEV), prm["a"], residual=res, accumulate=False, want_out=False) is None
    torch.testing.assert_close(res.cpu(), P.dyn_tanh(y, w, "a"), rtol=1e-5, atol=1e-5)
    res = x.to(DEV)
    out = ops.dyn_tanh(y.to(DEV), prm["a"], residual=res, params_out=prm["b"])
    want_x = x + P.dyn_tanh(y, w, "a")
    torch.testing.assert_close(res.cpu(), want_x, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(out.float().cpu(), P.dyn_tanh(want_x, w, "b"), **TOL[dtype])
    out = ops.dyn_tanh(None, None, residual=res, params_out=prm["b"])
    torch.testing.assert_close(res.cpu(), want_x, rtol=1e-5, atol=1e-5)       # reading leaves the stream alone
    torch.testing.assert_close(out.float().cpu(), P.dyn_tanh(want_x, w, "b"), **TOL[dtype])
    out = ops.dyn_tanh(y.to(DEV), prm["a"], residual=res)                     # no second squashing: the sum itself
    torch.testing.assert_close(out.float().cpu(), want_x + P.dyn_tanh(y, w, "a"), **TOL[dtype])


# ----------------------------------------------------------------------------------------------- bias + rotation + value norm + store
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,D,E,rot", [(4, 2, 32, 16, 32), (3, 1, 20, 12, 10), (2, 2, 64, 256, 2), (1, 1, 128, 100, 0), (2, 1, 8, 500, 4), (6, 2, 96, 160, 96), (2, 2, 64, 64, 16),
                                         (5, 5, 160, 8, 96)])
def test_bias_rotation_value_norm_store(dtype, H, G, D, E, rot):
    from semi_pd_amd import ops
    g = torch.Generator().manual_seed(D + rot)
    T, N, eps, base = 11, 40, 1e-5, 5000.0
    extra = 24                                           # columns of another mixer behind q | k | v
    row = torch.randn(T, H * D + G * D + G * E + extra, generator=g).to(dtype)
    bq, bk, bv = (torch.randn(n, generator=g).to(dtype) for n in (H * D, G * D, G * E))
    pos = torch.tensor([0, 1, 2, 3, 500, 501, 77, 4000, 4001, 9, 10])
    loc = (torch.randperm(N - 1, generator=g) + 1)[:T]
    inv_freq = base ** (-2.0 * torch.arange(rot // 2, dtype=torch.float32) / max(rot, 1))
    kp, vp = torch.zeros(N, G, D, dtype=dtype, device=DEV), torch.zeros(N, G, E, dtype=dtype, device=DEV)
    dev_row = row.to(DEV)
    ops.bias_rope_vnorm_kv_store(dev_row, H, G, D, E, H * D, H * D + G * D, bq.to(DEV), bk.to(DEV), bv.to(DEV), pos.to(DEV),
                                 inv_freq.to(DEV) if rot else None, rot, eps, kp, vp, loc.to(DEV))

    def rotated(x, n):          # the oracle rotates positions 0 .. T-1 of one sequence: one call per token at its own position
        x = x.view(T, n, D)
        return torch.stack([P.rotate_pairs(x[t: t + 1].expand(int(pos[t]) + 1, n, D), base, rot)[-1] if rot else x[t]
                            for t in range(T)])

    q = rotated(row[:, : H * D].float() + bq.float(), H)
    k = rotated(row[:, H * D: H * D + G * D].float() + bk.float(), G)
    v = P.unit_rms((row[:, H * D + G * D: H * D + G * D + G * E].float() + bv.float()).view(T, G, E), eps)
    tol = TOL[dtype]
    torch.testing.assert_close(dev_row[:, : H * D].float().cpu().view(T, H, D), q, **tol)
    torch.testing.assert_close(kp[loc.to(DEV)].float().cpu(), k, **tol)
    torch.testing.assert_close(vp[loc.to(DEV)].float().cpu(), v, **tol)
    assert torch.equal(dev_row[:, H * D:].cpu(), row[:, H * D:])              # only q is rewritten in place
    untouched = torch.ones(N, dtype=torch.bool)
    untouched[loc] = False
    assert kp[untouched.to(DEV)].abs().max() == 0 and vp[untouched.to(DEV)].abs().max() == 0


# ----------------------------------------------------------------------------------------------- window attention
def _window_case(H, G, D, E, window, keep, dtype, form, reqs, seed=0, decode=False, standout=None, bias=-1.0, out_scale=1.0):
    """reqs: [(prefix, extend)].  Sequences are laid out in the pools through a random slot order; returns what the kernel
    and the oracle make of the same rounded inputs."""
    from semi_pd_amd import ops
    g = torch.Generator().manual_seed(seed)
    total = sum(p + e for p, e in reqs)
    n_slots = total + 7
    perm = (torch.randperm(n_slots - 1, generator=g) + 1)[:total]
    kp, vp = torch.zeros(n_slots, G, D, dtype=dtype), torch.zeros(n_slots, G, E, dtype=dtype)
    max_len = max(p + e for p, e in reqs)
    r2t = torch.zeros(len(reqs) + 3, max_len + 4, dtype=torch.int32)
    rows = torch.randperm(len(reqs) + 3, generator=g)[: len(reqs)]
    scale = D ** -0.5
    hb = bias + 0.5 * torch.randn(H, generator=g)
    q_all, want, at = [], [], 0
    for b, (pre, ext) in enumerate(reqs):
        n = pre + ext
        q, k, v = torch.randn(n, H, D, generator=g), torch.randn(n, G, D, generator=g), torch.randn(n, G, E, generator=g)
        if standout is not None:
            # the query at `qi` points along one direction; key `kj` points the same way (strength > 0) or the opposite way
            # (< 0: weight ~ 0 although visible), and carries values that cannot be missed if it is wrongly seen or left out
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
        ref = out_scale * P.sigmoid_attention(q, k, v, scale, hb, P.window_mask(n, window or n + 1, keep)).reshape(n, H * E)
        want.append(ref[pre:])
        q_all.append(q[pre:].reshape(ext, H * D))
    q_cat = torch.cat(q_all).to(DEV)
    out = torch.empty(q_cat.shape[0], H * E, dtype=dtype, device=DEV)
    ext_lens = [e for _, e in reqs]
    starts = [sum(ext_lens[:i]) for i in range(len(reqs))]
    if decode:
        assert all(e == 1 for e in ext_lens)
        q_start = q_len = None
    else:
        q_start = torch.tensor(starts, dtype=torch.int32, device=DEV)
        q_len = torch.tensor(ext_lens, dtype=torch.int32, device=DEV)
    ops.window_attention_fwd(q_cat, out, kp.to(DEV), vp.to(DEV), r2t.to(DEV), rows.to(DEV),
                             torch.tensor([p + e for p, e in reqs], dtype=torch.int64, device=DEV), q_start, q_len,
                             max(ext_lens), scale, window, keep, hb.to(DEV), True, None, out_scale, form=form)
    return out.float().cpu(), torch.cat(want)


REQS = [(0, 1), (0, 70), (63, 2), (64, 65), (100, 1), (5, 130), (31, 3)]
FORMS = [(torch.float32, 1), (torch.bfloat16, 1), (torch.bfloat16, 2), (torch.float16, 2)]


def _sum_tol(dtype, n_keys):
    """Unnormalised weights: a row is a sum over up to n_keys keys, and its rounding error grows with it."""
    t = TOL[dtype]
    return dict(rtol=t["rtol"], atol=t["atol"] * max(1.0, n_keys ** 0.5 / 2))


@pytest.mark.parametrize("window,keep", [(0, 0), (1, 0), (1, 3), (5, 5), (32, 1), (33, 40), (64, 7), (1000, 2)])
@pytest.mark.parametrize("dtype,form", FORMS)
def test_window_attention_every_window(window, keep, dtype, form):
    got, want = _window_case(4, 2, 64, 32, window, keep, dtype, form, REQS, seed=window + keep, out_scale=1.25)
    torch.testing.assert_close(got, want, **_sum_tol(dtype, (window or 140) + keep))


@pytest.mark.parametrize("H,G,D,E", [(4, 4, 96, 64), (8, 2, 128, 128), (2, 1, 256, 256), (3, 1, 32, 16), (32, 1, 64, 32),
                                     (6, 3, 160, 80), (6, 2, 96, 160)])
@pytest.mark.parametrize("dtype,form", [(torch.bfloat16, 2), (torch.float32, 1)])
def test_window_attention_head_counts_and_sizes(H, G, D, E, dtype, form):
    for decode in (False, True):
        reqs = [(70, 1), (0, 1), (129, 1), (33, 1)] if decode else [(0, 40), (70, 30), (16, 1)]
        got, want = _window_case(H, G, D, E, 48, 6, dtype, form, reqs, seed=H + D, decode=decode)
        torch.testing.assert_close(got, want, **_sum_tol(dtype, 54))


@pytest.mark.parametrize("D,E", [(40, 24), (100, 7), (512, 8), (32, 400)])
def test_window_attention_sizes_only_the_row_form_takes(D, E):
    for dtype in (torch.bfloat16, torch.float32):
        got, want = _window_case(4, 2, D, E, 16, 3, dtype, 0, [(0, 35), (20, 1), (17, 9)], seed=D)
        torch.testing.assert_close(got, want, **_sum_tol(dtype, 19))


@pytest.mark.parametrize("dtype,form", [(torch.float32, 1), (torch.bfloat16, 1), (torch.bfloat16, 2)])
@pytest.mark.parametrize("decode", [False, True])
def test_window_and_kept_edges_stand_out(dtype, form, decode):
    """For the last query of every request: the key just OUTSIDE the window (position query - window) and the first key
    behind the kept ones (position keep) match the query perfectly and carry huge values -- unless they are visible through
    the other rule; the key just inside the window (query - window + 1) and the last kept key (keep - 1) match it too and
    carry their own.  A mask one position off, on either rule, moves the result by orders of magnitude."""
    window, keep = 24, 5

    def standout(pre, ext):
        qi = pre + ext - 1
        keys = {}
        for j, inside in ((qi - window, False), (qi - window + 1, True), (keep, False), (keep - 1, True)):
            if 0 <= j < qi:
                seen = (qi - j < window) or (j < keep)
                assert seen or not inside
                keys[j] = (j, 6.0, (3.0 if j % 2 else -3.0) if seen else 500.0)
        return [([qi], list(keys.values()))]

    lens = (4, 5, 6, 24, 25, 28, 29, 30, 31, 71, 100)
    reqs = [(p, 1) for p in lens] if decode else [(0, p + 1) for p in lens] + [(40, 9), (47, 2), (20, 77)]
    got, want = _window_case(2, 1, 32, 32, window, keep, dtype, form, reqs, seed=3, standout=standout, decode=decode, bias=-6.0)
    last = torch.tensor([e for _, e in reqs]).cumsum(0) - 1
    assert want[last].abs().max() < 20        # the unseen keys' values are nowhere in the truth of the rows built for them
    assert want[last].abs().max() > 2         # ... and the seen ones' are
    torch.testing.assert_close(got, want, **_sum_tol(dtype, window + keep))


@pytest.mark.parametrize("dtype,form", [(torch.float32, 1), (torch.bfloat16, 2)])
def test_one_far_key_among_hundreds(dtype, form):
    """A window of 700 positions over 900: the one key that matters lies 650 back; next to it, one position behind the
    window's edge, a decoy with huge values."""
    def standout(pre, ext):
        qi = pre + ext - 1
        return [([qi], [(qi - 650, 6.0, 4.0), (qi - 700, 6.0, 900.0)])]

    for decode in (False, True):
        reqs = [(899, 1), (760, 1)] if decode else [(500, 400), (0, 760)]
        got, want = _window_case(2, 2, 64, 32, 700, 0, dtype, form, reqs, seed=9, standout=standout, decode=decode, bias=-9.0)
        last = torch.tensor([e for _, e in reqs]).cumsum(0) - 1
        assert 3 < want[last].abs().max() < 8
        torch.testing.assert_close(got, want, **_sum_tol(dtype, 40))


# ----------------------------------------------------------------------------------------------- minGRU
def _gru_reference(z_lin, x_lin, g_lin, bz, bx, out_scale):
    S = P.min_gru_states(z_lin.float() + bz.float(), x_lin.float() + bx.float())
    return out_scale * S * torch.nn.functional.silu(g_lin.float()), S


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("R", [1, 48, 300])
def test_min_gru_portions_decode_and_slot_reuse(dtype, R):
    """Three sequences through state rows 3, 1 and 3 again: whole, in portions of every size (the chunked form for the long
    one), token by token; a row that another request leaves full of its state starts the next one from zero all the same."""
    from semi_pd_amd import ops
    g = torch.Generator().manual_seed(R)
    ld, z_off, x_off, g_off = 3 * R + 20, 11, 11 + R, 20 + 2 * R
    bz, bx = torch.randn(R, generator=g).to(dtype), torch.randn(R, generator=g).to(dtype)
    state = torch.full((5, R + 3), 99.0, device=DEV)          # rows wider than the layer: a column range of a wider pool
    view = state[:, 2: 2 + R]

    def run(rows, slot, seq_len, q_lens):
        """rows [n, ld] of ONE request whose last row sits at seq_len - 1, cut as q_lens says (None: one decode row)."""
        out = torch.empty(rows.shape[0], R, dtype=dtype, device=DEV)
        idx = torch.tensor([slot], dtype=torch.int64, device=DEV)
        if q_lens is None:
            ops.min_gru(rows.to(DEV), z_off, x_off, g_off, R, bz.to(DEV), bx.to(DEV), out, view, idx,
                        torch.tensor([seq_len], dtype=torch.int64, device=DEV), None, None, 1, out_scale=0.75)
        else:
            ops.min_gru(rows.to(DEV), z_off, x_off, g_off, R, bz.to(DEV), bx.to(DEV), out, view, idx,
                        torch.tensor([seq_len], dtype=torch.int64, device=DEV), torch.tensor([0], dtype=torch.int32, device=DEV),
                        torch.tensor([rows.shape[0]], dtype=torch.int32, device=DEV), rows.shape[0], out_scale=0.75)
        return out.float().cpu()

    for slot, n, cuts in ((3, 700, [300, 2, 1, 333, 64]), (1, 90, [90]), (3, 41, [2, 1, 1, 30, 7])):
        rows = torch.randn(n, ld, generator=g).to(dtype)
        want, S = _gru_reference(rows[:, z_off: z_off + R], rows[:, x_off: x_off + R], rows[:, g_off: g_off + R], bz, bx, 0.75)
        got, at = [], 0
        for c in cuts:
            got.append(run(rows[at: at + c], slot, at + c, None if (c == 1 and at > 0) else c))
            at += c
        assert at == n
        torch.testing.assert_close(torch.cat(got), want, **TOL[dtype])
        torch.testing.assert_close(view[slot].cpu(), S[-1], rtol=1e-4, atol=1e-5)
    assert (state[:, :2] == 99).all() and (state[:, 2 + R:] == 99).all() and (state[0] == 99).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_min_gru_batches_of_unequal_requests(dtype):
    """Five requests side by side -- a long portion, short ones, continued and new sequences -- against each alone."""
    from semi_pd_amd import ops
    g = torch.Generator().manual_seed(5)
    R = 72
    reqs = [(0, 300), (40, 1), (0, 2), (7, 65), (0, 1)]         # (tokens before this launch, tokens in it)
    state = torch.zeros(9, R, device=DEV)
    slots = [4, 2, 7, 1, 5]
    rows_all, want_all = [], []
    for (pre, ext), slot in zip(reqs, slots):
        rows = torch.randn(pre + ext, 3 * R, generator=g).to(dtype)
        z0 = torch.zeros(R)
        y, S = _gru_reference(rows[:, :R], rows[:, R: 2 * R], rows[:, 2 * R:], z0, z0, 1.0)
        state[slot] = S[pre - 1].to(DEV) if pre else torch.full((R,), -5.0, device=DEV)     # what a new request finds is junk
        rows_all.append(rows[pre:])
        want_all.append(y[pre:])
    ext = [e for _, e in reqs]
    out = torch.empty(sum(ext), R, dtype=dtype, device=DEV)
    ops.min_gru(torch.cat(rows_all).to(DEV), 0, R, 2 * R, R, None, None, out, state, torch.tensor(slots, dtype=torch.int64, device=DEV),
                torch.tensor([p + e for p, e in reqs], dtype=torch.int64, device=DEV),
                torch.tensor([sum(ext[:i]) for i in range(len(ext))], dtype=torch.int32, device=DEV),
                torch.tensor(ext, dtype=torch.int32, device=DEV), max(ext))
    torch.testing.assert_close(out.float().cpu(), torch.cat(want_all), **TOL[dtype])


# ----------------------------------------------------------------------------------------------- experts
@pytest.mark.parametrize("dtype,side_by_side", [(torch.float32, True), (torch.bfloat16, True), (torch.bfloat16, False)])
@pytest.mark.parametrize("X,K,W,F,T", [(4, 2, 64, 32, 9), (6, 6, 128, 128, 70), (1, 1, 32, 16, 3), (3, 2, 100, 28, 17), (3, 2, 104, 30, 17),
                                       (8, 3, 256, 64, 700)])
def test_ungated_experts(dtype, side_by_side, X, K, W, F, T, monkeypatch):
    from semi_pd_amd.layers.moe import UngatedMoE
    monkeypatch.setenv("SEMIPD_MOE_SIDE_BY_SIDE", "1" if side_by_side else "0")
    g = torch.Generator().manual_seed(X * W)
    w = {"router": (torch.randn(X, W, generator=g) * 4 / W ** 0.5).to(torch.bfloat16)}
    for e in range(X):
        w[f"e{e}.up"] = (torch.randn(F, W, generator=g) / W ** 0.5).to(torch.bfloat16)
        w[f"e{e}.down"] = (torch.randn(W, F, generator=g) / F ** 0.5).to(torch.bfloat16)
    with torch.device(DEV):
        m = UngatedMoE(X, K, W, F, "relu2", params_dtype=dtype)
    m.router.copy_(w["router"])
    m.w_up.copy_(torch.stack([w[f"e{e}.up"] for e in range(X)]))
    m.w_down.copy_(torch.stack([w[f"e{e}.down"] for e in range(X)]))
    m.post_load_weights()
    assert (m.w_down_cat is not None) == (side_by_side or W % 8 != 0)
    h = torch.randn(T, W, generator=g).to(dtype)
    got = m(h.to(DEV)).float().cpu()
    want = P.expert_mixture(h, w, "", {"router": {"experts": X, "top": K}})
    # (two experts whose scores tie to the last bit may swap places between the two sums: a row in two hundred may differ)
    t = TOL[dtype]
    bad = ((got - want).abs() > t["atol"] + t["rtol"] * want.abs()).any(-1).sum().item()
    assert bad <= T // 200, f"{bad} of {T} rows differ"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T", [1, 19, 64])
def test_squared_relu_in_the_first_expert_gemm_keeps_the_bits(dtype, T):
    """Decode-sized calls: the activation in the epilogue of the grouped streaming GEMM against GEMM + the separate kernel."""
    from semi_pd_amd import ops
    g = torch.Generator().manual_seed(T)
    X, K, W, F = 6, 2, 256, 128
    h = torch.randn(T, W, generator=g).to(dtype).to(DEV)
    w_up = (torch.randn(X, F, W, generator=g) / W ** 0.5).to(dtype).to(DEV)
    _, ids = ops.topk_softmax(torch.randn(T, X, generator=g).to(DEV), K, True)
    block_m = min(64, 16 * -(-T // 16))
    numel = T * K
    max_sorted = -(-(numel + X * (block_m - 1)) // block_m) * block_m
    sorted_ids = torch.empty(max_sorted, dtype=torch.int32, device=DEV)
    expert_ids = torch.empty(max_sorted // block_m, dtype=torch.int32, device=DEV)
    post = torch.empty(1, dtype=torch.int32, device=DEV)
    ops.moe_align_block_size(ids, X, block_m, sorted_ids, expert_ids, post, None, torch.empty(X + 1, dtype=torch.int32, device=DEV))
    plain, fused = (torch.zeros(numel, F, dtype=dtype, device=DEV) for _ in range(2))
    ops.moe_stream_gemm(h, w_up, plain, None, sorted_ids, expert_ids, post, numel, K, False, block_m)
    ops.bias_relu_square_(plain, None)
    ops.moe_stream_gemm(h, w_up, fused, None, sorted_ids, expert_ids, post, numel, K, False, block_m, fuse_relu_square=True)
    assert torch.equal(plain, fused) and plain.abs().max() > 0


# ----------------------------------------------------------------------------------------------- model level
def _left(heads, kv_heads, dim, vdim, size, keep, rot):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": 0.7 * dim ** -0.5,
            "mask": {"size": size, "keep_first": keep}, "rot": {"base": 3000.0, "dims": rot}}


def _layer(left, right, ls, rs, moe):
    mlp = None if moe is None else {"kind": "moe", "expert": {"ff": moe[2]}, "router": {"experts": moe[0], "top": moe[1]}}
    return {"type": "parallel", "mixer": {"left": left, "right": {"width": right}, "left_scale": ls, "right_scale": rs}, "mlp": mlp}


CONFIGS = {
    # layers of different geometry, one without experts, a partial rotation, top == experts; layers 1 .. 2 run three times
    "mixed": {"architecture": "Tigotar", "vocab": 200, "width": 64, "norm": {"eps": 1e-5}, "logit_scale": 0.5,
              "loop": {"start": 1, "stop": 3, "times": 3},
              "layers": [_layer(_left(4, 2, 32, 16, 24, 5, 32), 48, 1.1, 0.8, (4, 2, 32)),
                         _layer(_left(2, 2, 64, 32, 40, 0, 16), 80, 0.7, 1.3, None),
                         _layer(_left(4, 1, 32, 48, 9, 3, 32), 64, 1.0, 1.0, (6, 6, 48))]},
    # sizes of one; a window that sees the query alone plus one kept position; the whole model is the repeated span, once
    "minimal": {"architecture": "Tigotar", "vocab": 64, "width": 32, "norm": {"eps": 1e-6}, "logit_scale": 1.0,
                "loop": {"start": 0, "stop": 1, "times": 1},
                "layers": [_layer(_left(1, 1, 32, 32, 1, 1, 2), 16, 1.0, 1.0, (1, 1, 16))]},
    # sizes no vector path takes; more kept positions than the window is long; a window longer than any sequence; no loop key
    "awkward": {"architecture": "Tigotar", "vocab": 301, "width": 100, "norm": {"eps": 1e-5}, "logit_scale": 2.0,
                "layers": [_layer(_left(3, 1, 20, 12, 7, 9, 10), 36, 0.9, 1.2, (3, 2, 28)),
                           _layer(_left(2, 2, 24, 20, 1000, 2, 24), 52, 1.0, 0.5, None)]},
    # a span of two layers run twice, then a layer behind it; the kept positions reach past the window of the last layer
    "tail": {"architecture": "Tigotar", "vocab": 128, "width": 64, "norm": {"eps": 1e-6}, "logit_scale": 0.25,
             "loop": {"start": 0, "stop": 2, "times": 2},
             "layers": [_layer(_left(2, 1, 32, 32, 16, 2, 32), 32, 1.0, 1.0, (2, 1, 64)),
                        _layer(_left(4, 4, 16, 16, 5, 1, 8), 96, 1.2, 0.9, None),
                        _layer(_left(8, 2, 32, 16, 12, 20, 32), 64, 0.8, 1.1, (5, 3, 40))]},
}


def _write_checkpoint(path, cfg, seed):
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    w = P.random_weights(cfg, seed)
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
    mr = _build_runner(sa, 0, 0, InstanceRole.OTHER, 29651, max_total_tokens=max_tokens)
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
    path = str(tmp_path_factory.mktemp("tigotar_mixed"))
    cfg = CONFIGS["mixed"]
    w = _write_checkpoint(path, cfg, seed=11)
    # a pool far smaller than the tokens that pass through it: slots, rows and state rows come back and are used again
    sched = _scheduler(path, request.param, max_tokens=448)
    lens = {"a": 150, "b": 1, "c": 97, "d": 2, "e": 64, "f": 131}
    prompts = {n: _tokens(k, cfg["vocab"], seed=ord(n)) for n, k in lens.items()}
    truth = {n: P.forward(cfg, w, t) for n, t in prompts.items()}
    return request.param, sched, prompts, truth, (cfg, w)


def _pools_are_whole(sched):
    assert sched.token_to_kv_pool_allocator.available_size() == 448 and sched.req_to_token_pool.available_size() == 5
    assert sched.model_runner.state_pool.available_size() == 4 and not sched.live


def test_every_layer_run_matches_the_plain_model(mixed_model):
    dtype, sched, prompts, truth, (cfg, w) = mixed_model
    seen = {}
    sched.model_runner.model.layer_probe = lambda i, x: seen.__setitem__(i, x.detach().float().cpu().clone())
    try:
        _run_schedule(sched, {"e": prompts["e"]}, [[("e", 64)]])
    finally:
        sched.model_runner.model.layer_probe = None
    _, layers = P.forward(cfg, w, prompts["e"], return_layers=True)
    assert len(seen) == layers.shape[0] == 7          # one layer once, a span of two three times
    for i in range(7):
        tol = dict(rtol=1e-4, atol=2e-4) if dtype == "float32" else dict(rtol=0.1, atol=0.25)
        torch.testing.assert_close(seen[i], layers[i], **tol)


def test_whole_prompts_match_the_plain_model(mixed_model):
    dtype, sched, prompts, truth, _ = mixed_model
    got = _run_schedule(sched, prompts, [[(n, len(t))] for n, t in prompts.items()])
    for n in prompts:
        assert _rel_err(got[n], truth[n]) < LIMIT[dtype], n
    _pools_are_whole(sched)


def test_decoding_token_by_token_matches_the_prompt_pass(mixed_model):
    """Ten tokens as a prompt, then one token per step through the captured decode graphs: past the windows of every layer
    (9, 24, 40) and their kept positions, 140 steps long."""
    dtype, sched, prompts, truth, _ = mixed_model
    for n in ("a", "f", "d"):
        T = len(prompts[n])
        first = min(10, T - 1)
        got = _run_schedule(sched, {n: prompts[n]}, [[(n, first)]] + [[(n, 1)] for _ in range(T - first)])
        assert _rel_err(got[n], truth[n]) < LIMIT[dtype], n
    assert sched.stats["decode_steps"] > 0
    _pools_are_whole(sched)


def test_portions_of_every_size_down_to_two(mixed_model):
    dtype, sched, prompts, truth, _ = mixed_model
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
    that end while others go on, new ones taking their rows, slots and state rows."""
    dtype, sched, prompts, truth, _ = mixed_model
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
    _pools_are_whole(sched)


def test_logits_do_not_depend_on_the_cut_or_the_neighbours(mixed_model):
    """The same request alone and whole, and in a batch cut into portions: equal up to rounding (fp32: ~1e-6)."""
    dtype, sched, prompts, truth, _ = mixed_model
    alone = _run_schedule(sched, {"c": prompts["c"]}, [[("c", 97)]])["c"]
    mixed = _run_schedule(sched, {k: prompts[k] for k in "ce"}, [[("c", 40), ("e", 3)], [("c", 1), ("e", 60)], [("c", 56), ("e", 1)]])["c"]
    assert _rel_err(mixed, alone) < (2e-5 if dtype == "float32" else 5e-2)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,vocab", [("minimal", 64), ("awkward", 301), ("tail", 128)])
def test_other_sizes(name, vocab, dtype, tmp_path):
    """minimal: heads, groups, experts and windows of one, the whole model one repeated span that runs once.  awkward: sizes
    that no vector path takes (width 100, heads of 20 / 12, 28-wide experts, a vocabulary of 301), no repeated span at all.
    tail: the span is in front and a layer follows it."""
    cfg = CONFIGS[name]
    w = _write_checkpoint(str(tmp_path), cfg, seed=5)
    sched = _scheduler(str(tmp_path), dtype, max_tokens=192)
    prompts = {"x": _tokens(70, vocab, 3), "y": _tokens(23, vocab, 4), "z": _tokens(1, vocab, 5)}
    got = _run_schedule(sched, prompts, [[("x", 30), ("y", 2), ("z", 1)], [("x", 1), ("y", 1)], [("x", 1), ("y", 1)],
                                         [("x", 37), ("y", 19)], [("x", 1)]])
    for n, t in prompts.items():
        assert _rel_err(got[n], P.forward(cfg, w, t)) < LIMIT[dtype], n


def test_long_prompt_takes_the_chunked_recurrence_and_long_decoding(tmp_path):
    """600 tokens in one portion (the chunked form of the recurrence, many tiles of the prompt attention), then 200 decode
    steps, in fp32 against the plain model."""
    cfg = CONFIGS["mixed"]
    w = _write_checkpoint(str(tmp_path), cfg, seed=31)
    sched = _scheduler(str(tmp_path), "float32", max_tokens=832, max_requests=2)
    t = _tokens(800, cfg["vocab"], 77)
    got = _run_schedule(sched, {"p": t}, [[("p", 600)]] + [[("p", 1)]] * 200)
    assert _rel_err(got["p"], P.forward(cfg, w, t)) < LIMIT["float32"]


def _check_generation(cfg, w, prompts, outs, steps):
    exact = 0
    for p, o in zip(prompts, outs):
        assert len(o) == steps
        logits = P.forward(cfg, w, p + o)
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
    """The same through a prefill and a decode process on one GPU: the pool regions of every layer run, the slab of recurrent
    state rows and every parameter reach the prefill process through IPC handles; the decode process hands out the state
    rows, prompts are cut into 48-token portions in the prefill process (the state row carries the recurrence from portion
    to portion) and decoded in the other."""
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
