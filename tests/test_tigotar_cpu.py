"""Host-side pieces of the Tigotar integration: configuration reader and the order of layer runs, checkpoint name mapping,
the state pool's bookkeeping, state rows through the batch preparation, and the plain model's own invariants
(tests/test_gpu_tigotar.py compares the engine with it)."""
import json

import pytest
import torch

from oracle import tigotar as P


def _left(heads, kv_heads, dim, vdim, size, keep, rot):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": 0.25,
            "mask": {"size": size, "keep_first": keep}, "rot": {"base": 3000.0, "dims": rot}}


def _layer(left, right, moe):
    mlp = None if moe is None else {"kind": "moe", "expert": {"ff": moe[2]}, "router": {"experts": moe[0], "top": moe[1]}}
    return {"type": "parallel", "mixer": {"left": left, "right": {"width": right}, "left_scale": 1.5, "right_scale": 0.5}, "mlp": mlp}


CFG = {"architecture": "Tigotar", "vocab": 90, "width": 48, "norm": {"eps": 1e-5}, "logit_scale": 0.5,
       "loop": {"start": 1, "stop": 3, "times": 2},
       "layers": [_layer(_left(3, 1, 16, 8, 6, 2, 8), 24, (3, 2, 20)), _layer(_left(2, 2, 24, 8, 9, 0, 24), 40, None),
                  _layer(_left(4, 2, 8, 16, 4, 4, 8), 16, (5, 5, 12)), _layer(_left(2, 1, 16, 16, 50, 1, 16), 32, (2, 1, 8))]}


def test_config_reader_takes_every_size_from_the_file():
    from semi_pd_amd.model_loader import config_from_hf_dict
    c = config_from_hf_dict(CFG)
    assert type(c).__name__ == "TigotarConfig" and c.architectures == ("Tigotar",)
    assert (c.vocab_size, c.hidden_size, c.norm_eps, c.logit_scale, c.num_hidden_layers) == (90, 48, 1e-5, 0.5, 4)
    assert (c.loop_start, c.loop_stop, c.loop_times) == (1, 3, 2)
    m = c.layers[2].mixer
    a = m.left
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.scale, a.window, a.keep_first, a.rot_dims, a.rot_base) == \
        (4, 2, 8, 16, 0.25, 4, 4, 8, 3000.0)
    assert (m.right_width, m.left_scale, m.right_scale) == (16, 1.5, 0.5)
    assert [(l.experts, l.top, l.ff) for l in c.layers] == [(3, 2, 20), (0, 0, 0), (5, 5, 12), (2, 1, 8)]
    for path, value in ((("layers", 0, "type"), "attention"), (("layers", 2, "mlp", "kind"), "dense"),
                        (("layers", 0, "mixer", "left", "kv_heads"), 2), (("layers", 0, "mixer", "left", "rot", "dims"), 7),
                        (("layers", 3, "mlp", "router", "top"), 3), (("loop", "stop"), 5), (("loop", "times"), 0),
                        (("layers", 1, "mixer", "left", "mask", "chunk"), 4)):
        bad = json.loads(json.dumps(CFG))
        node = bad
        for k in path[:-1]:
            node = node[k]
        node[path[-1]] = value
        with pytest.raises(ValueError):
            config_from_hf_dict(bad)


def test_layer_runs_follow_the_repeated_span():
    from semi_pd_amd.model_loader import config_from_hf_dict
    runs = config_from_hf_dict(CFG).runs()
    assert [(r.layer, r.loop_pass, r.enters_pass) for r in runs] == \
        [(0, -1, False), (1, 0, True), (2, 0, False), (1, 1, True), (2, 1, False), (3, -1, False)]
    assert [r.run for r in runs] == list(range(6))
    assert [(i, t, f) for i, t, f in P.layer_runs(CFG)] == [(r.layer, r.loop_pass, r.enters_pass) for r in runs]
    for loop, want in (({"start": 0, "stop": 4, "times": 1}, [0, 1, 2, 3]), ({"start": 3, "stop": 4, "times": 3}, [0, 1, 2, 3, 3, 3]),
                       ({"start": 2, "stop": 2, "times": 4}, [0, 1, 2, 3]), (None, [0, 1, 2, 3])):
        cfg = json.loads(json.dumps(CFG))
        if loop is None:
            del cfg["loop"]
        else:
            cfg["loop"] = loop
        c = config_from_hf_dict(cfg)
        assert [r.layer for r in c.runs()] == want == [i for i, _, _ in P.layer_runs(cfg)]
        assert sum(r.enters_pass for r in c.runs()) == (loop["times"] if loop and loop["stop"] > loop["start"] else 0)


def test_checkpoint_names_reach_every_parameter_and_merge_the_projections():
    from semi_pd_amd.model_executor.model_runner import build_model
    from semi_pd_amd.model_loader import config_from_hf_dict, load_weights
    c = config_from_hf_dict(CFG)
    w = P.random_weights(CFG, seed=2)
    with torch.device("cpu"):
        model = build_model(c, torch.float32)
    loaded = load_weights(model, c, w.items())
    params = dict(model.named_parameters())
    assert set(loaded) == set(params)
    pre = "layers.2.mix."
    merged = torch.cat([w["l2.mix.left." + n] for n in "qkv"] + [w["l2.mix.right." + n] for n in "zxg"]).float()
    assert torch.equal(params[pre + "in_proj.weight"], merged)
    assert torch.equal(params[pre + "out_proj.weight"], torch.cat([w["l2.mix.left.o"], w["l2.mix.right.o"]], 1).float())
    assert torch.equal(params[pre + "bias_k"], w["l2.mix.left.k.b"].float())
    assert torch.equal(params[pre + "bias_x"], w["l2.mix.right.x.b"].float())
    assert torch.equal(params[pre + "head_bias"], w["l2.mix.left.pb"].float()) and params[pre + "head_bias"].dtype == torch.float32
    assert torch.equal(params["layers.2.mlp.w_up"], torch.stack([w[f"l2.mlp.e{e}.up"] for e in range(5)]).float())
    assert torch.equal(params["layers.2.mlp.w_down"][3], w["l2.mlp.e3.down"].float())
    assert torch.equal(params["layers.0.mlp.router"], w["l0.mlp.router"].float())
    assert torch.equal(params["layers.3.norm2b.alpha"], w["l3.norm2b.alpha"].float())
    assert torch.equal(params["embed_norm.bias"], w["embed.norm.b"].float())
    assert torch.equal(params["loop_step"], w["loop.step"].float()) and params["loop_in.weight"].shape == (48, 96)
    assert not any(n.startswith("layers.1.norm2") or n.startswith("layers.1.mlp") for n in params)   # no experts, no second pair
    # one KV-pool region and one range of state columns per layer RUN, not per layer
    geo = model.kv_geometry
    assert geo["num_kv_heads"] == [1, 2, 2, 2, 2, 1] and geo["v_head_dim"] == [8, 8, 16, 8, 16, 16] and geo["num_layers"] == 6
    assert model.state_geometry == [24, 40, 16, 40, 16, 32]
    with pytest.raises(KeyError):
        load_weights(model, c, list(w.items()) + [("l1.mix.left.gate", torch.zeros(1))])
    short = dict(w)
    del short["l2.mlp.e4.up"]
    with pytest.raises(RuntimeError):
        load_weights(model, c, short.items())


def test_state_pool_rows_and_columns():
    from semi_pd_amd.mem_cache.memory_pool import RecurrentStatePool
    pool = RecurrentStatePool(3, [24, 40, 6], "cpu")
    assert pool.slab.shape == (4, 24 + 40 + 8) and pool.slab.dtype == torch.float32
    bufs = [pool.get_state_buffer(i) for i in range(3)]
    assert [tuple(b.shape) for b in bufs] == [(4, 24), (4, 40), (4, 6)]
    bufs[1][2].fill_(7.0)
    assert pool.slab[2, 24:64].eq(7).all() and pool.slab.sum() == 7 * 40          # a layer's columns, one request's row
    a, b, c = pool.alloc(), pool.alloc(), pool.alloc()
    assert sorted((a, b, c)) == [1, 2, 3] and pool.alloc() is None and pool.available_size() == 0     # row 0 is the dummy row
    pool.free(b)
    with pytest.raises(ValueError):
        pool.free(b)
    with pytest.raises(ValueError):
        pool.free(0)
    assert pool.alloc() == b


def test_state_rows_follow_requests_through_batches():
    """A request takes a state row with its first portion, keeps it while its row of the request table changes hands between
    portions, and gives it back with everything else; a batch carries the rows in the order of its requests."""
    from semi_pd_amd.managers.io_struct import SamplingParams
    from semi_pd_amd.managers.schedule_batch import ChunkCache, Req, ScheduleBatch
    from semi_pd_amd.mem_cache.memory_pool import RecurrentStatePool, ReqToTokenPool, TokenToKVPoolAllocator
    r2t = ReqToTokenPool(3, 32, "cpu")
    alloc = TokenToKVPoolAllocator(64, torch.float32, "cpu", None)
    states = RecurrentStatePool(2, [8], "cpu")
    cache = ChunkCache(r2t, alloc, states)
    sp = SamplingParams(max_new_tokens=4, ignore_eos=True)
    a, b = Req("a", list(range(10)), sp), Req("b", list(range(5)), sp)
    for r, n in ((a, 6), (b, 5)):
        r.fill_ids, r.extend_input_len = r.origin_input_ids[:n], n
    batch = ScheduleBatch.init_new([a, b], r2t, alloc, cache, "cpu")
    batch.prepare_for_extend()
    assert batch.state_indices.tolist() == [a.state_slot, b.state_slot] and {a.state_slot, b.state_slot} == {1, 2}
    assert batch.get_model_worker_batch().state_indices is batch.state_indices
    # between two portions the request's table row goes back; the state row stays
    cache.cache_unfinished_req(a)
    r2t.free(a.req_pool_idx)
    kept = a.state_slot
    a.fill_ids, a.extend_input_len = a.origin_input_ids, 4
    nxt = ScheduleBatch.init_new([a], r2t, alloc, cache, "cpu")
    nxt.prepare_for_extend()
    assert a.state_slot == kept and nxt.state_indices.tolist() == [kept] and states.available_size() == 0
    # a third request finds no state row
    c = Req("c", [1, 2], sp)
    c.fill_ids, c.extend_input_len = [1, 2], 2
    with pytest.raises(RuntimeError, match="state"):
        ScheduleBatch.init_new([c], r2t, alloc, cache, "cpu").alloc_state_slots()
    cache.release_req(b)
    assert b.state_slot is None and states.available_size() == 1 and alloc.available_size() == 64 - 10
    # a request that ends while a step beyond its end is in flight (the overlapped decode loop) keeps its state row until
    # that step's slot is given back: the step still writes the row
    b2 = Req("b2", [1, 2, 3], sp)
    b2.fill_ids, b2.extend_input_len = [1, 2, 3], 3
    ScheduleBatch.init_new([b2], r2t, alloc, cache, "cpu").prepare_for_extend()
    b2.output_ids = [7]
    b2.kv_slots.append(int(alloc.alloc(1)[0]))          # the slot of the step launched beyond the end
    row = b2.state_slot
    cache.cache_finished_req(b2)
    assert b2.state_slot == row and len(b2.kv_slots) == 1
    alloc.free(b2.kv_slots)
    b2.kv_slots = []
    cache.release_state(b2)
    assert b2.state_slot is None and states.available_size() == 1
    b3 = Req("b3", [4, 5], sp)
    b3.fill_ids, b3.extend_input_len = [4, 5], 2
    ScheduleBatch.init_new([b3], r2t, alloc, cache, "cpu").prepare_for_extend()
    b3.output_ids = [9]
    cache.cache_finished_req(b3)                          # nothing in flight: the row goes back at once
    assert b3.state_slot is None and states.available_size() == 1
    # rows that another instance allocated travel with the batch and are never this side's to release
    guest = Req("g", [1, 2], sp)
    guest.fill_ids, guest.extend_input_len = [1, 2], 2
    gb = ScheduleBatch.init_new([guest], r2t, alloc, ChunkCache(r2t, alloc), "cpu")
    gb.prepare_for_extend(pre_allocated_req_pool_indices=[2], pre_allocated_slots=[[40, 41]], pre_allocated_state_slots=[2])
    assert gb.state_indices.tolist() == [2] and guest.state_slot is None
    # a request that has lost its state cannot continue from cached tokens
    a.state_slot = None
    with pytest.raises(RuntimeError, match="given up"):
        ScheduleBatch.init_new([a], r2t, alloc, cache, "cpu").alloc_state_slots()
    # models without recurrent layers: no pool, no rows
    plain = ScheduleBatch.init_new([c], r2t, alloc, ChunkCache(r2t, alloc), "cpu")
    plain.alloc_state_slots()
    assert plain.state_indices is None


def test_plain_model_invariants():
    """The oracle's own consistency: a prefix of a sequence gives the prefix of its logits (nothing looks ahead), the loop
    changes the result, the kept positions matter beyond the window, the recurrence carries beyond it too."""
    w = P.random_weights(CFG, seed=4)
    g = torch.Generator().manual_seed(0)
    toks = torch.randint(0, 90, (40,), generator=g).tolist()
    full, layers = P.forward(CFG, w, toks, return_layers=True)
    assert layers.shape == (6, 40, 48) and full.shape == (40, 90)
    torch.testing.assert_close(P.forward(CFG, w, toks[:17]), full[:17], rtol=1e-5, atol=1e-5)
    once = json.loads(json.dumps(CFG))
    once["loop"]["times"] = 1
    assert (P.forward(once, {**w, "loop.step": w["loop.step"][:1]}, toks) - full).abs().max() > 1e-3
    # masks: the window's two edges and the kept positions
    m = P.window_mask(12, 4, 2)
    assert m[9].nonzero().flatten().tolist() == [0, 1, 6, 7, 8, 9] and m[3].nonzero().flatten().tolist() == [0, 1, 2, 3]
    assert P.window_mask(5, 1, 0).nonzero().tolist() == [[i, i] for i in range(5)]
    # the pair rotation is a rotation, and leaves the tail of a head alone
    x = torch.randn(7, 2, 10, generator=g)
    y = P.rotate_pairs(x, 100.0, 6)
    torch.testing.assert_close(y[..., :6].norm(dim=-1), x[..., :6].norm(dim=-1), rtol=1e-5, atol=1e-5)
    assert torch.equal(y[..., 6:], x[..., 6:]) and torch.equal(y[0], x[0])
    # the recurrence: a gate that is shut keeps the state, one that is open replaces it with the candidate
    z = torch.tensor([[30.0], [-30.0], [-30.0], [30.0]])
    u = torch.tensor([[1.0], [5.0], [5.0], [-2.0]])
    torch.testing.assert_close(P.min_gru_states(z, u).flatten(), torch.tensor([1.5, 1.5, 1.5, torch.sigmoid(torch.tensor(-2.0)).item()]),
                               rtol=1e-5, atol=1e-5)
    # experts: top == experts is the plain softmax mixture
    h = torch.randn(5, 48, generator=g)
    mlp = CFG["layers"][2]["mlp"]
    s = torch.softmax(h @ w["l2.mlp.router"].float().T, -1)
    every = sum(s[:, e: e + 1] * (torch.relu(h @ w[f"l2.mlp.e{e}.up"].float().T) ** 2 @ w[f"l2.mlp.e{e}.down"].float().T) for e in range(5))
    torch.testing.assert_close(P.expert_mixture(h, w, "l2.mlp.", mlp), every, rtol=1e-4, atol=1e-5)


def test_command_line_of_a_model_folder(tmp_path):
    """A Tigotar folder on the command line: the class comes from config.json; float32 is accepted (every kernel of the path
    takes it); the trace runner wants a device."""
    import argparse
    from semi_pd_amd.entrypoints import trace_replay
    from semi_pd_amd.server_args import ServerArgs, add_cli_args, from_cli_args
    with open(tmp_path / "config.json", "w") as f:
        json.dump(CFG, f)
    ap = argparse.ArgumentParser()
    add_cli_args(ap)
    sa = from_cli_args(ap.parse_args(["--model-path", str(tmp_path), "--dtype", "float32", "--skip-tokenizer-init"]))
    assert type(sa.model_config).__name__ == "TigotarConfig" and sa.torch_dtype == torch.float32 and not sa.enable_semi_pd
    assert ServerArgs(model_path=str(tmp_path), enable_semi_pd=True, skip_tokenizer_init=True).enable_semi_pd
    if not torch.cuda.is_available():
        assert trace_replay.main(["--model", str(tmp_path), "--dtype", "bfloat16", "--out", str(tmp_path / "o"),
                                  "--max-tokens", "64"]) == 2
