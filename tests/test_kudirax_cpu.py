"""Host-side pieces of the Kudirax integration: configuration reader, checkpoint name mapping, KV-pool regions, and the plain
model's own invariants (tests/test_gpu_kudirax.py compares the engine with it)."""
import json
import os

import pytest
import torch

from oracle import kudirax as K


def _mixer(heads, kv_heads, dim, vdim, chunk, v_mix):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": chunk}, "softcap": 12.0,
            "scale": 0.2, "v_mix": v_mix}


CFG = {"architecture": "Kudirax", "vocab": 100, "width": 48, "norm": {"eps": 1e-5}, "layers": [
    {"type": "attention", "mixer": _mixer(3, 1, 16, 8, 4, False), "mlp": None},
    {"type": "attention", "mixer": _mixer(2, 2, 24, 8, 9, True), "mlp": {"kind": "dense", "ff": 80}},
    {"type": "attention", "mixer": _mixer(4, 2, 8, 8, 6, True), "mlp": {"kind": "dense", "ff": 32}}]}


def test_config_reader_takes_every_size_from_the_file():
    from semi_pd_amd.model_loader import config_from_hf_dict
    c = config_from_hf_dict(CFG)
    assert type(c).__name__ == "KudiraxConfig" and c.architectures == ("Kudirax",)
    assert (c.vocab_size, c.hidden_size, c.norm_eps, c.num_hidden_layers) == (100, 48, 1e-5, 3)
    m = c.layers[1].mixer
    assert (m.heads, m.kv_heads, m.dim, m.vdim, m.chunk, m.softcap, m.scale, m.v_mix) == (2, 2, 24, 8, 9, 12.0, 0.2, True)
    assert [l.ff for l in c.layers] == [0, 80, 32]
    bad = json.loads(json.dumps(CFG))
    bad["layers"][0]["type"] = "recurrent"
    with pytest.raises(ValueError):
        config_from_hf_dict(bad)
    bad = json.loads(json.dumps(CFG))
    bad["layers"][1]["mlp"]["kind"] = "experts"
    with pytest.raises(ValueError):
        config_from_hf_dict(bad)
    bad = json.loads(json.dumps(CFG))
    bad["layers"][0]["mixer"]["kv_heads"] = 2
    with pytest.raises(ValueError):
        config_from_hf_dict(bad)


def test_checkpoint_names_reach_every_parameter_and_merge_the_projections():
    from semi_pd_amd.model_executor.model_runner import build_model
    from semi_pd_amd.model_loader import config_from_hf_dict, load_weights
    c = config_from_hf_dict(CFG)
    w = K.random_weights(CFG, seed=2)
    with torch.device("cpu"):
        model = build_model(c, torch.float32)
    loaded = load_weights(model, c, w.items())
    params = dict(model.named_parameters())
    assert set(loaded) == set(params)
    l1 = "layers.1.mix."
    merged = torch.cat([w["l1.mix.q"], w["l1.mix.k"], w["l1.mix.v"], w["l1.mix.g"]]).float()
    assert torch.equal(params[l1 + "qkvg_proj.weight"], merged)
    assert torch.equal(params[l1 + "sink"], w["l1.mix.sink"].float()) and params[l1 + "sink"].dtype == torch.float32
    assert torch.equal(params["layers.2.mlp.down.bias"], w["l2.mlp.down.b"].float())
    assert torch.equal(params["final_norm.bias"], w["final.norm.b"].float())
    # the vocabulary is padded to the embedding's granule with zero rows; the real rows are the checkpoint's
    assert params["embed.weight"].shape[0] == 128 and torch.equal(params["embed.weight"][:100], w["embed"].float())
    assert params["embed.weight"][100:].abs().sum() == 0
    assert "layers.0.norm2.weight" not in params          # no feed-forward, no second norm
    del w["l2.mix.g"]
    with pytest.raises(RuntimeError):
        load_weights(model, c, w.items())


def test_pool_regions_per_layer():
    from semi_pd_amd.mem_cache.memory_pool import MHATokenToKVPool
    pool = MHATokenToKVPool(10, 1, torch.bfloat16, [1, 2, 2], [16, 24, 8], 3, "cpu", v_head_dim=[8, 8, 8])
    assert not pool.uniform
    assert [tuple(b.shape) for b in pool.k_buffer] == [(11, 1, 16), (11, 2, 24), (11, 2, 8)]
    assert [tuple(b.shape) for b in pool.v_buffer] == [(11, 1, 8), (11, 2, 8), (11, 2, 8)]
    spans = sorted((b.data_ptr(), b.data_ptr() + b.numel() * 2) for b in pool.k_buffer + pool.v_buffer)
    base = pool.slab.data_ptr()
    assert all(a[1] <= b[0] for a, b in zip(spans, spans[1:])) and all((a[0] - base) % 256 == 0 for a in spans)
    assert spans[0][0] == base and spans[-1][1] <= base + pool.slab.numel()
    k, v = pool.get_kv_size_bytes()
    assert k == 11 * 2 * (16 + 48 + 16) and v == 11 * 2 * (8 + 16 + 16)
    same = MHATokenToKVPool(10, 1, torch.bfloat16, 2, 16, 3, "cpu")
    assert same.uniform and tuple(same.slab.shape) == (3, 2, 11, 2, 16)       # the layout every other model keeps


def test_plain_model_prefix_property_and_block_locality():
    """The plain model is causal (a prefix's logits do not change when tokens follow), and a token before the block of the
    LAST layer-0 query cannot reach it through layer 0 alone -- checked on the mask function itself."""
    w = K.random_weights(CFG, seed=3)
    toks = torch.randint(0, 100, (30,), generator=torch.Generator().manual_seed(1)).tolist()
    full = K.forward(CFG, w, toks)
    torch.testing.assert_close(K.forward(CFG, w, toks[:17]), full[:17], rtol=1e-5, atol=1e-5)
    m = K.visible(10, 4)
    assert m[5].tolist() == [False] * 4 + [True, True] + [False] * 4
    assert m[8].tolist() == [False] * 8 + [True, False] and K.visible(3, None).tolist() == torch.ones(3, 3).tril().bool().tolist()
    s = torch.zeros(1, 2, 2)
    p = K.sink_softmax(s, K.visible(2, None), torch.tensor([0.0]))
    torch.testing.assert_close(p[0], torch.tensor([[0.5, 0.0], [1 / 3, 1 / 3]]))


def test_command_line_reads_the_folder_and_float32_is_for_models_that_have_it(tmp_path):
    import argparse
    from semi_pd_amd import server_args as SA
    with open(tmp_path / "config.json", "w") as f:
        json.dump(CFG, f)
    ap = argparse.ArgumentParser()
    SA.add_cli_args(ap)
    sa = SA.from_cli_args(ap.parse_args(["--model-path", str(tmp_path), "--dtype", "float32", "--skip-tokenizer-init"]))
    assert type(sa.model_config).__name__ == "KudiraxConfig" and sa.torch_dtype == torch.float32 and sa.load_format == "auto"
    from semi_pd_amd.models.llama import LlamaConfig
    with pytest.raises(ValueError):
        SA.ServerArgs(model_config=LlamaConfig(), dtype="float32")
    assert SA.ServerArgs(model_config=LlamaConfig(), dtype="bfloat16").torch_dtype == torch.bfloat16


def test_replay_runner_refuses_without_a_device():
    from semi_pd_amd.entrypoints import trace_replay
    if torch.cuda.is_available():
        pytest.skip("a device is present")
    assert trace_replay.main(["--model", "/nonexistent", "--dtype", "float32", "--out", "/tmp/x", "--max-tokens", "64"]) == 2
