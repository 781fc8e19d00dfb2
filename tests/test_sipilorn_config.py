"""The Sipilorn configuration: what its config.json turns into, what is refused, the run order of
its looped layers, and what its caches and states ask of the cache manager (all on the CPU)."""
import copy
import json
import os

import pytest
import torch

import plain_sipilorn as plain
from sipilorn_models import SIPILORN_CONFIGS, SP_A, SP_B, SP_C, SP_D, make_sipilorn_dir
from tffinfer_amd.config.base import ConfigError, LayerCall
from tffinfer_amd.models import build_model_skeleton, config_from_dict, load_config
from tffinfer_amd.parts import (GatedDeltaMixer, GatedGQAttention, KVCacheSpec, MixerPair, NoFeedForward,
                                ParallelBlock, RMSNorm, SwiGLU, TableExperts)
from tffinfer_amd.weights.loader import WeightError, check_weights
from tffinfer_amd.weights.safetensors_io import load_model_dir


def test_every_size_and_constant_comes_from_the_file():
    cfg = config_from_dict(copy.deepcopy(SP_A))
    model = build_model_skeleton(cfg)
    assert [type(b) for b in model.blocks] == [ParallelBlock] * 3
    assert [type(b.mixer) for b in model.blocks] == [MixerPair, GatedDeltaMixer, GatedDeltaMixer]
    assert [type(b.feed_forward) for b in model.blocks] == [SwiGLU, TableExperts, NoFeedForward]
    pair = model.blocks[0].mixer
    assert isinstance(pair.left, GatedGQAttention) and isinstance(pair.right, GatedDeltaMixer)
    assert (pair.left_scale, pair.right_scale) == (0.7, 1.3)
    a = pair.left
    assert (a.num_heads, a.num_kv_heads, a.head_dim, a.value_dim, a.scale, a.window, a.qk_norm_eps) == (4, 2, 16, 24, 0.3, 13, 1e-6)
    assert (a.position.rotary_dim, a.position.theta, a.position.pairing) == (8, 10000.0, "half")
    assert a.has_gate and a.external_output and pair.right.external_output
    spec = pair.cache_spec()
    assert isinstance(spec, KVCacheSpec) and (spec.num_kv_heads, spec.window, spec.keep_first) == (2, 13, 0)
    assert spec.head_dim >= 24        # keys of 16 and values of 24 share pages of one head size
    r = pair.right
    assert (r.num_heads, r.num_kv_heads, r.head_dim, r.value_dim, r.conv_taps, r.norm_eps) == (2, 1, 16, 8, 3, 1e-6)
    assert pair.state_spec().shape == (2 * 8 * 16 + 2 * (2 * 16 + 2 * 8),) and pair.state_spec().dtype == torch.float32
    d = model.blocks[2].mixer
    assert d.cache_spec() is None and d.state_spec().shape == (3 * 40 * 8 + 1 * (2 * 3 * 8 + 3 * 40),)
    assert not d.external_output
    ff = model.blocks[1].feed_forward
    assert (ff.num_experts, ff.top, ff.intermediate_size, ff.vocab_size) == (5, 2, 24, 300)
    assert model.blocks[0].feed_forward.intermediate_size == 72
    n = model.final_norm
    assert isinstance(n, RMSNorm) and (n.eps, n.size) == (1e-6, 64)
    assert isinstance(model.embedding.norm, RMSNorm) and model.embedding.norm.eps == 1e-6
    assert model.head.softcap == 20.0 and model.stream_offsets.rows == 3
    # another file: other constants, no loop, no cap, an attention without a window or a rotation
    b = build_model_skeleton(config_from_dict(copy.deepcopy(SP_B)))
    assert b.stream_offsets is None and b.head.softcap == 0.0 and b.final_norm.eps == 1e-5
    assert b.blocks[1].mixer.left.window == 8 and b.blocks[1].mixer.left.position.rotary_dim == 64
    assert b.blocks[2].mixer.conv_taps == 1 and b.blocks[2].mixer.state_spec().shape == (2 * 24 * 100,)
    c = build_model_skeleton(config_from_dict(copy.deepcopy(SP_C)))
    assert c.blocks[0].mixer.left.window == 0 and c.blocks[0].mixer.left.position is None
    assert c.blocks[0].mixer.cache_spec().window == 0
    # kv heads default to the heads, values to the keys' size
    m = copy.deepcopy(SP_C)
    del m["layers"][0]["mixer"]["left"]["kv_heads"], m["layers"][0]["mixer"]["left"]["vdim"]
    left = build_model_skeleton(config_from_dict(m)).blocks[0].mixer.left
    assert (left.num_kv_heads, left.value_dim) == (6, 32)


def test_the_run_order_of_looped_layers():
    """The span runs ``times`` times in a row, every run with a cache and state of its own; the pass's
    vector is added before the span's first layer, once a pass."""
    a = config_from_dict(copy.deepcopy(SP_A))
    assert a.layer_schedule() == [LayerCall(0, 0), LayerCall(1, 1, True, 0), LayerCall(2, 2), LayerCall(1, 3, True, 1),
                                  LayerCall(2, 4), LayerCall(1, 5, True, 2), LayerCall(2, 6)]
    assert config_from_dict(copy.deepcopy(SP_B)).layer_schedule() == [LayerCall(i, i) for i in range(3)]
    assert config_from_dict(copy.deepcopy(SP_C)).layer_schedule() == [
        LayerCall(0, 0, True, 0), LayerCall(1, 1), LayerCall(0, 2, True, 1), LayerCall(1, 3)]
    assert config_from_dict(copy.deepcopy(SP_D)).layer_schedule() == [
        LayerCall(0, 0, True, 0), LayerCall(0, 1, True, 1), LayerCall(1, 2)]
    for cfg in (SP_A, SP_B, SP_C, SP_D):        # the same order as the plain implementation's
        got = [(c.layer, c.offset if c.offset >= 0 else None) for c in config_from_dict(copy.deepcopy(cfg)).layer_schedule()]
        want = plain.run_order(cfg)
        loop = cfg.get("loop")
        want = [(i, t if (t is not None and i == loop["start"]) else None) for i, t in want]
        assert got == want
    # a loop of one pass still adds its vector; an empty span is no loop
    one = copy.deepcopy(SP_A)
    one["loop"] = {"start": 0, "stop": 2, "times": 1}
    assert [c.offset for c in config_from_dict(one).layer_schedule()] == [0, -1, -1]
    none = copy.deepcopy(SP_A)
    none["loop"] = {"start": 1, "stop": 1, "times": 4}
    assert config_from_dict(none).stream_offset_rows() == 0 and len(config_from_dict(none).layer_schedule()) == 3


def test_every_layer_call_gets_a_cache_and_a_state_of_its_own():
    from tffinfer_amd.cache.manager import CacheManager
    model = build_model_skeleton(config_from_dict(copy.deepcopy(SP_C)))
    needs = model.call_requirements()
    cache = CacheManager(needs, page_size=32, num_pages=24, max_seqs=2)
    # two pairs, each run twice: four key/value caches and four states
    assert sum(1 for n in needs if n[2] is not None) == 4 and sum(1 for n in needs if n[3] is not None) == 4
    cache.add_request("a")
    cache.reserve("a", 100)
    cache.commit("a", 100)
    cache.check()
    cache.release("a")
    assert all(g.pool.num_used == 0 for g in cache.groups)


def test_tensor_names_follow_the_files():
    names = build_model_skeleton(config_from_dict(copy.deepcopy(SP_A))).expected_tensors()
    for n in ("embed", "embed.norm", "loop.step", "final.norm", "head", "l0.norm1", "l0.norm2",
              "l0.mix.left.q", "l0.mix.left.q.norm", "l0.mix.left.k", "l0.mix.left.k.norm", "l0.mix.left.v", "l0.mix.left.g",
              "l0.mix.left.o", "l0.mix.right.q", "l0.mix.right.q.conv", "l0.mix.right.k.conv", "l0.mix.right.v.conv",
              "l0.mix.right.b", "l0.mix.right.a", "l0.mix.right.A_log", "l0.mix.right.dt_bias", "l0.mix.right.norm",
              "l0.mix.right.g", "l0.mix.right.o", "l0.mlp.gate", "l0.mlp.up", "l0.mlp.down",
              "l1.mix.q", "l1.mix.v.conv", "l1.mix.A_log", "l1.mix.o", "l1.mlp.table", "l1.mlp.e0.up", "l1.mlp.e4.down",
              "l2.norm1", "l2.mix.q"):
        assert n in names, n
    assert not any(n.endswith(("router", "e0.gate", "mix.left.norm")) for n in names)
    assert names["l2.norm2"].optional and not names["l0.norm2"].optional
    assert names["loop.step"].shape == (3, 64) and names["l1.mlp.table"].shape == (300, 2)
    assert names["l0.mix.left.q"].shape == (64, 64) and names["l0.mix.left.v"].shape == (48, 64)
    assert names["l0.mix.left.o"].shape == (64, 96) and names["l0.mix.left.g"].shape == (96, 64)
    assert names["l0.mix.left.q.norm"].shape == (16,) and names["l0.mix.right.norm"].shape == (8,)
    assert names["l1.mix.q"].shape == (48, 64) and names["l1.mix.v"].shape == (64, 64) and names["l1.mix.q.conv"].shape == (48, 4)
    assert names["l1.mix.b"].shape == (4, 64) and names["l1.mix.dt_bias"].shape == (4,)


def test_round_trip_and_refusals(tmp_path):
    d = make_sipilorn_dir(str(tmp_path / "m"), SP_A, 1, sharp=False)
    cfg = load_config(d)
    back = cfg.to_dict()
    assert back["layers"] == SP_A["layers"] and back["loop"] == SP_A["loop"] and back["logit_softcap"] == 20.0
    assert config_from_dict(json.loads(json.dumps(back))).layer_schedule() == cfg.layer_schedule()
    found = load_model_dir(d)
    names = build_model_skeleton(cfg).expected_tensors()
    check_weights(names, found, set(), d)
    assert "l2.norm2" not in found and found["l1.mlp.table"].dtype == torch.int32
    table = found["l1.mlp.table"]
    assert int(table.min()) >= 0 and int(table.max()) < 5 and bool((table[:, 0] != table[:, 1]).all())
    del found["l0.mix.right.dt_bias"]
    with pytest.raises(WeightError) as e:
        check_weights(names, found, set(), d)
    assert e.value.missing == ["l0.mix.right.dt_bias"]
    for breaker, text in (
            (lambda c: c["layers"][0].update(type="other"), "mixer"),
            (lambda c: c["layers"][1]["mlp"].update(kind="sparse"), "feed-forward"),
            (lambda c: c["layers"][0]["mixer"]["left"].pop("scale"), "scale"),
            (lambda c: c["layers"][0]["mixer"]["left"].update(kv_heads=3), "kv heads"),
            (lambda c: c["layers"][1]["mixer"].update(kv_heads=3), "kv heads"),
            (lambda c: c["layers"][1]["mixer"].update(dim=300), "256"),
            (lambda c: c["layers"][1]["mixer"].update(conv=0), "taps"),
            (lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=20), "rotary"),
            (lambda c: c["layers"][0]["mixer"]["left"]["mask"].update(size=0), "size"),
            (lambda c: c["layers"][0]["mixer"].pop("right"), "right"),
            (lambda c: c["loop"].update(stop=4), "loop"),
            (lambda c: c["loop"].update(times=0), "loop"),
            (lambda c: c.pop("norm"), "norm"),
            (lambda c: c.update(logit_softcap=-1.0), "logit_softcap"),
            (lambda c: c["layers"][1]["mlp"]["router"].update(top=9), "top")):
        bad = copy.deepcopy(SP_A)
        breaker(bad)
        with pytest.raises(ConfigError) as e:
            build_model_skeleton(config_from_dict(bad))
        assert text in str(e.value), (text, str(e.value))


def test_a_table_that_names_an_expert_that_is_not_there_is_refused(tmp_path):
    d = make_sipilorn_dir(str(tmp_path / "m"), SP_D, 2, sharp=False)
    found = load_model_dir(d)
    found["l1.mlp.table"] = found["l1.mlp.table"].clone()
    found["l1.mlp.table"][7, 0] = 4
    model = build_model_skeleton(load_config(d))
    with pytest.raises(ConfigError):
        model.load_tensors(found, torch.float32, "cpu")


def test_the_plain_recurrence_is_the_sum_it_stands_for():
    """With decay 1 and beta 1 and keys that are orthonormal, the delta rule stores each value under its
    key and a later query along that key reads it back; writing a key twice replaces its value."""
    D, E = 4, 3
    k = torch.eye(D, dtype=torch.float64)[[0, 1, 2, 1]].view(4, 1, D)
    v = torch.arange(12, dtype=torch.float64).view(4, 1, E)
    ones = torch.ones(4, 1, dtype=torch.float64)
    o = plain.delta_rule(k, k, v, ones, ones)
    assert torch.equal(o, v)          # the read-out sees the token's own write
    q = torch.eye(D, dtype=torch.float64)[[0, 0, 0, 0]].view(4, 1, D)
    assert torch.equal(plain.delta_rule(q, k, v, ones, ones)[:, 0], v[0, 0].expand(4, E))
    half = plain.delta_rule(q, k, v, ones, 0.5 * ones)[:, 0]
    assert torch.allclose(half[3], v[0, 0] * 0.125)


def test_the_plain_window_and_rotation():
    vis = plain.window_visible(6, 3)
    assert vis[5].tolist() == [False, False, False, True, True, True] and vis[1].tolist() == [True, True] + [False] * 4
    assert bool(plain.window_visible(6, None)[5].all())
    x = torch.ones(3, 1, 6, dtype=torch.float64)
    y = plain.rotate_half_layout(x, 4, 100.0)
    assert torch.equal(y[0], x[0]) and torch.equal(y[..., 4:], x[..., 4:])
    a = torch.tensor(2.0, dtype=torch.float64)
    assert torch.allclose(y[2, 0, 0], torch.cos(a) - torch.sin(a)) and torch.allclose(y[2, 0, 2], torch.cos(a) + torch.sin(a))
    assert torch.allclose(y[2, 0, 1], torch.cos(a / 10) - torch.sin(a / 10))
    conv = plain.causal_conv_silu(torch.tensor([[1.0], [2.0], [3.0]], dtype=torch.float64), torch.tensor([[10.0, 1.0]], dtype=torch.float64))
    assert torch.allclose(conv[:, 0], plain.silu(torch.tensor([1.0, 12.0, 23.0], dtype=torch.float64)))


def test_the_test_configurations_differ_from_each_other():
    seen = set()
    for name, (cfg, _) in SIPILORN_CONFIGS.items():
        key = (cfg["width"], cfg["vocab"], cfg["norm"]["eps"], len(cfg["layers"]))
        assert key not in seen
        seen.add(key)
    assert {L["type"] for L in SP_D["layers"]} == {"delta"} and "loop" not in SP_B and "logit_softcap" not in SP_C
    assert os.path.basename(__file__).startswith("test_")


@pytest.mark.parametrize("name,layer", [("spA", 0), ("spB", 1)])
def test_the_sharpened_weights_show_a_window_that_is_one_token_off_and_a_lost_state(tmp_path, name, layer):
    """What the comparisons on the GPU rest on: in the plain implementation itself, a window one token longer or
    shorter, or a request that goes on from an empty state, moves some row of logits by more than three tenths of
    its largest entry, beyond what any row may differ by in the runs in bfloat16."""
    from helpers import random_tokens, rel_err, tol
    cfg, seed = SIPILORN_CONFIGS[name]
    d = make_sipilorn_dir(str(tmp_path / name), cfg, seed)
    c, P = plain.load(d)
    toks = random_tokens(90, c["vocab"], 5)
    ref = plain.forward(c, P, toks)
    for dw in (-1, 1):
        off = copy.deepcopy(c)
        off["layers"][layer]["mixer"]["left"]["mask"]["size"] += dw
        out = plain.forward(off, P, toks)
        assert max(rel_err(out[i], ref[i]) for i in range(len(toks))) > 0.3 > 4 * tol("bfloat16", name)
    tail = plain.forward(c, P, toks[50:])
    assert max(rel_err(tail[i], ref[50 + i]) for i in range(len(tail))) > 0.3
