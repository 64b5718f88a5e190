"""CPU checks of the Mepatar serving path that need no GPU: the plain oracle's mechanisms against closed forms and against each other, the configuration
reader, the checkpoint loader's fused layouts, the named states of the slot cache and the step descriptors."""

import json
import math

import pytest
import torch

from oracle import mepatar as O
from tests import mepatar_util as U

F64 = torch.float64


def test_group_norm_is_a_norm_per_group():
    g = torch.Generator().manual_seed(0)
    x, w = torch.randn(5, 24, generator=g, dtype=F64), torch.rand(24, generator=g, dtype=F64) + 0.5
    got = O.group_rms_norm(x, w, 3, 1e-6)
    for i in range(3):
        part = x[:, 8 * i : 8 * i + 8]
        assert torch.allclose(got[:, 8 * i : 8 * i + 8], part / torch.sqrt((part ** 2).mean(-1, keepdim=True) + 1e-6) * w[8 * i : 8 * i + 8])
    assert torch.allclose(O.group_rms_norm(x, w, 1, 1e-6), O.unit_rms(x, 1e-6) * w)


def test_causal_conv_matches_a_library_convolution_and_starts_from_zeros():
    g = torch.Generator().manual_seed(1)
    h, w = torch.randn(11, 6, generator=g, dtype=F64), torch.randn(6, 4, generator=g, dtype=F64)
    want = torch.nn.functional.conv1d(torch.nn.functional.pad(h.T[None], (3, 0)), w[:, None, :], groups=6)[0].T
    assert torch.allclose(O.causal_conv(h, w), want)
    assert torch.allclose(O.causal_conv(h, w)[0], w[:, -1] * h[0])  # the last column weighs the current token


def test_rotary_layouts_pair_the_right_entries_and_keep_the_rest():
    x = torch.arange(2 * 1 * 8, dtype=F64).reshape(2, 1, 8) + 1
    for layout, pairs in (("half", [(0, 2), (1, 3)]), ("interleaved", [(0, 1), (2, 3)])):
        y = O.rotary(x, 4, 100.0, layout)
        assert torch.equal(y[0], x[0]) and torch.equal(y[:, :, 4:], x[:, :, 4:])  # position 0 and the entries beyond dims stay
        for i, (a, b) in enumerate(pairs):
            ang = 1.0 * 100.0 ** (-2.0 * i / 4)
            assert math.isclose(float(y[1, 0, a]), float(x[1, 0, a]) * math.cos(ang) - float(x[1, 0, b]) * math.sin(ang))
            assert math.isclose(float(y[1, 0, b]), float(x[1, 0, b]) * math.cos(ang) + float(x[1, 0, a]) * math.sin(ang))


def test_retention_is_a_decayed_sum_over_the_past():
    g = torch.Generator().manual_seed(2)
    T, dk, dv = 9, 4, 3
    q, k, v = torch.randn(T, 1, dk, generator=g, dtype=F64), torch.randn(T, 1, dk, generator=g, dtype=F64), torch.randn(T, 1, dv, generator=g, dtype=F64)
    got = O.retention(q, k, v, [0.8])
    for t in range(T):
        want = sum(0.8 ** (t - s) * (q[t, 0] @ k[s, 0]) * v[s, 0] for s in range(t + 1))
        assert torch.allclose(got[t, 0], want)


def test_window_mask_edges():
    assert O.visible(10, 10, 1, 0) and not O.visible(10, 9, 1, 0) and not O.visible(10, 11, 5, 0)
    assert O.visible(10, 6, 5, 0) and not O.visible(10, 5, 5, 0)
    assert O.visible(10, 2, 5, 3) and not O.visible(10, 3, 5, 3)
    # with one hot key the output is its value exactly when it is visible
    T = 12
    q, k, v = torch.ones(T, 2, 2, dtype=F64) * 5, torch.zeros(T, 1, 2, dtype=F64), torch.zeros(T, 1, 3, dtype=F64)
    k[4], v[4] = 5.0, 1.0
    out = O.window_attention(q, k, v, 1.0, torch.ones(2, dtype=F64), 3, 0)
    assert out[6, 1, 0] > 0.99 and out[7, 1, 0] == 0 and out[3, 0, 0] == 0


def test_delta_rule_stores_and_overwrites_a_value():
    """With beta = 1 and no decay a unit key retrieves exactly the last value written under it."""
    k = torch.zeros(3, 1, 4, dtype=F64)
    k[:, 0, 1] = 1.0
    v = torch.tensor([[[1.0, 2.0]], [[5.0, -1.0]], [[0.5, 0.5]]], dtype=F64)
    one = torch.ones(3, 1, dtype=F64)
    out = O.delta_rule(k.clone(), k, v, one, one)
    assert torch.allclose(out, v)
    out = O.delta_rule(k.clone(), k, v, one * 0.5, one)  # half steps from what is stored towards the new value
    assert torch.allclose(out[0, 0], 0.5 * v[0, 0]) and torch.allclose(out[1, 0], 0.5 * (0.5 * v[0, 0]) + 0.5 * v[1, 0])


def test_router_weights_are_the_softmax_scores_not_renormalised():
    g = torch.Generator().manual_seed(3)
    h, w = torch.randn(7, 5, generator=g, dtype=F64), torch.randn(6, 5, generator=g, dtype=F64)
    ids, wts = O.route(h, w, 2)
    s = torch.softmax(h @ w.T, -1)
    assert torch.allclose(wts, torch.gather(s, 1, ids)) and bool((wts.sum(-1) < 1).all())
    assert torch.equal(ids[:, 0], s.argmax(-1))


def test_expert_clamps_gate_above_and_up_on_both_sides():
    w = {"e.gate": torch.tensor([[10.0], [-10.0]], dtype=F64), "e.up": torch.tensor([[10.0], [-10.0]], dtype=F64), "e.down": torch.eye(2, dtype=F64)}
    y = O.expert_ff(torch.ones(1, 1, dtype=F64), w, "e.", 2.0)[0]
    assert math.isclose(float(y[0]), 2.0 / (1 + math.exp(-1.702 * 2.0)) * 3.0)       # gate 10 -> 2, up 10 -> 2
    assert math.isclose(float(y[1]), -10.0 / (1 + math.exp(1.702 * 10.0)) * (-1.0))  # gate -10 stays, up -10 -> -2


def test_whole_sequence_equals_its_prefix():
    """Causality of the whole oracle: the logits of a prefix do not change when tokens follow."""
    cfg = U.make_config(U.default_layers())
    w = U.make_weights(cfg, 1)
    toks = [3, 17, 99, 4, 4, 60, 12, 7, 100, 31, 5, 88]
    full = O.forward(toks, w, cfg)
    assert torch.allclose(O.forward(toks[:7], w, cfg), full[:7], atol=1e-12)


def test_config_reader_and_loader_fuse_the_projections(tmp_path):
    from llm_quest_amd import registry
    from llm_quest_amd.mepatar.mepatar_model import MepatarConfig

    cfg = U.make_config(U.default_layers())
    w = U.make_weights(cfg, 2)
    model = registry.load_model(U.save(str(tmp_path), cfg, w), "float32", "cpu")
    assert "Mepatar" in registry.architectures() and model.vocab_size == cfg["vocab"]
    b0, b1, b2, b3 = model.blocks[0], model.blocks[1], model.blocks[2], model.blocks[3]
    assert torch.equal(b0.mixer.w_in, torch.cat([w["l0.mix.q"], w["l0.mix.k"], w["l0.mix.v"], w["l0.mix.g"]]))
    assert torch.equal(b1.mixer.w_qkv, torch.cat([w["l1.mix.q"], w["l1.mix.k"], w["l1.mix.v"]])) and torch.equal(b1.mixer.b_qkv, torch.cat([w["l1.mix.q.b"], w["l1.mix.k.b"], w["l1.mix.v.b"]]))
    assert torch.equal(b2.mixer.w_in, torch.cat([w["l2.mix." + n] for n in "qkvgba"])) and torch.equal(b2.mixer.conv, torch.cat([w["l2.mix." + n + ".conv"] for n in "qkv"]))
    gu = b0.ff.w_gate_up[5]  # 40 rows of gate and up each -> two blocks of [32 gate | 32 up], the second one padded with zero rows
    assert gu.shape[0] == 128 and torch.equal(gu[:32], w["l0.mlp.e5.gate"][:32]) and torch.equal(gu[32:64], w["l0.mlp.e5.up"][:32])
    assert torch.equal(gu[64:72], w["l0.mlp.e5.gate"][32:]) and torch.equal(gu[96:104], w["l0.mlp.e5.up"][32:]) and float(gu[72:96].abs().max()) == 0 and float(gu[104:].abs().max()) == 0
    assert torch.equal(b1.ff.w_gate_up, torch.cat([w["l1.mlp.gate"], w["l1.mlp.up"]]))
    assert b3.ff is None and torch.equal(b0.canon.weight, w["l0.canon1"])
    bad = json.loads(json.dumps(cfg))
    bad["layers"][0]["type"] = "convolution"
    with pytest.raises(ValueError):
        MepatarConfig(bad)
    bad = json.loads(json.dumps(cfg))
    bad["norm"]["groups"] = 5
    with pytest.raises(ValueError):
        MepatarConfig(bad)


def test_slot_cache_named_states_and_step_descriptors(tmp_path):
    from llm_quest_amd import registry
    from llm_quest_amd.common.mixers import SeqStep

    cfg = U.make_config(U.default_layers())
    model = registry.load_model(U.save(str(tmp_path), cfg, U.make_weights(cfg, 3)), "float32", "cpu")
    cache = model.new_cache("cpu", max_tokens=16, slots=1)
    assert cache.rows[0] is None and cache.rows[1].shape == (1, 16, 2 * (24 + 40)) and set(cache.named[2]) == {"S", "conv", "canon"}
    assert cache.state(2, "conv").shape == (1, 3, 2 * 2 * 24 + 4 * 40) and cache.state(0, "canon").shape == (1, 2, 72)
    a = cache.open("a")
    cache.state(0, "S")[a].fill_(3.0)
    cache.state(2, "conv")[a].fill_(3.0)
    b = cache.open("b")  # a second slot appears: the first one's state stays, the new one starts at zero
    assert cache.slots == 2 and float(cache.state(0, "S")[a].min()) == 3.0 and float(cache.state(0, "S")[b].abs().max()) == 0.0
    cache.advance(a, [5, 6, 7])
    st = SeqStep(cache, [(a, [1, 2]), (b, [9, 8, 7])], "cpu", torch.float32)
    assert st.row_seq.tolist() == [0, 0, 1, 1, 1] and st.pos.tolist() == [3, 4, 0, 1, 2] and st.seq_off.tolist() == [0, 2, 5] and not st.fresh
    cache.close("a")
    c = cache.open("c")  # the freed slot comes back zeroed
    assert c == a and float(cache.state(0, "S")[c].abs().max()) == 0.0 and float(cache.state(2, "conv")[c].abs().max()) == 0.0 and cache.length[c] == 0
