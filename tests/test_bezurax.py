"""Bezurax without a GPU: its config.json reader and plan, its tensor names, what it asks of the cache, and the plain
implementation held against hand-worked values."""

from __future__ import annotations

import copy
import math

import pytest
import torch

import bezurax_helpers as bh
import plain_bezurax as plain

F64 = torch.float64


def test_config_is_read_key_by_key_and_refuses_what_it_does_not_know():
    from mini_engine_amd.config.registry import architecture_name_of, get_architecture
    from mini_engine_amd.models.bezurax import BezuraxConfig

    cfg = bh.configs()["A"]
    assert architecture_name_of(cfg) == "Bezurax"
    typed = get_architecture("Bezurax").config_from_dict(cfg)
    assert (typed.vocab, typed.width, typed.logit_scale, typed.norm_eps, typed.norm_groups) == (300, 96, 0.5, 1e-5, 3)
    assert BezuraxConfig.from_dict(typed.to_config_json()) == typed
    for path, value in ((("layers", 0, "type"), "attention"), (("layers", 0, "mixer", "left", "kv_heads"), 3),
                        (("layers", 0, "mixer", "left", "vdim"), 16), (("layers", 0, "mixer", "left", "mask", "pool"), 0),
                        (("layers", 0, "mlp", "kind"), "dense"), (("layers", 2, "weights_of"), 2), (("layers", 2, "weights_of"), 7),
                        (("norm", "groups"), 5)):
        bad = copy.deepcopy(cfg)
        at = bad
        for k in path[:-1]:
            at = at[k]
        at[path[-1]] = value
        with pytest.raises(ValueError):
            BezuraxConfig.from_dict(bad)
    for path in (("layers", 0, "mixer", "left", "scale"), ("layers", 0, "mixer", "right_scale"), ("layers", 0, "mlp", "router", "groups"),
                 ("layers", 1, "mlp", "expert", "limit"), ("logit_scale",)):
        lacking = copy.deepcopy(cfg)
        at = lacking
        for k in path[:-1]:
            at = at[k]
        del at[path[-1]]
        with pytest.raises(ValueError, match=path[-1]):
            BezuraxConfig.from_dict(lacking)


def test_the_decays_inner_size_comes_from_the_tensor(tmp_path):
    """No key of config.json gives the inner size of the decay: a folder's config takes it from the shape of the tensor, also
    for a layer that runs another layer's weights."""
    from mini_engine_amd.models.bezurax import BezuraxConfig, plan_from_config

    cfg = bh.configs()["A"]
    folder = bh.write_folder(str(tmp_path / "a"), cfg, seed=1)
    import json
    import os

    with open(os.path.join(folder, "config.json")) as f:
        written = json.load(f)
    for layer in written["layers"]:
        layer["mixer"]["right"].pop("decay_rank", None)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(written, f)
    with pytest.raises(ValueError, match="w1"):
        plan_from_config(BezuraxConfig.from_dict(written))
    plan = plan_from_config(BezuraxConfig.from_folder(folder))
    assert [layer.mixer.right.decay_rank for layer in plan.layers] == [8, 12]


def test_plan_takes_every_size_and_constant_from_the_config():
    from mini_engine_amd.models.bezurax import BezuraxConfig, plan_from_config

    plan = plan_from_config(BezuraxConfig.from_dict(bh.configs()["A"]))
    assert plan.tie_word_embeddings and plan.logit_scale == 0.5 and plan.vocab_size == 300 and plan.hidden_size == 96
    assert plan.final_norm.groups == 3 and plan.final_norm.eps == 1e-5
    # three runs of two layers' weights: the third entry runs layer 0 again
    assert len(plan.layers) == 2 and plan.order == (0, 1, 0)
    a0, a1 = plan.layers
    assert a0.arrangement == "parallel" and a0.ffn_norm is not None and a0.mixer_norm_name == "l0.norm1" and a0.ffn_norm_name == "l0.norm2"
    assert a0.mixer.kind == "pair" and (a0.mixer.left_scale, a0.mixer.right_scale) == (0.7, 1.2)
    left, right = a0.mixer.left, a0.mixer.right
    assert (left.num_heads, left.num_kv_heads, left.head_dim, left.scale, left.window, left.pooled_block) == (4, 2, 24, 0.2, 40, 5)
    assert left.position is None and left.qk_norm_over == "projection" and left.values_from_keys and left.qk_norm_eps == 1e-5
    assert (right.num_heads, right.head_dim, right.decay_rank, right.norm_eps) == (2, 16, 8, 1e-5)
    assert abs(right.decay_coef - math.exp(-0.5)) < 1e-15
    ff = a0.ffn
    assert (ff.num_experts, ff.top_k, ff.intermediate_size, ff.activation, ff.activation_limit) == (6, 2, 40, "clamped_sigmoid", 1.2)
    assert (ff.scoring, ff.num_groups, ff.keep_groups, ff.route_scale, ff.shared_size, ff.shared_limit) == ("sigmoid_normalized", 3, 2, 1.5, 24, 0.8)
    assert a1.ffn.shared_size == 0 and (a1.mixer.left.window, a1.mixer.left.pooled_block) == (17, 3)
    # a layer without a feed-forward has no second norm
    pb = plan_from_config(BezuraxConfig.from_dict(bh.configs()["B"]))
    assert pb.layers[1].ffn is None and pb.layers[1].ffn_norm is None and pb.order == (0, 1, 1, 0)
    assert pb.final_norm.groups == 1 and pb.final_norm.eps == 1e-6
    # a layer may name one that names another in turn, and a later one: all of them run the tensors of the one that has them
    chain = dict(bh.configs()["B"])
    b0, b1 = chain["layers"][0], chain["layers"][1]
    chain["layers"] = [dict(b0, weights_of=3), dict(b1, weights_of=2), dict(b1, weights_of=3), b0]
    pc = plan_from_config(BezuraxConfig.from_dict(chain))
    assert len(pc.layers) == 1 and pc.order == (0, 0, 0, 0) and pc.layers[0].mixer_prefix == "l3.mix"


def test_tensor_names_and_shapes():
    _, wants = bh.wants_of(bh.configs()["A"])
    assert wants["embed"].shape == (300, 96) and wants["final.norm"].shape == (96,) and "head" not in wants
    assert wants["l0.norm1"].shape == (96,) and wants["l0.norm2"].shape == (96,)
    assert wants["l0.mix.left.q"].shape == (96, 96) and wants["l0.mix.left.k"].shape == (48, 96) and "l0.mix.left.v" not in wants
    assert wants["l0.mix.left.q.norm"].shape == (96,) and wants["l0.mix.left.k.norm"].shape == (48,) and wants["l0.mix.left.o"].shape == (96, 96)
    for role in ("r", "k", "v", "g", "a"):
        assert wants[f"l0.mix.right.{role}"].shape == (32, 96)
    assert wants["l0.mix.right.w1"].shape == (8, 96) and wants["l0.mix.right.w2"].shape == (32, 8)
    assert all(wants[f"l0.mix.right.{r}"].shape == (32,) for r in ("w0", "a.b", "norm")) and wants["l0.mix.right.o"].shape == (96, 32)
    assert wants["l0.mlp.router"].shape == (6, 96) and wants["l0.mlp.e5.gate"].shape == (40, 96) and wants["l0.mlp.e0.down"].shape == (96, 40)
    assert wants["l0.mlp.shared.up"].shape == (24, 96) and wants["l0.mlp.shared.down"].shape == (96, 24) and wants["l0.mlp.shared.sg"].shape == (1, 96)
    assert "l1.mlp.shared.sg" not in wants and wants["l1.mix.right.r"].shape == (72, 96)
    assert not any(n.startswith("l2.") for n in wants)  # the third layer runs the first one's
    _, wants_b = bh.wants_of(bh.configs()["B"])
    assert "l1.norm2" not in wants_b and not any(n.startswith("l1.mlp") for n in wants_b)


def test_every_run_of_a_layer_gets_pages_pooled_pages_and_a_state_of_its_own():
    from mini_engine_amd.cache.storage import plan_layout
    from mini_engine_amd.models.bezurax import BezuraxConfig, plan_from_config
    from mini_engine_amd.parts.base import KVCacheNeed, StateNeed
    from mini_engine_amd.parts.decoder import Decoder

    decoder = Decoder(plan_from_config(BezuraxConfig.from_dict(bh.configs()["A"])), torch.float32, "cpu")
    needs = [decoder.blocks[i].mixer.cache_need() for i in decoder.plan.order]
    assert all(isinstance(n, tuple) and isinstance(n[0], KVCacheNeed) and isinstance(n[1], StateNeed) for n in needs)
    assert (needs[0][0].window, needs[0][0].pooled_block, needs[0][0].num_kv_heads, needs[0][0].head_dim) == (40, 5, 2, 24)
    assert needs[0][1].shape == (2, 16, 16) and needs[1][1].shape == (3, 24, 24) and needs[1][1].dtype == torch.float32
    layout = plan_layout(decoder)
    # three runs, three sets of pages and three states; pages behind a window with pooled blocks are never given back early
    assert sorted(layout.layer_group) == [0, 1, 2] and sorted(layout.state_layers) == [0, 1, 2]
    assert all(g.window == 0 for g in layout.groups)


# ------------------------------------------------------------------------------ the plain implementation by hand
def test_plain_norm_in_groups_by_hand():
    x = torch.tensor([[3.0, 4.0, 0.0, 2.0]], dtype=F64)
    got = plain.group_rms_norm(x, torch.tensor([1.0, 2.0, 3.0, 0.5], dtype=F64), 2, 0.0)
    want = [3 / math.sqrt(12.5), 2 * 4 / math.sqrt(12.5), 0.0, 0.5 * 2 / math.sqrt(2.0)]
    assert torch.allclose(got, torch.tensor([want], dtype=F64))
    one = plain.group_rms_norm(x, torch.ones(4, dtype=F64), 1, 0.25)
    assert torch.allclose(one, x / math.sqrt(29 / 4 + 0.25))


def test_plain_window_and_pooled_blocks_by_hand():
    tokens, blocks = plain.pooled_window_visibility(12, window=4, pool=3)
    assert blocks.shape == (12, 4)
    # position 7 sees 4..7; block 0 (0..2) ends at 2 <= 3 and is seen, block 1 (3..5) ends at 5 > 3 and is not: token 3 is not
    # seen at all
    assert tokens[7].nonzero().flatten().tolist() == [4, 5, 6, 7] and blocks[7].tolist() == [True, False, False, False]
    # position 9: 6..9, and block 1 ends at 5 <= 5
    assert tokens[9].nonzero().flatten().tolist() == [6, 7, 8, 9] and blocks[9].tolist() == [True, True, False, False]
    assert not blocks[5].any() and blocks[6].tolist() == [True, False, False, False] and tokens[2].tolist()[:4] == [True, True, True, False]
    # a block of one key: every token that has left the window is seen again as a block
    tokens1, blocks1 = plain.pooled_window_visibility(6, window=2, pool=1)
    assert torch.equal(tokens1 | blocks1, torch.ones(6, 6, dtype=torch.bool).tril()) and not (tokens1 & blocks1).any()


def test_plain_attention_takes_values_from_the_keys_and_pools_means():
    """One head of two elements, identity projections: with the scale 0 all visible entries weigh the same, so the result is
    the plain mean of the visible values, and those are the keys before their norm."""
    d = 2
    w = {"p.q": torch.eye(d, dtype=F64), "p.k": torch.eye(d, dtype=F64), "p.o": torch.eye(d, dtype=F64),
         "p.q.norm": torch.ones(d, dtype=F64), "p.k.norm": torch.tensor([5.0, 7.0], dtype=F64)}
    m = {"heads": 1, "kv_heads": 1, "dim": d, "vdim": d, "scale": 0.0, "mask": {"size": 2, "pool": 2}}
    h = torch.tensor([[1.0, 0.0], [3.0, 0.0], [0.0, 2.0], [0.0, 4.0], [8.0, 8.0]], dtype=F64)
    out = plain.pooled_window_attention(h, w, "p", m, 1e-6)
    assert torch.allclose(out[1], (h[0] + h[1]) / 2)
    assert torch.allclose(out[2], (h[1] + h[2]) / 2)  # token 0 has left the window and its block is not yet wholly before it
    assert torch.allclose(out[3], ((h[0] + h[1]) / 2 + h[2] + h[3]) / 3)  # block 0 counts once, as the mean of its two values
    assert torch.allclose(out[4], ((h[0] + h[1]) / 2 + h[3] + h[4]) / 3)


def test_plain_delta_rule_by_hand():
    """One head of one element: S_t = w S - a u (u S) + k v with u = k / sqrt(k^2 + 1e-6), o = S r; the head's norm turns o into
    its sign."""
    z = torch.zeros(1, 1, dtype=F64)
    one = torch.ones(1, 1, dtype=F64)
    w = {"p.r": one, "p.k": 2 * one, "p.v": 3 * one, "p.g": z, "p.a": z, "p.a.b": torch.zeros(1, dtype=F64), "p.w1": z, "p.w2": z,
         "p.w0": torch.zeros(1, dtype=F64), "p.norm": torch.ones(1, dtype=F64), "p.o": one}
    h = torch.tensor([[1.0], [-0.5]], dtype=F64)
    out, S = plain.delta_rule(h, w, "p", {"heads": 1, "dim": 1}, 0.0)
    decay = math.exp(-math.exp(-0.5) * 0.5)  # sigmoid(0) = 1/2 inside
    s1 = 2 * 3
    u2 = -1 / math.sqrt(1 + 1e-6)
    s2 = decay * s1 - 0.5 * u2 * u2 * s1 + (-1.0) * (-1.5)
    assert abs(float(S) - s2) < 1e-12
    # o_1 = s1 * 1 > 0, o_2 = s2 * (-0.5) < 0; over their root mean square +1 and -1; times sigmoid(0) of the gate
    assert torch.allclose(out.flatten(), torch.tensor([0.5, -0.5], dtype=F64))
    # carried state: the second token from the first token's state gives the same
    _, first = plain.delta_rule(h[:1], w, "p", {"heads": 1, "dim": 1}, 0.0)
    _, second = plain.delta_rule(h[1:], w, "p", {"heads": 1, "dim": 1}, 0.0, state=first)
    assert abs(float(second) - s2) < 1e-12


def test_plain_delta_rule_removes_along_the_unit_key():
    """With a = 1 and no decay to speak of, writing a key that is already stored first takes out what the state held along it."""
    d = 3
    big = 40.0  # sigmoid(40) = 1 for a; w0 = -40 makes the decay exp(0) = 1
    eye = torch.eye(d, dtype=F64)
    z = torch.zeros(d, d, dtype=F64)
    w = {"p.r": eye, "p.k": eye, "p.v": eye, "p.g": z, "p.a": z, "p.a.b": torch.full((d,), big, dtype=F64), "p.w1": torch.zeros(1, d, dtype=F64),
         "p.w2": torch.zeros(d, 1, dtype=F64), "p.w0": torch.full((d,), -big, dtype=F64), "p.norm": torch.ones(d, dtype=F64), "p.o": eye}
    e0 = torch.tensor([[2.0, 0.0, 0.0]], dtype=F64)
    _, S = plain.delta_rule(torch.cat((e0, e0)), w, "p", {"heads": 1, "dim": d}, 0.0)
    # after the first token S = k v^T = 4 at [0, 0]; the second removes u u^T S (all of it) and writes 4 again
    assert abs(float(S[0, 0, 0]) - 4.0) < 1e-5 and float(S.abs().sum()) - float(S[0, 0, 0]) < 1e-9


def test_plain_router_keeps_groups_and_weighs_by_scores():
    r = {"experts": 6, "top": 2, "groups": {"count": 3, "keep": 2}, "scale": 3.0}
    logit = lambda p: math.log(p / (1 - p))
    # scores: group 0 = (0.9, 0.1), group 1 = (0.6, 0.5), group 2 = (0.55, 0.5): sums 1.0, 1.1, 1.05: group 0 is dropped although it
    # holds the largest score; the picks are 0.6 and 0.55
    z = torch.tensor([[logit(p) for p in (0.9, 0.1, 0.6, 0.5, 0.55, 0.5)]], dtype=F64)
    picked, weights = plain.route(z, r)
    assert sorted(picked[0].tolist()) == [2, 4]
    by = dict(zip(picked[0].tolist(), weights[0].tolist()))
    assert abs(by[2] - 3.0 * 0.6 / 1.15) < 1e-12 and abs(by[4] - 3.0 * 0.55 / 1.15) < 1e-12
    # groups of one expert: a group's score is that expert's
    one = {"experts": 3, "top": 1, "groups": {"count": 3, "keep": 1}, "scale": 1.0}
    picked, weights = plain.route(torch.tensor([[0.0, 2.0, 1.0]], dtype=F64), one)
    assert picked.tolist() == [[1]] and abs(float(weights) - 1.0) < 1e-12


def test_plain_expert_clamps_before_the_activation():
    eye = torch.eye(2, dtype=F64)
    w = {"e.gate": eye, "e.up": eye, "e.down": eye}
    h = torch.tensor([[5.0, -9.0], [-3.0, 0.5]], dtype=F64)
    got = plain.clamped_expert(torch.stack((h[0], torch.tensor([h[1, 0], h[1, 1]], dtype=F64))), w, "e", 2.0)
    sig = lambda g: 1 / (1 + math.exp(-1.702 * g))
    # gate clamped from above only; up clamped on both sides, plus one
    want = [[2.0 * sig(2.0) * (2.0 + 1), -9.0 * sig(-9.0) * (-2.0 + 1)], [-3.0 * sig(-3.0) * (2.0 + 1), 0.5 * sig(0.5) * (0.5 + 1)]]
    got2 = plain.clamped_expert(torch.tensor([[5.0, -9.0]], dtype=F64), {"e.gate": eye, "e.up": torch.tensor([[0.0, 1.0], [1.0, 0.0]], dtype=F64), "e.down": eye}, "e", 2.0)
    assert torch.allclose(got2, torch.tensor([[2.0 * sig(2.0) * (-2.0 + 1), -9.0 * sig(-9.0) * (2.0 + 1)]], dtype=F64))
    assert torch.allclose(got[0], torch.tensor([2.0 * sig(2.0) * 3.0, -9.0 * sig(-9.0) * (-2.0 + 1)], dtype=F64))
    assert torch.allclose(got[1], torch.tensor([-3.0 * sig(-3.0) * (-2.0 + 1), 0.5 * sig(0.5) * 1.5], dtype=F64)) and len(want) == 2


def test_plain_shared_expert_is_added_for_every_token_through_its_gate():
    cfg = bh.configs()["A"]
    mlp = cfg["layers"][0]["mlp"]
    w = {k: v.to(F64) for k, v in bh.random_tensors(cfg, 3).items()}
    g = torch.Generator().manual_seed(0)
    h = torch.randn(5, 96, generator=g, dtype=F64)
    with_shared = plain.routed_experts(h, w, "l0.mlp", mlp)
    without = plain.routed_experts(h, w, "l0.mlp", dict(mlp, shared=None))
    gate = torch.sigmoid(h @ w["l0.mlp.shared.sg"].T)
    assert gate.shape == (5, 1)
    assert torch.allclose(with_shared - without, gate * plain.clamped_expert(h, w, "l0.mlp.shared", 0.8))


def test_plain_forward_runs_a_layers_weights_again_and_scales_the_logits():
    cfg = bh.configs()["A"]
    w = bh.random_tensors(cfg, 5)
    toks = [3, 17, 250, 9, 9, 41]
    res: list = []
    logits = plain.forward(cfg, w, toks, residuals=res)
    assert logits.shape == (6, 300) and len(res) == 3
    twice = copy.deepcopy(cfg)
    twice["logit_scale"] = 1.0
    assert torch.allclose(plain.forward(twice, w, toks) * 0.5, logits)
    # the third run uses layer 0's weights: with its own copy of them under another name the result is the same
    own = copy.deepcopy(cfg)
    own["layers"][2] = copy.deepcopy(cfg["layers"][0])
    w2 = dict(w)
    w2.update({"l2" + k[2:]: v for k, v in w.items() if k.startswith("l0.")})
    assert torch.allclose(plain.forward(own, w2, toks), logits)
    # causal: a later token changes nothing before it
    assert torch.allclose(plain.forward(cfg, w, toks[:4]), logits[:4])
