"""Sevadra without a GPU: its config.json reader and plan, its tensor names, what it asks of the cache, and the plain
implementation held against hand-worked values."""

from __future__ import annotations

import copy
import json
import math
import os

import pytest
import torch

import plain_sevadra as plain
import sevadra_helpers as sh

F64 = torch.float64


def _set(cfg, path, value):
    out = copy.deepcopy(cfg)
    at = out
    for k in path[:-1]:
        at = at[k]
    if value is KeyError:
        del at[path[-1]]
    else:
        at[path[-1]] = value
    return out


def test_config_is_read_key_by_key_and_refuses_what_it_cannot_run():
    from mini_engine_amd.config.registry import architecture_name_of, get_architecture
    from mini_engine_amd.models.sevadra import SevadraConfig

    cfg = sh.configs()["A"]
    assert architecture_name_of(cfg) == "Sevadra"
    typed = get_architecture("Sevadra").config_from_dict(cfg)
    assert (typed.vocab, typed.width, typed.norm_eps, typed.side_dim, len(typed.layers)) == (300, 96, 1e-5, 8, 5)
    assert SevadraConfig.from_dict(typed.to_config_json()) == typed
    assert SevadraConfig.from_dict(sh.configs()["B"]).side_dim == 0
    for path, value in ((("layers", 0, "type"), "retention"), (("layers", 2, "mixer", "kv_heads"), 3), (("layers", 2, "mixer", "rot", "dims"), 26),
                        (("layers", 2, "mixer", "rot", "dims"), 7), (("layers", 1, "mixer", "left", "kv_heads"), 3), (("layers", 0, "mlp", "kind"), "gated"),
                        (("layers", 3, "mixer", "kv_from"), 3), (("layers", 3, "mixer", "kv_from"), 1), (("layers", 3, "mixer", "kv_from"), 4),
                        (("layers", 3, "mixer", "kv_rank"), 16), (("layers", 3, "mixer", "rot", "base"), 5.0)):
        with pytest.raises(ValueError):
            SevadraConfig.from_dict(_set(cfg, path, value))
    for path in (("layers", 0, "mixer", "scale"), ("layers", 0, "mixer", "kv_rank"), ("layers", 1, "mixer", "right_scale"), ("layers", 1, "mixer", "right", "dim"),
                 ("layers", 1, "mlp", "router", "top"), ("layers", 1, "mlp", "expert", "ff"), ("layers", 2, "mixer", "rot", "scaling", "high"),
                 ("layers", 4, "mlp", "ff"), ("norm", "eps"), ("width",)):
        with pytest.raises(ValueError, match=path[-1]):
            SevadraConfig.from_dict(_set(cfg, path, KeyError))


def test_what_no_key_gives_comes_from_the_tensors(tmp_path):
    """The decay's inner size is the row count of its tensor; a router has a correction when the checkpoint holds one."""
    from mini_engine_amd.models.sevadra import SevadraConfig, plan_from_config

    cfg = sh.configs()["A"]
    tensors = sh.random_tensors(cfg, 1)
    del tensors["l2.mlp.correction"]
    folder = sh.write_folder(str(tmp_path / "a"), cfg, tensors=tensors)
    with open(os.path.join(folder, "config.json")) as f:
        written = json.load(f)
    assert "decay_rank" not in written["layers"][1]["mixer"]["right"]
    with pytest.raises(ValueError, match="w1"):
        plan_from_config(SevadraConfig.from_dict(written))
    plan = plan_from_config(SevadraConfig.from_folder(folder))
    assert plan.layers[1].mixer.right.decay_rank == 8
    assert plan.layers[1].ffn.score_correction and not plan.layers[2].ffn.score_correction


def test_plan_takes_every_size_and_constant_from_the_config():
    from mini_engine_amd.models.sevadra import SevadraConfig, plan_from_config

    plan = plan_from_config(SevadraConfig.from_dict(sh.configs()["A"]))
    assert plan.tie_word_embeddings and plan.vocab_size == 300 and plan.hidden_size == 96 and plan.order == (0, 1, 2, 3, 4)
    assert plan.final_norm.eps == 1e-5 and plan.final_norm.groups == 1 and plan.token_table_columns == 40
    l0, l1, l2, l3, l4 = plan.layers
    assert all(lay.arrangement == "result_norm" for lay in plan.layers)
    assert [lay.token_input.index for lay in plan.layers] == [0, 1, 2, 3, 4] and l2.token_input.dim == 8 and l2.token_input.prefix == "l2.side"
    m = l0.mixer
    assert (m.kind, m.num_heads, m.head_dim, m.rotary_dim, m.value_dim, m.latent_rank, m.scale, m.cache_from) == ("latent_attention", 4, 16, 8, 24, 32, 0.2, None)
    assert m.position.pairing == "neighbours" and m.position.rotary_dim == 8 and m.output_gate and not m.sink
    assert (l0.ffn.kind, l0.ffn.intermediate_size, l0.ffn.activation) == ("activated_mlp", 160, "relu2")
    left, right = l1.mixer.left, l1.mixer.right
    assert (l1.mixer.kind, l1.mixer.left_scale, l1.mixer.right_scale) == ("pair", 0.7, 1.2)
    assert (left.num_heads, left.num_kv_heads, left.head_dim, left.v_dim, left.scale, left.softcap, left.unit_sink) == (4, 2, 24, 16, 0.25, 3.0, True)
    assert left.position is None and left.conv_taps == 0 and left.qk_norm_over == "projection" and left.window == 0
    assert (right.kind, right.num_heads, right.head_dim, right.decay_rank) == ("time_mix", 2, 16, 8)
    f = l1.ffn
    assert (f.num_experts, f.identity_experts, f.top_k, f.intermediate_size, f.shared_size) == (6, 2, 2, 40, 24)
    assert (f.scoring, f.gated, f.shared_gated, f.activation, f.score_correction) == ("softmax_all", False, False, "relu2", True)
    a = l2.mixer
    assert (a.conv_taps, a.softcap, a.unit_sink, a.v_dim, a.position.kind, a.position.rotary_dim) == (3, 0.0, False, 32, "scaled_rotary", 16)
    assert (a.position.factor, a.position.low, a.position.high, a.position.original, a.position.pairing) == (4.0, 1.0, 4.0, 64.0, "halves")
    assert l3.mixer.cache_from == 0 and l3.ffn is None and l3.ffn_norm is None
    assert l4.mixer.position.kind == "rotary" and l4.mixer.position.theta == 500.0 and l4.mixer.conv_taps == 0


def test_tensor_names_and_shapes():
    _, wants = sh.wants_of(sh.configs()["A"])
    shapes = {k: tuple(v.shape) for k, v in wants.items()}
    expect = {
        "embed": (300, 96), "side.embed": (300, 40), "final.norm": (96,), "l0.norm1": (96,), "l0.norm2": (96,),
        "l0.mix.q": (4 * 24, 96), "l0.mix.dkv": (40, 96), "l0.mix.dkv.norm": (32,), "l0.mix.uk": (64, 32), "l0.mix.uv": (96, 32), "l0.mix.g": (4, 96),
        "l0.mix.o": (96, 96), "l0.mlp.up": (160, 96), "l0.mlp.down": (96, 160), "l0.side.gate": (8, 96), "l0.side.proj": (96, 8), "l0.side.norm": (96,),
        "l1.mix.left.q": (96, 96), "l1.mix.left.k": (48, 96), "l1.mix.left.v": (32, 96), "l1.mix.left.q.norm": (96,), "l1.mix.left.k.norm": (48,),
        "l1.mix.left.o": (96, 64), "l1.mix.right.mu.w": (96,), "l1.mix.right.r": (32, 96), "l1.mix.right.w1": (8, 96), "l1.mix.right.w2": (32, 8),
        "l1.mix.right.w0": (32,), "l1.mix.right.u": (2, 16), "l1.mix.right.norm": (32,), "l1.mix.right.o": (96, 32),
        "l1.mlp.router": (8, 96), "l1.mlp.correction": (8,), "l1.mlp.e5.up": (40, 96), "l1.mlp.e5.down": (96, 40), "l1.mlp.shared.up": (24, 96),
        "l2.mix.q.conv": (96, 3), "l2.mix.k.conv": (48, 3), "l2.mix.v.conv": (64, 3), "l2.mix.o": (96, 128), "l2.mlp.router": (5, 96),
        "l3.mix.q": (2 * 32, 96), "l3.mix.uk": (48, 32), "l3.mix.uv": (32, 32), "l3.mix.g": (2, 96),
    }
    for name, shape in expect.items():
        assert shapes.get(name) == shape, (name, shapes.get(name), shape)
    for absent in ("l3.mix.dkv", "l3.mix.dkv.norm", "l3.norm2", "l1.mlp.e6.up", "l1.mlp.e0.gate", "l1.mlp.shared.gate", "l4.mix.q.conv", "head",
                   "l1.mix.left.q.conv", "l2.mlp.shared.up"):
        assert absent not in shapes, absent
    assert "side.embed" not in sh.wants_of(sh.configs()["B"])[1]


def test_what_the_mixers_ask_of_the_cache():
    from mini_engine_amd.cache.storage import plan_layout
    from mini_engine_amd.models.sevadra import SevadraConfig, plan_from_config
    from mini_engine_amd.parts.base import KVCacheNeed, StateNeed
    from mini_engine_amd.parts.decoder import Decoder

    dec = Decoder(plan_from_config(SevadraConfig.from_dict(sh.configs()["A"])), torch.float32, "cpu")
    needs = [b.mixer.cache_need() for b in dec.blocks]
    assert needs[0] == KVCacheNeed(1, 40, 0, value_dim=32)  # one key/value head: the latent and the shared key part
    assert needs[1] == (KVCacheNeed(2, 24, 0, value_dim=16), StateNeed((2 * 16 * 16 + 96,), torch.float32))  # pages; S and the last input
    assert needs[2] == (KVCacheNeed(2, 24, 0, value_dim=32), StateNeed((2 * (96 + 48 + 64),), torch.float32))  # pages; two projections
    assert needs[3] is None and dec.cache_owner == [0, 1, 2, 0, 4]
    assert needs[4] == KVCacheNeed(6, 16, 0, value_dim=16)
    layout = plan_layout(dec)
    assert sorted(layout.state_layers) == [1, 2] and sorted(layout.layer_group) == [0, 1, 2, 4]


# ------------------------------------------------------------------------------ the plain implementation by hand
def test_slowed_rotation_frequencies_by_hand():
    f = plain.rotary_frequencies(sh.rot(100.0, 8, (8.0, 2.0, 3.0, 40)))
    plainf = [100.0 ** (-2 * i / 8) for i in range(4)]
    # wavelengths 6.28, 19.9, 62.8, 198.7 against 40/3 = 13.3 and 40/2 = 20: as it is; blended; slowed; slowed
    s = (40 / (2 * math.pi / plainf[1]) - 2.0) / (3.0 - 2.0)
    want = [plainf[0], (1 - s) * plainf[1] / 8 + s * plainf[1], plainf[2] / 8, plainf[3] / 8]
    assert 0 < s < 1 and torch.allclose(f, torch.tensor(want, dtype=F64), rtol=1e-12)
    assert torch.allclose(plain.rotary_frequencies(sh.rot(100.0, 8)), torch.tensor(plainf, dtype=F64), rtol=1e-12)


def test_rotation_layouts_by_hand():
    x = torch.arange(1.0, 7.0, dtype=F64).reshape(1, 1, 6)
    pos = torch.tensor([3])
    r = {"base": 10.0, "dims": 4}
    a0, a1 = 3.0, 3.0 * 10.0 ** -0.5
    halves = plain.rotate(x, pos, r, "halves")[0, 0]
    want = [1 * math.cos(a0) - 3 * math.sin(a0), 2 * math.cos(a1) - 4 * math.sin(a1), 3 * math.cos(a0) + 1 * math.sin(a0), 4 * math.cos(a1) + 2 * math.sin(a1), 5, 6]
    assert torch.allclose(halves, torch.tensor(want, dtype=F64), atol=1e-12)
    inter = plain.rotate(x, pos, r, "interleaved")[0, 0]
    want = [1 * math.cos(a0) - 2 * math.sin(a0), 2 * math.cos(a0) + 1 * math.sin(a0), 3 * math.cos(a1) - 4 * math.sin(a1), 4 * math.cos(a1) + 3 * math.sin(a1), 5, 6]
    assert torch.allclose(inter, torch.tensor(want, dtype=F64), atol=1e-12)


def test_short_convolution_by_hand():
    u = torch.tensor([[1.0, 10.0], [2.0, 20.0], [3.0, 30.0], [4.0, 40.0]], dtype=F64)
    w = torch.tensor([[0.5, -1.0, 2.0], [1.0, 0.0, 0.1]], dtype=F64)  # the last tap meets the current token
    y = plain.short_convolution(u, w)
    assert torch.allclose(y[:, 0], torch.tensor([2.0, 3.0, 0.5 - 2 + 6, 1 - 3 + 8], dtype=F64))
    assert torch.allclose(y[:, 1], torch.tensor([1.0, 2.0, 10 + 3.0, 20 + 4.0], dtype=F64))


def test_capped_scores_and_the_sink_by_hand():
    q = torch.tensor([[[2.0]], [[3.0]]], dtype=F64)  # [T, 1 head, d = 1]
    k = torch.tensor([[[1.0]], [[-1.0]]], dtype=F64)
    v = torch.tensor([[[1.0, 0.0]], [[0.0, 1.0]]], dtype=F64)
    out = plain.softmax_attention(q, k, v, 0.5, softcap=0.8, sink=True)
    s00 = 0.8 * math.tanh(2 * 0.5 / 0.8)
    s10, s11 = 0.8 * math.tanh(3 * 0.5 / 0.8), 0.8 * math.tanh(-3 * 0.5 / 0.8)
    assert torch.allclose(out[0, 0], torch.tensor([math.exp(s00) / (1 + math.exp(s00)), 0.0], dtype=F64))
    den = 1 + math.exp(s10) + math.exp(s11)
    assert torch.allclose(out[1, 0], torch.tensor([math.exp(s10) / den, math.exp(s11) / den], dtype=F64))
    plain_out = plain.softmax_attention(q, k, v, 0.5)
    assert torch.allclose(plain_out[0, 0], torch.tensor([1.0, 0.0], dtype=F64))


def test_time_mixing_against_a_loop_over_scalars():
    g = torch.Generator().manual_seed(0)
    width, heads, d, rank, t = 6, 2, 3, 2, 5
    w = {"m." + n: torch.randn(s, generator=g, dtype=F64) * 0.5 for n, s in (
        ("r", (heads * d, width)), ("k", (heads * d, width)), ("v", (heads * d, width)), ("g", (heads * d, width)), ("w1", (rank, width)),
        ("w2", (heads * d, rank)), ("w0", (heads * d,)), ("u", (heads, d)), ("norm", (heads * d,)), ("o", (width, heads * d)))}
    for s in "rkvgw":
        w["m.mu." + s] = torch.rand(width, generator=g, dtype=F64)
    h = torch.randn(t, width, generator=g, dtype=F64)
    got = plain.time_mixing(h, w, "m", {"heads": heads, "dim": d}, 1e-5)
    S = [[[0.0] * d for _ in range(d)] for _ in range(heads)]
    rows = []
    for i in range(t):
        prev = h[i - 1] if i else torch.zeros(width, dtype=F64)
        mix = {s: h[i] + (prev - h[i]) * w["m.mu." + s] for s in "rkvgw"}
        r, k, v = (w["m." + n] @ mix[n] for n in "rkv")
        gate = w["m.g"] @ mix["g"]
        gate = gate / (1 + torch.exp(-gate))
        decay = torch.exp(-torch.exp(w["m.w2"] @ torch.tanh(w["m.w1"] @ mix["w"]) + w["m.w0"]))
        row = []
        for hd in range(heads):
            o = [sum(float(r[hd * d + a]) * (S[hd][a][b] + float(w["m.u"][hd, a]) * float(k[hd * d + a]) * float(v[hd * d + b])) for a in range(d))
                 for b in range(d)]
            for a in range(d):
                for b in range(d):
                    S[hd][a][b] = float(decay[hd * d + a]) * S[hd][a][b] + float(k[hd * d + a]) * float(v[hd * d + b])
            rms = math.sqrt(sum(x * x for x in o) / d + 1e-5)
            row += [x / rms for x in o]
        rows.append(torch.tensor(row, dtype=F64) * w["m.norm"] * gate)
    assert torch.allclose(got, torch.stack(rows) @ w["m.o"].T, atol=1e-10)


def test_routing_by_hand():
    # three experts and two identity experts; the correction changes the choice, not the weights
    w = {"p.router": torch.eye(5, dtype=F64), "p.correction": torch.tensor([0.0, 0.0, 0.5, 0.0, 0.3], dtype=F64)}
    h = torch.tensor([[2.0, 1.0, 0.0, 0.0, 0.5]], dtype=F64)
    mlp = {"router": {"experts": 3, "identity": 2, "top": 2}}
    s = torch.softmax(h[0], dim=-1)
    picked, weights = plain.route(h, w, "p", mlp)
    assert picked.tolist() == [[2, 0]] and torch.allclose(weights[0], torch.stack((s[2], s[0])))  # without the correction: 0 and 1
    for n in ("up", "down"):
        for e in range(3):
            w[f"p.e{e}.{n}"] = torch.full((4, 5) if n == "up" else (5, 4), 0.1 * (e + 1), dtype=F64)
    w["p.correction"] = torch.tensor([0.0, 0.0, 0.0, 0.0, 0.6], dtype=F64)  # expert 0 and the identity expert 4
    out = plain.routed_ff(h, w, "p", mlp)[0]
    z = 0.1 * float(h.sum())
    expert0 = torch.full((5,), 4 * 0.1 * z * z, dtype=F64)
    assert torch.allclose(out, s[0] * expert0 + s[4] * h[0])


def test_the_layers_norm_their_results_and_take_the_tokens_input():
    cfg = sh.model(7, 4, 1e-5, 2, [sh.layer(sh.attention(1, 1, 4, 4, 0.5), sh.dense(3))])
    w = {k: v.to(F64) for k, v in sh.random_tensors(cfg, 3).items()}
    toks = [3, 1, 6]
    logits, after = plain.forward(cfg, w, toks, return_layers=True)
    x = w["embed"][toks]
    x = x + plain.rms_norm(plain.attention_mixer(x, w, "l0.mix", cfg["layers"][0]["mixer"], 1e-5), w["l0.norm1"], 1e-5)
    x = x + plain.rms_norm(plain.squared_relu_ff(x, w, "l0.mlp"), w["l0.norm2"], 1e-5)
    e = w["side.embed"][toks][:, 0:2]
    y = (plain.gelu_tanh(x @ w["l0.side.gate"].T) * e) @ w["l0.side.proj"].T
    x = x + y / torch.sqrt((y * y).mean(-1, keepdim=True) + 1e-5) * w["l0.side.norm"]
    assert torch.allclose(after[0], x, atol=1e-12)
    assert torch.allclose(logits, plain.rms_norm(x, w["final.norm"], 1e-5) @ w["embed"].T, atol=1e-12)
