"""Small Bezurax configurations of the tests' own, model folders with seeded random weights for them, and the plain
implementation's logits for a set of requests."""

from __future__ import annotations

import json
import os

import torch

import plain_bezurax as plain


def left(heads, kv_heads, dim, scale, window, pool):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale, "mask": {"size": window, "pool": pool}}


def right(heads, dim, decay_rank):
    return {"heads": heads, "dim": dim, "decay_rank": decay_rank}


def moe(experts, top, ff, limit, count, keep, scale, shared=None):
    out = {"kind": "moe", "expert": {"ff": ff, "limit": limit},
           "router": {"experts": experts, "top": top, "groups": {"count": count, "keep": keep}, "scale": scale}}
    if shared is not None:
        out["shared"] = {"ff": shared[0], "limit": shared[1]}
    return out


def layer(lft, rgt, left_scale, right_scale, mlp=None, weights_of=None):
    out = {"type": "parallel", "mixer": {"left": lft, "right": rgt, "left_scale": left_scale, "right_scale": right_scale}, "mlp": mlp}
    if weights_of is not None:
        out["weights_of"] = weights_of
    return out


def model(vocab, width, eps, groups, logit_scale, layers):
    return {"architecture": "Bezurax", "vocab": vocab, "width": width, "logit_scale": logit_scale, "norm": {"eps": eps, "groups": groups},
            "layers": layers}


def configs() -> dict[str, dict]:
    """Sizes, orders and constants that differ from one another in everything: one norm group and several; as many key/value
    heads as heads, and one; windows shorter than a page and longer than most prompts; pooled blocks of one key, of a page, of
    sizes that divide no page; groups of one expert, one group of all; every expert picked; layers without a feed-forward,
    without a shared expert, and layers that run an earlier or a later layer's weights; head sizes that are no multiple of 8."""
    a0 = layer(left(4, 2, 24, 0.2, 40, 5), right(2, 16, 8), 0.7, 1.2, moe(6, 2, 40, 1.2, 3, 2, 1.5, shared=(24, 0.8)))
    a1 = layer(left(2, 1, 32, 0.15, 17, 3), right(3, 24, 12), 1.1, 0.6, moe(4, 3, 32, 2.0, 1, 1, 1.0))
    b0 = layer(left(6, 6, 20, 0.22, 64, 16), right(1, 40, 20), 1.0, 1.0, moe(8, 1, 48, 0.9, 8, 3, 2.5, shared=(72, 1.5)))
    b1 = layer(left(3, 1, 16, 0.3, 9, 1), right(4, 12, 4), 0.5, 1.5)
    c0 = layer(left(5, 1, 12, 0.3, 33, 7), right(2, 28, 16), 0.9, 0.9, moe(4, 4, 24, 1.0, 2, 2, 1.0, shared=(8, 3.0)))
    e0 = layer(left(6, 2, 96, 0.1, 48, 10), right(3, 32, 16), 0.9, 1.1, moe(8, 3, 48, 1.4, 4, 2, 2.0, shared=(40, 1.1)))
    e1 = layer(left(4, 4, 32, 0.18, 20, 4), right(2, 48, 8), 1.2, 0.7, moe(6, 2, 32, 2.5, 2, 2, 1.0))
    d0 = layer(left(2, 2, 64, 0.125, 128, 32), right(2, 64, 32), 1.0, 0.8, moe(6, 2, 64, 1.5, 2, 1, 2.0, shared=(64, 1.0)))
    return {
        "A": model(300, 96, 1e-5, 3, 0.5, [a0, a1, dict(a0, weights_of=0)]),
        "B": model(500, 128, 1e-6, 1, 1.0, [b0, b1, dict(b1, weights_of=1), dict(b0, weights_of=0)]),
        # sizes that are no multiple of 8 (a width of 100, a feed-forward of 24, heads of 12 and 28)
        "C": model(131, 100, 1e-6, 5, 0.25, [c0, dict(c0, weights_of=0)]),
        # heads of 64 under a window of 128 keys and pooled blocks of two pages
        "D": model(260, 128, 1e-5, 2, 0.3, [d0, d0]),
        # heads of 96 and 32, three to a key/value head, blocks of 10 under a window of 48 (neither divides a page), a later
        # layer's weights run first
        "E": model(400, 192, 1e-6, 4, 0.4, [dict(e0, weights_of=1), e0, e1]),
    }


BLOCK_SIZES = {"A": 16, "B": 32, "C": 8, "D": 16, "E": 16}


def wants_of(cfg: dict):
    from mini_engine_amd.models.bezurax import BezuraxConfig, plan_from_config
    from mini_engine_amd.parts.decoder import Decoder

    typed = BezuraxConfig.from_dict(cfg)
    return typed, Decoder(plan_from_config(typed), torch.float32, "cpu").weight_wants()


def random_tensors(cfg: dict, seed: int, std: float = 0.08) -> dict[str, torch.Tensor]:
    """bfloat16 tensors by name: matrices from N(0, std); norm weights around one; biases from N(0, 1); router rows wide apart,
    so that few picks are close calls."""
    _, wants = wants_of(cfg)
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, want in wants.items():
        x = torch.randn(want.shape, generator=g)
        if name.endswith("norm") or ".norm" in name:
            t = 1.0 + 0.2 * x
        elif name.endswith((".a.b", ".w0")):
            t = x
        elif name.endswith((".router", ".sg")):
            t = 0.15 * x
        elif name.endswith(".w2"):
            t = 0.5 * x
        else:
            t = std * x
        out[name] = t.to(torch.bfloat16)
    return out


def write_folder(folder: str, cfg: dict, seed: int = 0, tensors: dict | None = None) -> str:
    from mini_engine_amd.weights.safetensors_io import write_file

    typed, _ = wants_of(cfg)
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(typed.to_config_json(), f, indent=1)
    write_file(os.path.join(folder, "model.safetensors"), tensors if tensors is not None else random_tensors(cfg, seed), {"format": "pt"})
    return folder


def read_weights(folder: str) -> dict[str, torch.Tensor]:
    from safetensors.torch import load_file

    return {k: v.to(torch.float64) for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}


def rows_that_bear_rounding(cfg: dict, weights: dict, tokens: list[int], share: float = 0.015) -> torch.Tensor:
    """A mask of the positions whose plain logits move by less than ``share`` of the row's largest when every part's normed
    input is rounded to bfloat16: where random weights make a row ill-conditioned, a bfloat16 engine and the plain
    implementation differ by what the model does to any rounding, not by a fault."""
    exact = plain.forward(cfg, weights, tokens)
    rounded = plain.forward(cfg, weights, tokens, after_norm=lambda z: z.to(torch.bfloat16).to(torch.float64))
    return (exact - rounded).abs().amax(-1) < share * exact.abs().amax(-1)


def rows_before_a_close_call(cfg: dict, weights: dict, tokens: list[int], gap: float = 0.004) -> int:
    """How many leading positions of a sequence no router decides by less than ``gap`` (of scores between 0 and 1): up to there
    a rounding of the activations cannot change which experts a token uses (nor, through the state and the keys that the token
    leaves, what later tokens read)."""
    gaps: list = []
    plain.forward(cfg, weights, tokens, router_gaps=gaps)
    if not gaps:
        return len(tokens)
    close = (torch.stack(gaps).amin(dim=0) < gap).nonzero()
    return int(close[0]) if close.numel() else len(tokens)


def plain_logits(cfg: dict, weights: dict, requests: dict[str, list[int]]) -> dict[str, torch.Tensor]:
    return {rid: plain.forward(cfg, weights, toks).to(torch.float32) for rid, toks in requests.items()}
