"""Small Sevadra configurations of the tests' own, model folders with seeded random weights for them, and the plain
implementation's logits for a set of requests."""

from __future__ import annotations

import json
import os

import torch

import plain_sevadra as plain


def rot(base, dims, scaling=None):
    out = {"base": base, "dims": dims}
    if scaling is not None:
        out["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return out


def attention(heads, kv_heads, dim, vdim, scale, rot=None, conv=0):
    out = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if rot is not None:
        out["rot"] = rot
    if conv:
        out["conv"] = conv
    return {"type": "attention", "mixer": out}


def parallel(left, right, left_scale, right_scale):
    """left: (heads, kv_heads, dim, vdim, scale, softcap); right: (heads, dim, decay_rank)."""
    lft = dict(zip(("heads", "kv_heads", "dim", "vdim", "scale", "softcap"), left))
    rgt = dict(zip(("heads", "dim", "decay_rank"), right))
    return {"type": "parallel", "mixer": {"left": lft, "right": rgt, "left_scale": left_scale, "right_scale": right_scale}}


def latent(heads, dim, rot_dim, vdim, rank, scale, base, kv_from=None):
    out = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "scale": scale, "rot": {"base": base, "dims": rot_dim}}
    if kv_from is not None:
        out["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": out}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, identity, top, ff, shared=None):
    out = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "identity": identity, "top": top}}
    if shared is not None:
        out["shared"] = {"ff": shared}
    return out


def layer(mixer: dict, mlp=None) -> dict:
    return dict(mixer, mlp=mlp)


def model(vocab, width, eps, side, layers):
    out = {"architecture": "Sevadra", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if side:
        out["token_side"] = {"dim": side}
    return out


def configs() -> dict[str, dict]:
    """Sizes, orders and constants that differ from one another in everything: every mixer first and last; layers without a
    feed-forward; as many key/value heads as heads, and one; value heads larger and smaller than the keys'; rotation over a part of
    a head and over all of it, with and without slowed pairs (a scaling that leaves pairs in each of its three ranges);
    convolutions of two taps and of more taps than a short portion has tokens, and none; routers without identity experts, with
    more identity experts than experts, picking one and picking all; with and without a shared expert; a token input of one
    element and none; sizes that are no multiple of 8; one head."""
    a = model(300, 96, 1e-5, 8, [
        layer(latent(4, 16, 8, 24, 32, 0.2, 10000.0), dense(160)),
        layer(parallel((4, 2, 24, 16, 0.25, 3.0), (2, 16, 8), 0.7, 1.2), moe(6, 2, 2, 40, shared=24)),
        layer(attention(4, 2, 24, 32, 0.3, rot(10000.0, 16, (4.0, 1.0, 4.0, 64)), conv=3), moe(5, 0, 3, 32)),
        layer(latent(2, 24, 8, 16, 32, 0.18, 10000.0, kv_from=0)),
        layer(attention(6, 6, 16, 16, 0.35, rot(500.0, 16)), dense(64)),
    ])
    b = model(131, 100, 1e-6, 0, [
        layer(attention(5, 1, 12, 20, 0.4, rot(100.0, 12, (8.0, 2.0, 3.0, 40)), conv=2), moe(3, 4, 2, 24, shared=12)),
        layer(parallel((3, 3, 28, 28, 0.2, 1.5), (5, 12, 4), 1.1, 0.6)),
        layer(latent(3, 12, 4, 20, 20, 0.3, 50.0), moe(4, 0, 4, 20)),
    ])
    c = model(64, 32, 1e-5, 1, [
        layer(parallel((1, 1, 32, 8, 0.2, 50.0), (1, 32, 1), 1.0, 1.0), moe(2, 1, 1, 16)),
        layer(attention(1, 1, 32, 32, 0.2, rot(10000.0, 32), conv=6), dense(8)),
        layer(latent(1, 8, 2, 8, 8, 0.35, 10000.0), None),
        layer(latent(1, 16, 2, 4, 8, 0.3, 10000.0, kv_from=2), moe(1, 1, 2, 8, shared=8)),
    ])
    # heads of 64 and 128, a cached latent of 128 elements: sizes that the matrix-core kernels take
    d = model(260, 256, 1e-5, 16, [
        layer(attention(4, 2, 64, 64, 0.125, rot(10000.0, 64, (4.0, 1.0, 4.0, 256))), moe(8, 2, 2, 64, shared=64)),
        layer(latent(8, 32, 32, 48, 96, 0.12, 500000.0), dense(512)),
        layer(parallel((2, 1, 128, 128, 0.09, 30.0), (4, 64, 16), 0.8, 0.9), moe(4, 0, 2, 128)),
        layer(latent(4, 64, 32, 32, 96, 0.1, 500000.0, kv_from=1), dense(256)),
    ])
    return {"A": a, "B": b, "C": c, "D": d}


BLOCK_SIZES = {"A": 16, "B": 8, "C": 16, "D": 32}


def with_decay_ranks(cfg: dict) -> dict:
    """``cfg`` as its config.json is written: without the decay's inner size (the checkpoint's shapes give it)."""
    out = json.loads(json.dumps(cfg))
    for lay in out["layers"]:
        if lay["type"] == "parallel":
            lay["mixer"]["right"].pop("decay_rank", None)
    return out


def wants_of(cfg: dict):
    from mini_engine_amd.models.sevadra import SevadraConfig, plan_from_config
    from mini_engine_amd.parts.decoder import Decoder

    typed = SevadraConfig.from_dict(cfg)
    return typed, Decoder(plan_from_config(typed), torch.float32, "cpu").weight_wants()


def random_tensors(cfg: dict, seed: int, std: float = 0.08) -> dict[str, torch.Tensor]:
    """bfloat16 tensors by name: matrices from N(0, std); norm weights around one; the blends' mu in 0..1; decay biases around -1;
    router rows and corrections wide enough apart that few picks are close calls."""
    _, wants = wants_of(cfg)
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, want in wants.items():
        x = torch.randn(want.shape, generator=g)
        if name.endswith("norm"):
            t = 1.0 + 0.2 * x
        elif ".mu." in name:
            t = torch.rand(want.shape, generator=g)
        elif name.endswith(".w0"):
            t = -1.0 + x
        elif name.endswith(".u"):
            t = 0.5 * x
        elif name.endswith(".w2"):
            t = 0.5 * x
        elif name.endswith(".router"):
            t = 1.0 * x
        elif name.endswith(".correction"):
            t = 0.1 * x
        elif name.endswith(".conv"):
            t = 0.5 * x
        elif name in ("embed", "side.embed"):
            t = x
        else:
            t = std * x
        out[name] = t.to(torch.bfloat16)
    return out


def write_folder(folder: str, cfg: dict, seed: int = 0, tensors: dict | None = None) -> str:
    from mini_engine_amd.weights.safetensors_io import write_file

    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(with_decay_ranks(cfg), f, indent=1)
    write_file(os.path.join(folder, "model.safetensors"), tensors if tensors is not None else random_tensors(cfg, seed), {"format": "pt"})
    return folder


def read_weights(folder: str) -> dict[str, torch.Tensor]:
    from safetensors.torch import load_file

    return {k: v.to(torch.float64) for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}


def rows_before_a_close_call(cfg: dict, weights: dict, tokens: list[int], gap: float = 0.004) -> int:
    """How many leading positions of a sequence no router decides by less than ``gap`` (of scores between 0 and 1): up to there a
    rounding of the activations cannot change which experts a token uses (nor, through the state and the keys that the token
    leaves, what later tokens read)."""
    gaps: list = []
    plain.forward(cfg, weights, tokens, router_gaps=gaps)
    if not gaps:
        return len(tokens)
    close = (torch.stack(gaps).amin(dim=0) < gap).nonzero()
    return int(close[0]) if close.numel() else len(tokens)


def rows_that_bear_rounding(cfg: dict, weights: dict, tokens: list[int], share: float = 0.01) -> torch.Tensor:
    """A mask of the positions whose plain logits move by less than ``share`` of the row's largest when the stream is rounded to
    bfloat16 wherever a sublayer reads it: where random weights make a row ill-conditioned, a bfloat16 engine and the plain
    implementation differ by what the model does to any rounding, not by a fault."""
    exact = plain.forward(cfg, weights, tokens)
    rounded = plain.forward(cfg, weights, tokens, reads=lambda z: z.to(torch.bfloat16).to(torch.float64))
    return (exact - rounded).abs().amax(-1) < share * exact.abs().amax(-1)


def plain_logits(cfg: dict, weights: dict, requests: dict[str, list[int]]) -> dict[str, torch.Tensor]:
    return {rid: plain.forward(cfg, weights, toks).to(torch.float32) for rid, toks in requests.items()}


def requests_for(cfg: dict, lengths: dict[str, int], seed: int = 0) -> dict[str, list[int]]:
    g = torch.Generator().manual_seed(seed)
    return {rid: torch.randint(0, int(cfg["vocab"]), (n,), generator=g).tolist() for rid, n in lengths.items()}
