"""The Sevadra decoder: its ``config.json`` keys, and the plan that assembles it from parts.

A Sevadra model is a list of layers whose norms sit on the sublayers' results: ``x += norm1(mixer(x))``, ``x += norm2(ff(x))`` (RMS
norms; what a sublayer takes in is the stream as it stands; the feed-forward may be absent), and, when the config has ``token_side``, an input
from the token itself behind the feed-forward of every layer: with e the layer's ``dim`` elements of the token's row of a table,
``y = W_proj (gelu_tanh(W_gate x) * e)`` and ``x += rmsnorm(y) * w``. The head is the embedding table behind the final norm.

Three mixers (``type`` of a layer entry):

``attention``         grouped-query softmax attention; optionally a short causal convolution over time on every channel of q, k and
                      v (``conv`` taps); q and k normed over their whole projection; rotation in pairs of halves over the first
                      ``rot.dims`` elements of a head, slow pairs slowed by ``rot.scaling`` (factor, low, high, original).
``parallel``          a pair of mixers that read the same input, ``left_scale * left + right_scale * right``. Left: attention
                      without rotation, q and k normed over their whole projection, scores bounded by ``softcap * tanh(s / softcap)``,
                      a softmax whose denominator holds one more term, exp(0). Right: linear attention with a decay per token and channel and a
                      bonus for the current token, every projection reading its own blend of the token and the one before.
``latent_attention``  attention over one cached latent per token (``kv_rank`` elements) and a turned key part that all heads share
                      (``rot_dim`` elements, pairs of neighbours), a sigmoid gate per head; with ``kv_from: j`` the layer reads
                      layer j's cached latents and has no latent projection of its own.

Two feed-forwards (``mlp.kind``): ``dense``, ``down(relu(up x)^2)``; ``moe``, ``router.experts`` such feed-forwards of ``expert.ff``
of which a token uses ``router.top``: scores are the softmax over all router outputs, picked by score plus ``correction``, weighted
by the scores as they are; the last ``router.identity`` outputs are identity experts (they hand the token's input on); an optional ``shared``
expert runs for every token.

config.json keys: ``architecture``, ``vocab``, ``width``, ``norm`` (``eps``), ``token_side`` (``dim``) or absent, ``layers`` (each ``type``,
``mixer``, ``mlp`` or null). Tensor names: ``embed``, ``side.embed``, ``final.norm``, ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.*``,
``l<i>.mlp.*``, ``l<i>.side.{gate,proj,norm}``. The decay's inner size, which no key gives, is the row count of
``l<i>.mix.right.w1``. A config gives no limit on the length of a sequence; ``max_position_embeddings`` here is the engine's own bound.
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any

from ..config.registry import ArchitectureEntry, register_architecture
from ..config.specs import (
    ActivatedMlpSpec,
    AttentionSpec,
    LatentAttentionSpec,
    LayerSpec,
    ModelPlan,
    NormSpec,
    PairMixerSpec,
    RotarySpec,
    RoutedExpertsSpec,
    ScaledRotarySpec,
    TimeMixSpec,
    TokenInputSpec,
)

ARCHITECTURE = "Sevadra"
MAX_POSITIONS = 1 << 20  # no key of the config bounds a sequence; the engine's max_model_len does

ATTENTION_NAMES = (("q", "q"), ("k", "k"), ("v", "v"), ("o", "o"), ("q_norm", "q.norm"), ("k_norm", "k.norm"), ("q_conv", "q.conv"),
                   ("k_conv", "k.conv"), ("v_conv", "v.conv"))
TIME_MIX_NAMES = (("mu_r", "mu.r"), ("mu_k", "mu.k"), ("mu_v", "mu.v"), ("mu_g", "mu.g"), ("mu_w", "mu.w"), ("r", "r"), ("k", "k"), ("v", "v"),
                  ("g", "g"), ("w1", "w1"), ("w2", "w2"), ("w0", "w0"), ("u", "u"), ("norm", "norm"), ("o", "o"))
LATENT_NAMES = (("q", "q"), ("dkv", "dkv"), ("dkv_norm", "dkv.norm"), ("uk", "uk"), ("uv", "uv"), ("g", "g"), ("o", "o"))
DENSE_NAMES = (("up", "up"), ("down", "down"))
MOE_NAMES = (("router", "router"), ("expert", "e"), ("up", "up"), ("down", "down"), ("shared", "shared"), ("correction", "correction"))
MIXER_TYPES = ("attention", "parallel", "latent_attention")


def _need(d: Any, keys: tuple[str, ...], where: str) -> None:
    if not isinstance(d, dict):
        raise ValueError(f"{where} must be a dictionary")
    missing = [k for k in keys if k not in d]
    if missing:
        raise ValueError(f"{where} lacks required keys: {', '.join(missing)}")


def _check_rot(rot: Any, where: str) -> None:
    _need(rot, ("base", "dims"), where)
    if int(rot["dims"]) < 2 or int(rot["dims"]) % 2:
        raise ValueError(f"{where}: dims={rot['dims']} must be a positive even number")
    if rot.get("scaling") is not None:
        _need(rot["scaling"], ("factor", "low", "high", "original"), where + ".scaling")


def _check_layer(layers: list, i: int) -> None:
    where = f"config.json layers[{i}]"
    layer = layers[i]
    _need(layer, ("type", "mixer"), where)
    kind, m = layer["type"], layer["mixer"]
    if kind not in MIXER_TYPES:
        raise ValueError(f"{where}: unknown mixer type {kind!r}; known: {', '.join(MIXER_TYPES)}")
    if kind == "attention":
        _need(m, ("heads", "kv_heads", "dim", "vdim", "scale"), where + ".mixer")
        if int(m["heads"]) % int(m["kv_heads"]):
            raise ValueError(f"{where}: heads={m['heads']} is not a multiple of kv_heads={m['kv_heads']}")
        if m.get("rot") is not None:
            _check_rot(m["rot"], where + ".mixer.rot")
            if int(m["rot"]["dims"]) > int(m["dim"]):
                raise ValueError(f"{where}: rot.dims={m['rot']['dims']} exceeds dim={m['dim']}")
    elif kind == "parallel":
        _need(m, ("left", "right", "left_scale", "right_scale"), where + ".mixer")
        _need(m["left"], ("heads", "kv_heads", "dim", "vdim", "scale"), where + ".mixer.left")
        if int(m["left"]["heads"]) % int(m["left"]["kv_heads"]):
            raise ValueError(f"{where}: heads={m['left']['heads']} is not a multiple of kv_heads={m['left']['kv_heads']}")
        _need(m["right"], ("heads", "dim"), where + ".mixer.right")
    else:
        _need(m, ("heads", "dim", "rot_dim", "vdim", "kv_rank", "scale", "rot"), where + ".mixer")
        _need(m["rot"], ("base",), where + ".mixer.rot")
        src = m.get("kv_from")
        if src is not None:
            src = int(src)
            if not 0 <= src < i or layers[src].get("type") != "latent_attention" or layers[src]["mixer"].get("kv_from") is not None:
                raise ValueError(f"{where}: kv_from must name an earlier latent_attention layer that has a projection of its own, not {src}")
            owner = layers[src]["mixer"]
            if (int(owner["kv_rank"]), int(owner["rot_dim"])) != (int(m["kv_rank"]), int(m["rot_dim"])) or owner["rot"] != m["rot"]:
                raise ValueError(f"{where}: kv_rank, rot_dim and rot must equal those of layer {src}, whose latents it reads")
    mlp = layer.get("mlp")
    if mlp is not None:
        _need(mlp, ("kind",), where + ".mlp")
        if mlp["kind"] == "dense":
            _need(mlp, ("ff",), where + ".mlp")
        elif mlp["kind"] == "moe":
            _need(mlp, ("expert", "router"), where + ".mlp")
            _need(mlp["expert"], ("ff",), where + ".mlp.expert")
            _need(mlp["router"], ("experts", "top"), where + ".mlp.router")
            if mlp.get("shared") is not None:
                _need(mlp["shared"], ("ff",), where + ".mlp.shared")
        else:
            raise ValueError(f"{where}: unknown feed-forward kind {mlp['kind']!r}; known: dense, moe")


@dataclass(frozen=True)
class SevadraConfig:
    """The numbers of ``config.json`` that the forward pass uses. ``layers`` keeps every layer's dictionary as it is written, checked
    for the keys it needs. ``has_correction``: per layer, whether the checkpoint holds a correction of the router's scores."""

    vocab: int
    width: int
    norm_eps: float
    side_dim: int  # 0: no token input
    layers: tuple[dict, ...]
    eos_token_ids: tuple[int, ...] = ()

    @classmethod
    def from_dict(cls, cfg: dict[str, Any], eos: Any = None) -> "SevadraConfig":
        _need(cfg, ("vocab", "width", "norm", "layers"), "config.json")
        _need(cfg["norm"], ("eps",), "config.json norm")
        layers = list(cfg["layers"])
        if not layers:
            raise ValueError("config.json lists no layers")
        for i in range(len(layers)):
            _check_layer(layers, i)
        side = cfg.get("token_side")
        if side is not None:
            _need(side, ("dim",), "config.json token_side")
        if eos is None:
            eos = cfg.get("eos_token_id")
        eos_ids = () if eos is None else ((int(eos),) if isinstance(eos, int) else tuple(int(e) for e in eos))
        return cls(vocab=int(cfg["vocab"]), width=int(cfg["width"]), norm_eps=float(cfg["norm"]["eps"]),
                   side_dim=0 if side is None else int(side["dim"]), layers=tuple(layers), eos_token_ids=eos_ids)

    @classmethod
    def from_folder(cls, folder: str) -> "SevadraConfig":
        """The folder's config.json; what no key gives is read from the tensors' shapes: the inner size of a layer's decay
        (``mixer.right.decay_rank``, the rows of ``w1``) and whether a routed feed-forward has a correction of its scores
        (``mlp.router.correction``)."""
        from ..weights.safetensors_io import read_folder_header

        with open(os.path.join(folder, "config.json")) as f:
            cfg = json.load(f)
        header = read_folder_header(folder)
        layers = []
        for i, layer in enumerate(cfg.get("layers", [])):
            if isinstance(layer, dict) and isinstance(layer.get("mixer"), dict):
                entry = header.get(f"l{i}.mix.right.w1")
                if entry is not None and isinstance(layer["mixer"].get("right"), dict):
                    layer = dict(layer, mixer=dict(layer["mixer"], right=dict(layer["mixer"]["right"], decay_rank=int(entry.shape[0]))))
                mlp = layer.get("mlp")
                if isinstance(mlp, dict) and isinstance(mlp.get("router"), dict):
                    layer = dict(layer, mlp=dict(mlp, router=dict(mlp["router"], correction=f"l{i}.mlp.correction" in header)))
            layers.append(layer)
        return cls.from_dict(dict(cfg, layers=layers))

    def to_config_json(self) -> dict[str, Any]:
        """A ``config.json`` dictionary that :meth:`from_dict` reads back to an equal object."""
        out = {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
               "layers": [dict(layer) for layer in self.layers]}
        if self.side_dim:
            out["token_side"] = {"dim": self.side_dim}
        return out


def _rotary(rot: dict, dims: int, pairing: str):
    sc = rot.get("scaling")
    if sc:
        return ScaledRotarySpec(rotary_dim=dims, theta=float(rot["base"]), factor=float(sc["factor"]), low=float(sc["low"]),
                                high=float(sc["high"]), original=float(sc["original"]), pairing=pairing)
    return RotarySpec(rotary_dim=dims, theta=float(rot["base"]), pairing=pairing, angles="float64")


def _attention(cfg: SevadraConfig, m: dict, left_of_pair: bool) -> AttentionSpec:
    rot = None if left_of_pair else m.get("rot")
    return AttentionSpec(
        hidden_size=cfg.width, num_heads=int(m["heads"]), num_kv_heads=int(m["kv_heads"]), head_dim=int(m["dim"]), scale=float(m["scale"]),
        qk_norm_eps=cfg.norm_eps, window=0, position=None if rot is None else _rotary(rot, int(rot["dims"]), "halves"),
        value_dim=int(m["vdim"]), qk_norm_over="projection", conv_taps=0 if left_of_pair else int(m.get("conv") or 0),
        softcap=float(m.get("softcap") or 0.0) if left_of_pair else 0.0, unit_sink=left_of_pair, names=ATTENTION_NAMES)


def mixer_spec(cfg: SevadraConfig, layer: dict, index_of: dict[int, int]):
    kind, m = layer["type"], layer["mixer"]
    if kind == "attention":
        return _attention(cfg, m, False)
    if kind == "parallel":
        right = m["right"]
        if int(right.get("decay_rank", 0)) < 1:
            raise ValueError("the inner size of a layer's decay is the row count of its mix.right.w1; read the config from its folder, or "
                             "give mixer.right.decay_rank")
        time_mix = TimeMixSpec(hidden_size=cfg.width, num_heads=int(right["heads"]), head_dim=int(right["dim"]),
                               decay_rank=int(right["decay_rank"]), norm_eps=cfg.norm_eps, names=TIME_MIX_NAMES)
        return PairMixerSpec(left=_attention(cfg, m["left"], True), right=time_mix, left_scale=float(m["left_scale"]),
                             right_scale=float(m["right_scale"]))
    r = int(m["rot_dim"])
    src = m.get("kv_from")
    return LatentAttentionSpec(
        hidden_size=cfg.width, num_heads=int(m["heads"]), head_dim=int(m["dim"]), rotary_dim=r, value_dim=int(m["vdim"]),
        latent_rank=int(m["kv_rank"]), scale=float(m["scale"]), norm_eps=cfg.norm_eps, position=_rotary(m["rot"], r, "neighbours"),
        sink=False, output_gate=True, names=LATENT_NAMES, cache_from=None if src is None else index_of[int(src)])


def ffn_spec(cfg: SevadraConfig, mlp: dict | None):
    if mlp is None:
        return None
    if mlp["kind"] == "dense":
        return ActivatedMlpSpec(hidden_size=cfg.width, intermediate_size=int(mlp["ff"]), activation="relu2", names=DENSE_NAMES)
    r, shared = mlp["router"], mlp.get("shared")
    return RoutedExpertsSpec(
        hidden_size=cfg.width, intermediate_size=int(mlp["expert"]["ff"]), num_experts=int(r["experts"]), top_k=int(r["top"]),
        activation="relu2", gated=False, scoring="softmax_all", identity_experts=int(r.get("identity") or 0),
        score_correction=bool(r.get("correction", True)), shared_size=0 if shared is None else int(shared["ff"]), shared_gated=False,
        names=MOE_NAMES)


def plan_from_config(cfg: SevadraConfig) -> ModelPlan:
    norm = NormSpec(dim=cfg.width, eps=cfg.norm_eps)
    index_of = {i: i for i in range(len(cfg.layers))}
    layers = []
    for i, layer in enumerate(cfg.layers):
        ffn = ffn_spec(cfg, layer.get("mlp"))
        token_input = None
        if cfg.side_dim:
            token_input = TokenInputSpec(table_name="side.embed", dim=cfg.side_dim, index=i, eps=cfg.norm_eps, prefix=f"l{i}.side",
                                         activation="gelu_tanh")
        layers.append(LayerSpec(
            mixer=mixer_spec(cfg, layer, index_of), ffn=ffn, mixer_norm=norm, ffn_norm=None if ffn is None else norm,
            mixer_prefix=f"l{i}.mix", ffn_prefix=f"l{i}.mlp", mixer_norm_name=f"l{i}.norm1", ffn_norm_name=f"l{i}.norm2",
            arrangement="result_norm", token_input=token_input))
    return ModelPlan(
        architecture=ARCHITECTURE, vocab_size=cfg.vocab, hidden_size=cfg.width, layers=tuple(layers), order=tuple(range(len(layers))),
        final_norm=norm, embed_name="embed", final_norm_name="final.norm", head_name="head", tie_word_embeddings=True,
        max_position_embeddings=MAX_POSITIONS, eos_token_ids=cfg.eos_token_ids, token_table_columns=cfg.side_dim * len(layers))


register_architecture(ArchitectureEntry(
    name=ARCHITECTURE, config_from_dict=SevadraConfig.from_dict, config_from_folder=SevadraConfig.from_folder,
    plan_from_config=plan_from_config))
