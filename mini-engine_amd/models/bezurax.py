"""The Bezurax decoder: its ``config.json`` keys, and the plan that assembles it from parts.

A Bezurax model is a list of layers, each *parallel* with two norms of the same stream: ``x += mixer(norm1(x)) + ff(norm2(x))``,
with root-mean-square norms in groups; the feed-forward may be absent. The head is the embedding table, and the logits are
multiplied by ``logit_scale``. A layer entry with ``weights_of: j`` has no tensors of its own: it runs layer j's weights with a
cache and state of its own (the plan's ``order`` then names layer j again).

The mixer of a layer (type ``parallel``) is a pair of mixers that read the same input, ``left_scale * left + right_scale *
right``:

``left``   grouped-query softmax attention without rotation; q and k normed over their whole projection (weights of the
           projections' sizes); the values are the keys as projected, before the norm (there is no value projection); the
           config's score scale; a sliding window of ``mask.size`` keys beside which a query sees the mean key and value of
           every block of ``mask.pool`` positions that lies wholly before the window.
``right``  linear attention by the generalized delta rule: a decay per head and key channel ``exp(-exp(-1/2) sigmoid(W_2
           tanh(W_1 h) + w_0))``, a removal rate ``sigmoid(W_a h + b)``, every head's output over its root mean square, a weight
           over all heads, a sigmoid gate.

The feed-forward (kind ``moe``): ``router.experts`` small gated feed-forwards with the activation ``g sigmoid(1.702 g) (u + 1)``
on ``g = min(gate, limit)``, ``u = clamp(up, -limit, limit)``; a token uses the ``router.top`` with the largest sigmoid scores
among the experts of the ``groups.keep`` best of ``groups.count`` groups, weighted by their scores over their sum, times
``router.scale``; an optional ``shared`` expert of its own size and limit runs for every token, times the sigmoid of one number
per token.

config.json keys: ``architecture``, ``vocab``, ``width``, ``logit_scale``, ``norm`` (``eps``, ``groups``), ``layers`` (each ``type``,
``mixer``, ``mlp`` or null, optionally ``weights_of``). Tensor names: ``embed``, ``final.norm``, ``l<i>.norm1``, ``l<i>.norm2``,
``l<i>.mix.left.{q,k,o,q.norm,k.norm}``, ``l<i>.mix.right.{r,k,v,g,a,a.b,w1,w2,w0,norm,o}``, ``l<i>.mlp.router``,
``l<i>.mlp.e<j>.{gate,up,down}``, ``l<i>.mlp.shared.{gate,up,down,sg}``. A config gives no limit on the length of a sequence;
``max_position_embeddings`` here is the engine's own bound.
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any

from ..config.registry import ArchitectureEntry, register_architecture
from ..config.specs import AttentionSpec, DeltaRuleSpec, LayerSpec, ModelPlan, NormSpec, PairMixerSpec, RoutedExpertsSpec

ARCHITECTURE = "Bezurax"
MAX_POSITIONS = 1 << 20  # no key of the config bounds a sequence; the engine's max_model_len does

LEFT_NAMES = (("q", "q"), ("k", "k"), ("o", "o"), ("q_norm", "q.norm"), ("k_norm", "k.norm"))
RIGHT_NAMES = (("r", "r"), ("k", "k"), ("v", "v"), ("g", "g"), ("a", "a"), ("a_bias", "a.b"), ("w1", "w1"), ("w2", "w2"), ("w0", "w0"),
               ("norm", "norm"), ("o", "o"))
MOE_NAMES = (("router", "router"), ("expert", "e"), ("gate", "gate"), ("up", "up"), ("down", "down"), ("shared", "shared"),
             ("shared_gate", "sg"))


def _need(d: dict, keys: tuple[str, ...], where: str) -> None:
    missing = [k for k in keys if k not in d]
    if missing:
        raise ValueError(f"{where} lacks required keys: {', '.join(missing)}")


def owner_of(layers, i: int) -> int:
    """The layer whose tensors layer i runs: itself, or the layer that its ``weights_of`` names (followed on if that one names
    another in turn)."""
    seen = {i}
    j = i
    while isinstance(layers[j], dict) and layers[j].get("weights_of") is not None:
        j = int(layers[j]["weights_of"])
        if not 0 <= j < len(layers) or j in seen:
            raise ValueError(f"config.json layers[{i}]: weights_of must lead to a layer that has tensors of its own, not to {j}")
        seen.add(j)
    return j


def _check_layer(layer: dict, where: str) -> None:
    _need(layer, ("type", "mixer"), where)
    if layer["type"] != "parallel":
        raise ValueError(f"{where}: unknown mixer type {layer['type']!r}; known: parallel")
    m = layer["mixer"]
    _need(m, ("left", "right", "left_scale", "right_scale"), where + ".mixer")
    left, right = m["left"], m["right"]
    _need(left, ("heads", "kv_heads", "dim", "vdim", "scale", "mask"), where + ".mixer.left")
    _need(left["mask"], ("size", "pool"), where + ".mixer.left.mask")
    if int(left["heads"]) % int(left["kv_heads"]):
        raise ValueError(f"{where}: heads={left['heads']} is not a multiple of kv_heads={left['kv_heads']}")
    if int(left["vdim"]) != int(left["dim"]):
        raise ValueError(f"{where}: the values are the keys, so vdim={left['vdim']} must equal dim={left['dim']}")
    if int(left["mask"]["size"]) < 1 or int(left["mask"]["pool"]) < 1:
        raise ValueError(f"{where}: mask.size and mask.pool must be positive")
    _need(right, ("heads", "dim"), where + ".mixer.right")
    mlp = layer.get("mlp")
    if mlp is not None:
        _need(mlp, ("kind", "expert", "router"), where + ".mlp")
        if mlp["kind"] != "moe":
            raise ValueError(f"{where}: unknown feed-forward kind {mlp['kind']!r}; known: moe")
        _need(mlp["expert"], ("ff", "limit"), where + ".mlp.expert")
        _need(mlp["router"], ("experts", "top", "groups", "scale"), where + ".mlp.router")
        _need(mlp["router"]["groups"], ("count", "keep"), where + ".mlp.router.groups")
        if mlp.get("shared") is not None:
            _need(mlp["shared"], ("ff", "limit"), where + ".mlp.shared")


@dataclass(frozen=True)
class BezuraxConfig:
    """The numbers of ``config.json`` that the forward pass uses. ``layers`` keeps every layer's dictionary as it is written,
    checked for the keys it needs."""

    vocab: int
    width: int
    logit_scale: float
    norm_eps: float
    norm_groups: int
    layers: tuple[dict, ...]
    eos_token_ids: tuple[int, ...] = ()

    @classmethod
    def from_dict(cls, cfg: dict[str, Any], eos: Any = None) -> "BezuraxConfig":
        _need(cfg, ("vocab", "width", "logit_scale", "norm", "layers"), "config.json")
        _need(cfg["norm"], ("eps", "groups"), "config.json norm")
        width, groups = int(cfg["width"]), int(cfg["norm"]["groups"])
        if groups < 1 or width % groups:
            raise ValueError(f"width={width} cannot be cut into norm.groups={groups} equal parts")
        layers = list(cfg["layers"])
        if not layers:
            raise ValueError("config.json lists no layers")
        for i, layer in enumerate(layers):
            where = f"config.json layers[{i}]"
            _check_layer(layer, where)
            owner_of(layers, i)
        if eos is None:
            eos = cfg.get("eos_token_id")
        eos_ids = () if eos is None else ((int(eos),) if isinstance(eos, int) else tuple(int(e) for e in eos))
        return cls(vocab=int(cfg["vocab"]), width=width, logit_scale=float(cfg["logit_scale"]), norm_eps=float(cfg["norm"]["eps"]),
                   norm_groups=groups, layers=tuple(layers), eos_token_ids=eos_ids)

    @classmethod
    def from_folder(cls, folder: str) -> "BezuraxConfig":
        """The folder's config.json; the inner size of every layer's decay, which no key gives, is read from the shape of its
        tensor (``mixer.right.decay_rank`` of the layer's dictionary is set to it)."""
        from ..weights.safetensors_io import read_folder_header

        with open(os.path.join(folder, "config.json")) as f:
            cfg = json.load(f)
        header = read_folder_header(folder)
        layers = []
        for i, layer in enumerate(cfg.get("layers", [])):
            try:
                owner = owner_of(cfg["layers"], i)
            except (ValueError, TypeError):
                owner = i  # (from_dict says what is wrong with it)
            entry = header.get(f"l{owner}.mix.right.w1")
            if entry is not None and isinstance(layer, dict) and isinstance(layer.get("mixer"), dict) and isinstance(layer["mixer"].get("right"), dict):
                layer = dict(layer, mixer=dict(layer["mixer"], right=dict(layer["mixer"]["right"], decay_rank=int(entry.shape[0]))))
            layers.append(layer)
        return cls.from_dict(dict(cfg, layers=layers))

    def to_config_json(self) -> dict[str, Any]:
        """A ``config.json`` dictionary that :meth:`from_dict` reads back to an equal object."""
        return {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "logit_scale": self.logit_scale,
                "norm": {"eps": self.norm_eps, "groups": self.norm_groups}, "layers": [dict(layer) for layer in self.layers]}


def mixer_spec(cfg: BezuraxConfig, m: dict) -> PairMixerSpec:
    left, right = m["left"], m["right"]
    d = int(left["dim"])
    attention = AttentionSpec(
        hidden_size=cfg.width, num_heads=int(left["heads"]), num_kv_heads=int(left["kv_heads"]), head_dim=d,
        scale=float(left["scale"]), qk_norm_eps=cfg.norm_eps, window=int(left["mask"]["size"]), position=None,
        value_dim=int(left["vdim"]), qk_norm_over="projection", values_from_keys=True, pooled_block=int(left["mask"]["pool"]),
        names=LEFT_NAMES)
    # the decay's inner size is the checkpoint's (the rows of w1): the loader holds it to the tensors' shapes
    delta = DeltaRuleSpec(hidden_size=cfg.width, num_heads=int(right["heads"]), head_dim=int(right["dim"]),
                          decay_rank=int(right.get("decay_rank", 0)), norm_eps=cfg.norm_eps, names=RIGHT_NAMES)
    return PairMixerSpec(left=attention, right=delta, left_scale=float(m["left_scale"]), right_scale=float(m["right_scale"]))


def ffn_spec(cfg: BezuraxConfig, mlp: dict | None):
    if mlp is None:
        return None
    r, shared = mlp["router"], mlp.get("shared")
    return RoutedExpertsSpec(
        hidden_size=cfg.width, intermediate_size=int(mlp["expert"]["ff"]), num_experts=int(r["experts"]), top_k=int(r["top"]),
        activation="clamped_sigmoid", activation_limit=float(mlp["expert"]["limit"]), scoring="sigmoid_normalized",
        num_groups=int(r["groups"]["count"]), keep_groups=int(r["groups"]["keep"]), route_scale=float(r["scale"]),
        shared_size=0 if shared is None else int(shared["ff"]), shared_limit=0.0 if shared is None else float(shared["limit"]),
        names=MOE_NAMES)


def plan_from_config(cfg: BezuraxConfig) -> ModelPlan:
    norm = NormSpec(dim=cfg.width, eps=cfg.norm_eps, groups=cfg.norm_groups)
    owners = [i for i, layer in enumerate(cfg.layers) if layer.get("weights_of") is None]
    layers = []
    for i in owners:
        layer = cfg.layers[i]
        if int(layer["mixer"]["right"].get("decay_rank", 0)) < 1:
            raise ValueError(f"config.json layers[{i}]: the inner size of the decay is the row count of l{i}.mix.right.w1; read the "
                             f"config from its folder, or give mixer.right.decay_rank")
        ffn = ffn_spec(cfg, layer.get("mlp"))
        layers.append(LayerSpec(
            mixer=mixer_spec(cfg, layer["mixer"]), ffn=ffn, mixer_norm=norm, ffn_norm=None if ffn is None else norm,
            mixer_prefix=f"l{i}.mix", ffn_prefix=f"l{i}.mlp", mixer_norm_name=f"l{i}.norm1", ffn_norm_name=f"l{i}.norm2",
            arrangement="parallel", residual_scale=1.0))
    # a layer that runs another's weights is a second run of that layer, with a cache and state of its own
    order = tuple(owners.index(owner_of(cfg.layers, i)) for i in range(len(cfg.layers)))
    return ModelPlan(
        architecture=ARCHITECTURE, vocab_size=cfg.vocab, hidden_size=cfg.width, layers=tuple(layers), order=order, final_norm=norm,
        embed_name="embed", final_norm_name="final.norm", head_name="head", tie_word_embeddings=True,
        max_position_embeddings=MAX_POSITIONS, eos_token_ids=cfg.eos_token_ids, logit_scale=cfg.logit_scale)


register_architecture(ArchitectureEntry(
    name=ARCHITECTURE, config_from_dict=BezuraxConfig.from_dict, config_from_folder=BezuraxConfig.from_folder,
    plan_from_config=plan_from_config))
