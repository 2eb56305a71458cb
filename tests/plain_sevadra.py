"""A plain, slow implementation of the Sevadra design in double precision: one function per mechanism, whole sequences at
once, no cache and no batching. It shares no code with the package; the tests hold the engine against it.

``w`` maps tensor names to tensors; ``cfg`` is the dictionary of ``config.json``. A layer is ``x += norm1(mixer(x))``, ``x +=
norm2(ff(x))`` (the norm on the sublayer's result; what a sublayer takes in is the stream as it stands), then a per-layer token input.
"""

from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms_norm(x, weight, eps: float):
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rotary_frequencies(rot: dict):
    """The turning rate of every pair: ``base^(-2i/dims)``, slowed where ``rot.scaling`` says so: wavelengths beyond
    ``original/low`` by ``factor``, those below ``original/high`` not at all, and a straight blend in between."""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F64)
    sc = rot.get("scaling")
    if sc:
        factor, low, high, original = float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"])
        out = []
        for fi in f.tolist():
            wavelength = 2.0 * math.pi / fi
            if wavelength < original / high:
                out.append(fi)
            elif wavelength > original / low:
                out.append(fi / factor)
            else:
                s = (original / wavelength - low) / (high - low)
                out.append((1.0 - s) * fi / factor + s * fi)
        f = torch.tensor(out, dtype=F64)
    return f


def rotate(x, positions, rot: dict, layout: str):
    """x [T, heads, d]: the first ``rot.dims`` elements of every head turned by the position; ``layout`` "halves" pairs i with
    i + dims/2, "interleaved" pairs 2i with 2i + 1."""
    dims = int(rot["dims"])
    a = positions.to(F64).unsqueeze(1) * rotary_frequencies(rot).unsqueeze(0)  # [T, dims/2]
    cos, sin = torch.cos(a).unsqueeze(1), torch.sin(a).unsqueeze(1)
    out = x.clone()
    if layout == "halves":
        u, v = x[..., : dims // 2], x[..., dims // 2: dims]
        out[..., : dims // 2] = u * cos - v * sin
        out[..., dims // 2: dims] = v * cos + u * sin
    else:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = u * cos - v * sin
        out[..., 1:dims:2] = v * cos + u * sin
    return out


def short_convolution(u, taps_weight):
    """u [T, C], taps_weight [C, taps]: ``y_t = sum_j w[:, j] * u_(t - taps + 1 + j)`` with zeros before the first token."""
    t, c = u.shape
    taps = taps_weight.shape[1]
    padded = torch.cat((torch.zeros(taps - 1, c, dtype=u.dtype), u), dim=0)
    y = torch.zeros_like(u)
    for j in range(taps):
        y = y + padded[j: j + t] * taps_weight[:, j]
    return y


def softmax_attention(q, k, v, scale: float, softcap: float = 0.0, sink: bool = False):
    """q [T, H, d], k [T, G, d], v [T, G, dv] -> [T, H, dv]; causal; query head h reads key/value head h // (H/G). ``softcap``
    bounds the scores through a tanh; ``sink`` adds one to the softmax's denominator."""
    t, heads, _ = q.shape
    per = heads // k.shape[1]
    causal = torch.ones(t, t, dtype=torch.bool).tril()
    out = torch.zeros(t, heads, v.shape[2], dtype=q.dtype)
    for h in range(heads):
        g = h // per
        s = (q[:, h] @ k[:, g].T) * scale
        if softcap:
            s = softcap * torch.tanh(s / softcap)
        s = s.masked_fill(~causal, -math.inf)
        m = s.max(dim=1, keepdim=True).values
        if sink:
            m = torch.clamp(m, min=0.0)
        e = torch.exp(s - m)
        denom = e.sum(dim=1, keepdim=True) + (torch.exp(-m) if sink else 0.0)
        out[:, h] = (e / denom) @ v[:, g]
    return out


def attention_mixer(h, w, p: str, m: dict, eps: float):
    """Grouped-query attention: optional short convolutions on q, k and v, q and k normed over their whole projection, rotation
    in halves, plain softmax."""
    t = h.shape[0]
    heads, kv, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q, k, v = h @ w[p + ".q"].T, h @ w[p + ".k"].T, h @ w[p + ".v"].T
    if m.get("conv"):
        q, k, v = (short_convolution(u, w[p + f".{n}.conv"]) for u, n in ((q, "q"), (k, "k"), (v, "v")))
    q = rms_norm(q, w[p + ".q.norm"], eps).reshape(t, heads, d)
    k = rms_norm(k, w[p + ".k.norm"], eps).reshape(t, kv, d)
    pos = torch.arange(t)
    if m.get("rot"):
        q, k = rotate(q, pos, m["rot"], "halves"), rotate(k, pos, m["rot"], "halves")
    o = softmax_attention(q, k, v.reshape(t, kv, dv), float(m["scale"]))
    return o.reshape(t, heads * dv) @ w[p + ".o"].T


def capped_sink_attention(h, w, p: str, m: dict, eps: float):
    """The left mixer of a pair: no rotation, scores bounded by ``softcap``, a softmax whose denominator holds one more term, exp(0)."""
    t = h.shape[0]
    heads, kv, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = rms_norm(h @ w[p + ".q"].T, w[p + ".q.norm"], eps).reshape(t, heads, d)
    k = rms_norm(h @ w[p + ".k"].T, w[p + ".k.norm"], eps).reshape(t, kv, d)
    v = (h @ w[p + ".v"].T).reshape(t, kv, dv)
    o = softmax_attention(q, k, v, float(m["scale"]), softcap=float(m.get("softcap") or 0.0), sink=True)
    return o.reshape(t, heads * dv) @ w[p + ".o"].T


def time_mixing(h, w, p: str, m: dict, eps: float):
    """The right mixer of a pair: each of r, k, v, g, w reads its own blend of the token and the one before it; a decay per head
    and key channel; the current token counts with a bonus u and enters the state afterwards."""
    t = h.shape[0]
    heads, d = int(m["heads"]), int(m["dim"])
    prev = torch.cat((torch.zeros(1, h.shape[1], dtype=h.dtype), h[:-1]), dim=0)
    mix = {s: h + (prev - h) * w[p + f".mu.{s}"] for s in ("r", "k", "v", "g", "w")}
    r = (mix["r"] @ w[p + ".r"].T).reshape(t, heads, d)
    k = (mix["k"] @ w[p + ".k"].T).reshape(t, heads, d)
    v = (mix["v"] @ w[p + ".v"].T).reshape(t, heads, d)
    gate = torch.nn.functional.silu(mix["g"] @ w[p + ".g"].T)
    decay = torch.exp(-torch.exp(torch.tanh(mix["w"] @ w[p + ".w1"].T) @ w[p + ".w2"].T + w[p + ".w0"])).reshape(t, heads, d)
    u = w[p + ".u"].reshape(heads, d)
    state = torch.zeros(heads, d, d, dtype=h.dtype)
    out = torch.zeros(t, heads, d, dtype=h.dtype)
    for i in range(t):
        kv = k[i].unsqueeze(2) * v[i].unsqueeze(1)  # [heads, d(key), d(value)]
        out[i] = torch.einsum("hkv,hk->hv", state + u.unsqueeze(2) * kv, r[i])
        state = decay[i].unsqueeze(2) * state + kv
    out = rms_norm(out, None, eps).reshape(t, heads * d) * w[p + ".norm"] * gate
    return out @ w[p + ".o"].T


def latent_projection(h, w, p: str, m: dict, eps: float):
    """(c [T, rank], shared rotated key part [T, r]) of a latent attention layer that has a projection of its own."""
    rank, r = int(m["kv_rank"]), int(m["rot_dim"])
    t = h.shape[0]
    dkv = h @ w[p + ".dkv"].T
    c = rms_norm(dkv[:, :rank], w[p + ".dkv.norm"], eps)
    rot = dict(m["rot"], dims=r)
    kr = rotate(dkv[:, rank:].reshape(t, 1, r), torch.arange(t), rot, "interleaved").reshape(t, r)
    return c, kr


def latent_attention(h, w, p: str, m: dict, latent, eps: float):
    """Attention whose keys and values are maps of the latent c; ``latent`` is (c, shared key part) of this layer or of the
    layer it names. Every head's result times the sigmoid of a gate."""
    t = h.shape[0]
    heads, d, r, dv, rank = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
    c, kr = latent
    q = (h @ w[p + ".q"].T).reshape(t, heads, d + r)
    rot = dict(m["rot"], dims=r)
    q_rot = rotate(q[..., d:], torch.arange(t), rot, "interleaved")
    k_plain = (c @ w[p + ".uk"].T).reshape(t, heads, d)
    value = (c @ w[p + ".uv"].T).reshape(t, heads, dv)
    qq = torch.cat((q[..., :d], q_rot), dim=2)
    kk = torch.cat((k_plain, kr.unsqueeze(1).expand(t, heads, r)), dim=2)
    o = softmax_attention(qq, kk, value, float(m["scale"]))
    gate = torch.sigmoid(h @ w[p + ".g"].T)  # [T, heads]
    o = o * gate.unsqueeze(2)
    return o.reshape(t, heads * dv) @ w[p + ".o"].T


def squared_relu_ff(h, w, p: str):
    z = torch.relu(h @ w[p + ".up"].T)
    return (z * z) @ w[p + ".down"].T


def route(h, w, p: str, mlp: dict, gaps: list | None = None):
    """(picked [T, top] expert indices, weights [T, top]): softmax over all router outputs, the choice by score plus correction,
    the weights the scores themselves. ``gaps`` collects, per token, how far the last pick's choice score lies above the best
    score that was not picked (infinite where everything is picked)."""
    top = int(mlp["router"]["top"])
    s = torch.softmax(h @ w[p + ".router"].T, dim=-1)
    choice = s + w[p + ".correction"] if (p + ".correction") in w else s
    ranked = torch.sort(choice, dim=-1, descending=True)
    picked = ranked.indices[:, :top]
    if gaps is not None:
        gaps.append(ranked.values[:, top - 1] - ranked.values[:, top] if choice.shape[1] > top
                    else torch.full((h.shape[0],), math.inf, dtype=h.dtype))
    return picked, torch.gather(s, 1, picked)


def routed_ff(h, w, p: str, mlp: dict, gaps: list | None = None):
    experts = int(mlp["router"]["experts"])
    picked, weights = route(h, w, p, mlp, gaps)
    out = torch.zeros_like(h)
    for i in range(h.shape[0]):
        for e, wt in zip(picked[i].tolist(), weights[i]):
            if e < experts:
                out[i] += wt * squared_relu_ff(h[i: i + 1], w, f"{p}.e{e}")[0]
            else:  # an identity expert: the input itself
                out[i] += wt * h[i]
    if mlp.get("shared"):
        out = out + squared_relu_ff(h, w, p + ".shared")
    return out


def token_side_input(x, tokens, w, cfg: dict, i: int, eps: float):
    dim = int(cfg["token_side"]["dim"])
    e = w["side.embed"][tokens][:, i * dim: (i + 1) * dim]
    g = gelu_tanh(x @ w[f"l{i}.side.gate"].T) * e
    y = g @ w[f"l{i}.side.proj"].T
    return rms_norm(y, w[f"l{i}.side.norm"], eps)


def forward(cfg: dict, weights: dict, tokens, return_layers: bool = False, router_gaps: list | None = None, reads=None):
    """Logits [T, vocab] of one sequence (float64); with ``return_layers`` also the stream after every layer. ``router_gaps``
    collects what :func:`route` says of every routed layer. ``reads`` (a function of the stream, or None) stands between the
    stream and every sublayer that reads it: what a rounding there does to the logits says how well a row bears roundings."""
    reads = reads or (lambda z: z)
    w = {k: (v.to(F64) if v.is_floating_point() else v) for k, v in weights.items()}
    eps = float(cfg["norm"]["eps"])
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    x = w["embed"][tokens]
    latents: dict[int, tuple] = {}
    after = []
    for i, layer in enumerate(cfg["layers"]):
        m, kind, p = layer["mixer"], layer["type"], f"l{i}.mix"
        h = reads(x)
        if kind == "attention":
            y = attention_mixer(h, w, p, m, eps)
        elif kind == "parallel":
            y = float(m["left_scale"]) * capped_sink_attention(h, w, p + ".left", m["left"], eps) \
                + float(m["right_scale"]) * time_mixing(h, w, p + ".right", m["right"], eps)
        elif kind == "latent_attention":
            src = m.get("kv_from")
            if src is None:
                latents[i] = latent_projection(h, w, p, m, eps)
                src = i
            y = latent_attention(h, w, p, m, latents[int(src)], eps)
        else:
            raise ValueError(kind)
        x = x + rms_norm(y, w[f"l{i}.norm1"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            h = reads(x)
            y = squared_relu_ff(h, w, f"l{i}.mlp") if mlp["kind"] == "dense" else routed_ff(h, w, f"l{i}.mlp", mlp, router_gaps)
            x = x + rms_norm(y, w[f"l{i}.norm2"], eps)
        if cfg.get("token_side"):
            x = x + token_side_input(reads(x), tokens, w, cfg, i, eps)
        after.append(x.clone())
    logits = rms_norm(x, w["final.norm"], eps) @ w["embed"].T
    return (logits, after) if return_layers else logits
