"""A plain, slow implementation of the Bezurax design in double precision: one function per mechanism, whole sequences at
once, no cache and no batching. It shares no code with the package; the tests hold the engine against it.

``weights`` maps tensor names to tensors; ``cfg`` is the dictionary of ``config.json``.
"""

from __future__ import annotations

import math

import torch

F64 = torch.float64


def group_rms_norm(x, w, groups: int, eps: float):
    """x [T, n] cut into ``groups`` equal consecutive parts, each over its own root mean square; the whole times w."""
    t, n = x.shape
    parts = x.reshape(t, groups, n // groups)
    parts = parts / torch.sqrt((parts * parts).mean(dim=-1, keepdim=True) + eps)
    return parts.reshape(t, n) * w


def pooled_window_visibility(num_tokens: int, window: int, pool: int):
    """(tokens [T, T] bool, blocks [T, B] bool): query i sees token j with 0 <= i - j < window and block b (the positions
    b pool .. b pool + pool - 1) when its last position is at most i - window."""
    i = torch.arange(num_tokens).unsqueeze(1)
    j = torch.arange(num_tokens).unsqueeze(0)
    tokens = (i - j >= 0) & (i - j < window)
    num_blocks = num_tokens // pool
    b = torch.arange(num_blocks).unsqueeze(0)
    blocks = (b * pool + pool - 1) <= (i - window)
    return tokens, blocks


def pooled_window_attention(h, w, prefix: str, m: dict, eps: float):
    """Grouped-query softmax attention without rotation whose values are the keys as projected; q and k normed over their
    whole projection; a sliding window beside the means of whole blocks of keys and values that lie before it."""
    heads, kv_heads, d = int(m["heads"]), int(m["kv_heads"]), int(m["dim"])
    window, pool, scale = int(m["mask"]["size"]), int(m["mask"]["pool"]), float(m["scale"])
    t = h.shape[0]
    q = h @ w[prefix + ".q"].T
    k_raw = h @ w[prefix + ".k"].T
    q = q / torch.sqrt((q * q).mean(dim=-1, keepdim=True) + eps) * w[prefix + ".q.norm"]
    k = k_raw / torch.sqrt((k_raw * k_raw).mean(dim=-1, keepdim=True) + eps) * w[prefix + ".k.norm"]
    q = q.reshape(t, heads, d)
    k = k.reshape(t, kv_heads, d)
    v = k_raw.reshape(t, kv_heads, d)
    nb = t // pool
    kb = k[: nb * pool].reshape(nb, pool, kv_heads, d).mean(dim=1)
    vb = v[: nb * pool].reshape(nb, pool, kv_heads, d).mean(dim=1)
    see_tokens, see_blocks = pooled_window_visibility(t, window, pool)
    out = torch.zeros(t, heads, d, dtype=h.dtype)
    per = heads // kv_heads
    for hd in range(heads):
        g = hd // per
        s_tok = (q[:, hd] @ k[:, g].T) * scale
        s_blk = (q[:, hd] @ kb[:, g].T) * scale
        s = torch.cat((s_blk.masked_fill(~see_blocks, -math.inf), s_tok.masked_fill(~see_tokens, -math.inf)), dim=1)
        p = torch.softmax(s, dim=1)
        out[:, hd] = p[:, :nb] @ vb[:, g] + p[:, nb:] @ v[:, g]
    return out.reshape(t, heads * d) @ w[prefix + ".o"].T


def delta_rule(h, w, prefix: str, m: dict, eps: float, state=None):
    """Generalized delta rule per head: S_t = diag(w_t) S_(t-1) - (a_t u_t)(u_t^T S_(t-1)) + k_t v_t^T, o_t = S_t^T r_t, u the unit
    key; heads' outputs over their root mean square, a weight, a sigmoid gate, the output projection. Returns (result, S)."""
    heads, d = int(m["heads"]), int(m["dim"])
    t = h.shape[0]
    r = (h @ w[prefix + ".r"].T).reshape(t, heads, d)
    k = (h @ w[prefix + ".k"].T).reshape(t, heads, d)
    v = (h @ w[prefix + ".v"].T).reshape(t, heads, d)
    lora = torch.tanh(h @ w[prefix + ".w1"].T) @ w[prefix + ".w2"].T + w[prefix + ".w0"]
    decay = torch.exp(-math.exp(-0.5) * torch.sigmoid(lora)).reshape(t, heads, d)
    a = torch.sigmoid(h @ w[prefix + ".a"].T + w[prefix + ".a.b"]).reshape(t, heads, d)
    u = k / torch.sqrt((k * k).sum(dim=-1, keepdim=True) + 1e-6)
    S = torch.zeros(heads, d, d, dtype=h.dtype) if state is None else state.clone()
    o = torch.zeros(t, heads, d, dtype=h.dtype)
    for i in range(t):
        for hd in range(heads):
            old = S[hd]
            sa = u[i, hd] @ old  # [d] over the value channels
            S[hd] = decay[i, hd].unsqueeze(1) * old - torch.outer(a[i, hd] * u[i, hd], sa) + torch.outer(k[i, hd], v[i, hd])
            o[i, hd] = S[hd].T @ r[i, hd]
    o = o / torch.sqrt((o * o).mean(dim=-1, keepdim=True) + eps)
    o = o.reshape(t, heads * d) * w[prefix + ".norm"] * torch.sigmoid(h @ w[prefix + ".g"].T)
    return o @ w[prefix + ".o"].T, S


def pair_mixer(h, w, prefix: str, m: dict, eps: float):
    left = pooled_window_attention(h, w, prefix + ".left", m["left"], eps)
    right, _ = delta_rule(h, w, prefix + ".right", m["right"], eps)
    return float(m["left_scale"]) * left + float(m["right_scale"]) * right


def clamped_expert(h, w, prefix: str, limit: float):
    g = torch.clamp(h @ w[prefix + ".gate"].T, max=limit)
    u = torch.clamp(h @ w[prefix + ".up"].T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[prefix + ".down"].T


def route(z, r: dict, gaps: list | None = None):
    """Router logits z [T, E] -> (picked experts [T, top], their weights [T, top]). ``gaps`` collects, per token, how far the
    closest decision was from going the other way (between the last group kept and the next, the last pick and the next)."""
    experts, top = int(r["experts"]), int(r["top"])
    count, keep = int(r["groups"]["count"]), int(r["groups"]["keep"])
    s = torch.sigmoid(z)
    t = s.shape[0]
    per = experts // count
    grouped = s.reshape(t, count, per)
    group_score = grouped.topk(min(2, per), dim=-1).values.sum(dim=-1)
    best = group_score.topk(keep, dim=-1).indices
    allowed = torch.zeros(t, count, dtype=torch.bool)
    allowed.scatter_(1, best, True)
    allowed = allowed.unsqueeze(-1).expand(t, count, per).reshape(t, experts)
    masked = s.masked_fill(~allowed, -math.inf)
    picked = masked.topk(top, dim=-1).indices
    if gaps is not None:
        gap = torch.full((t,), math.inf, dtype=s.dtype)
        if keep < count:
            ordered = group_score.sort(dim=-1, descending=True).values
            gap = torch.minimum(gap, ordered[:, keep - 1] - ordered[:, keep])
        if top < keep * per:
            ordered = masked.sort(dim=-1, descending=True).values
            gap = torch.minimum(gap, ordered[:, top - 1] - ordered[:, top])
        gaps.append(gap)
    weights = s.gather(1, picked)
    weights = weights / (weights.sum(dim=-1, keepdim=True) + 1e-20) * float(r["scale"])
    return picked, weights


def routed_experts(h, w, prefix: str, mlp: dict, gaps: list | None = None):
    r = mlp["router"]
    picked, weights = route(h @ w[prefix + ".router"].T, r, gaps)
    limit = float(mlp["expert"]["limit"])
    out = torch.zeros_like(h)
    for e in range(int(r["experts"])):
        y = clamped_expert(h, w, f"{prefix}.e{e}", limit)
        share = (weights * (picked == e)).sum(dim=-1, keepdim=True)
        out = out + share * y
    if mlp.get("shared") is not None:
        gate = torch.sigmoid(h @ w[prefix + ".shared.sg"].T)  # [T, 1]
        out = out + gate * clamped_expert(h, w, prefix + ".shared", float(mlp["shared"]["limit"]))
    return out


def forward(cfg: dict, w: dict, tokens, want=None, residuals: list | None = None, router_gaps: list | None = None, after_norm=None):
    """Logits [wanted or all, vocab] of one sequence from position 0; ``residuals`` collects the stream after every layer,
    ``router_gaps`` every router's closest decision per token; ``after_norm`` is applied to every part's normed input."""
    after_norm = after_norm or (lambda z: z)
    w = {name: t.to(F64) for name, t in w.items()}
    eps, groups = float(cfg["norm"]["eps"]), int(cfg["norm"]["groups"])
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{int(layer.get('weights_of', i))}"
        if layer["type"] != "parallel":
            raise ValueError(layer["type"])
        delta = pair_mixer(after_norm(group_rms_norm(x, w[p + ".norm1"], groups, eps)), w, p + ".mix", layer["mixer"], eps)
        if layer.get("mlp") is not None:
            delta = delta + routed_experts(after_norm(group_rms_norm(x, w[p + ".norm2"], groups, eps)), w, p + ".mlp", layer["mlp"], router_gaps)
        x = x + delta
        if residuals is not None:
            residuals.append(x.clone())
    if want is not None:
        x = x[torch.as_tensor(want, dtype=torch.long)]
    x = after_norm(group_rms_norm(x, w["final.norm"], groups, eps))
    return (x @ w["embed"].T) * float(cfg["logit_scale"])
