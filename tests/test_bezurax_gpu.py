"""Bezurax on the GPU: each new kernel against the plain implementation's function for the same mechanism, then whole
models of the tests' own sizes through the engine's step function, cache and state manager and scheduler, cut in every way."""

from __future__ import annotations

import math

import pytest
import torch

import bezurax_helpers as bh
import plain_bezurax as plain
import trace_helpers as th

pytestmark = pytest.mark.gpu

F64 = torch.float64
TOL = {torch.float32: 2e-5, torch.bfloat16: 2e-2}


def rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    """Largest error of a row against that row's largest value."""
    got, want = got.detach().cpu().to(F64), want.detach().cpu().to(F64)
    return float(((got - want).abs().amax(-1) / want.abs().amax(-1).clamp_min(1e-30)).max())


def shuffled_table(items_len: list[int], bs: int, seed: int):
    """A block table whose pages lie in no order (as pages that were freed and taken again do), and the pool's size."""
    need = [-(-n // bs) for n in items_len]
    g = torch.Generator().manual_seed(seed)
    pages = torch.randperm(sum(need) + 3, generator=g).tolist()
    table = torch.full((len(items_len), max(need)), -1, dtype=torch.int32)
    at = 0
    for i, n in enumerate(need):
        table[i, :n] = torch.tensor(pages[at : at + n], dtype=torch.int32)
        at += n
    return table, sum(need) + 3


# ------------------------------------------------------------------------------------- the norm in groups
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("dim,groups", [(96, 3), (128, 1), (100, 5), (1024, 2), (60, 60)])
def test_the_residual_sum_and_the_norm_in_groups(dim, groups, dtype):
    from mini_engine_amd.ops import kernels as K

    g = torch.Generator().manual_seed(dim + groups)
    x = torch.randn(7, dim, generator=g)
    delta = torch.randn(7, dim, generator=g).to(dtype)
    w = 1 + 0.3 * torch.randn(dim, generator=g)
    dev = x.cuda()
    got = K.add_group_rmsnorm(dev, delta.cuda(), w.cuda(), 1e-5, dtype, groups=groups)
    new = x.to(F64) + delta.to(F64)
    assert rel_err(dev, new) < 1e-6  # the residual stays in float32
    assert rel_err(got, plain.group_rms_norm(new, w.to(F64), groups, 1e-5)) < TOL[dtype]


# ------------------------------------------------------------------- attention over a window and pooled blocks
def pooled_case(nh, nkv, d, window, pool, bs, lens, dtype, seed, mark=None):
    """Random projections (queries, keys; the values are the keys as projected) of some sequences, rounded to ``dtype``; what
    the plain implementation makes of each; pages in no order. ``mark`` (item, query position, key position, shown): that query
    of head 0 points along a direction u that every key of the item is orthogonal to; if ``shown``, the key at the key position
    points along u, so that it, or the pooled block it lies in, carries the softmax wherever it is seen."""
    g = torch.Generator().manual_seed(seed)
    width = (nh + nkv) * d
    rows = [torch.randn(n, width, generator=g) for n in lens]
    if mark is not None:
        item, qpos, kpos, shown = mark
        u = torch.randn(d, generator=g)
        u = u / u.norm()
        keys = rows[item][:, nh * d : nh * d + d]
        keys -= (keys @ u)[:, None] * u[None, :]
        rows[item][qpos, :d] = 40 * u
        if shown:
            rows[item][kpos, nh * d : nh * d + d] = 40 * u
    rows = [r.to(dtype) for r in rows]
    qw, kw = 1 + 0.2 * torch.randn(nh * d, generator=g), 1 + 0.2 * torch.randn(nkv * d, generator=g)
    if mark is not None:
        qw[:d], kw[:d] = 1.0, 1.0  # (the norms' weights leave the direction alone)
    m = {"heads": nh, "kv_heads": nkv, "dim": d, "scale": (1.0 if mark else 0.3) / math.sqrt(d), "mask": {"size": window, "pool": pool}}
    sel = torch.eye(width, dtype=F64)
    w = {"m.q": sel[: nh * d], "m.k": sel[nh * d :], "m.q.norm": qw.to(F64), "m.k.norm": kw.to(F64), "m.o": torch.eye(nh * d, dtype=F64)}
    want = [plain.pooled_window_attention(r.to(F64), w, "m", m, 1e-5) for r in rows]
    table, pages = shuffled_table(lens, bs, seed)
    return rows, qw, kw, m, want, table, pages


def run_pooled(rows, qw, kw, m, table, pages, bs, dtype, cuts, tiled, out_cols=None):
    """The steps of ``cuts`` ([(item, lo, hi), ...] each) through the page writes and the attention kernels: the general kernel, or
    with ``tiled`` the matrix-core kernels. ``out_cols`` (row, column, scale): the result goes into wider rows."""
    from mini_engine_amd.ops import kernels as K

    nh, nkv, d = m["heads"], m["kv_heads"], m["dim"]
    window, pool = m["mask"]["size"], m["mask"]["pool"]
    kc, kp = (torch.zeros(pages, nkv, bs, d, dtype=dtype).cuda() for _ in range(2))
    vc, vp = (torch.zeros(pages, nkv, d, bs, dtype=dtype).cuda() for _ in range(2))
    outs = {i: [] for i in range(len(rows))}
    for step in cuts:
        proj = torch.cat([rows[i][lo:hi] for i, lo, hi in step]).cuda().contiguous()
        pos = torch.tensor([p for i, lo, hi in step for p in range(lo, hi)], dtype=torch.int32).cuda()
        item = torch.tensor([n for n, (i, lo, hi) in enumerate(step) for _ in range(lo, hi)], dtype=torch.int32).cuda()
        tab = table[[i for i, lo, hi in step]].cuda().contiguous()
        q = K.whole_norm_scatter(proj, qw.cuda(), kw.cuda(), pos, item, tab, kc, vc, nh, nkv, d, d, 1e-5, k_pool=kp, v_pool=vp,
                                 pooled_block=pool, single_tokens=all(hi - lo == 1 for i, lo, hi in step))
        row, col, scale = out_cols or (nh * d, 0, 1.0)
        out = torch.full((proj.shape[0], row), 7.0, dtype=dtype).cuda()
        if tiled:
            qlens = [hi - lo for i, lo, hi in step]
            starts = [lo for i, lo, hi in step]
            item_start = torch.tensor([0] + list(torch.tensor(qlens).cumsum(0)), dtype=torch.int32).cuda()
            K.attention_pooled_bf16(q, kc, vc, kp, vp, pos, item_start, starts, qlens, tab, m["scale"], window, pool, out=out, out_col=col,
                                    out_scale=scale)
        else:
            K.attention_pooled(q, kc, vc, kp, vp, pos, item, tab, m["scale"], window, pool, out=out, out_col=col, out_scale=scale)
        if out_cols:  # nothing beside the result's columns is written
            assert bool((out[:, :col] == 7.0).all()) and bool((out[:, col + nh * d :] == 7.0).all())
        at = 0
        for i, lo, hi in step:
            outs[i].append(out[at : at + hi - lo, col : col + nh * d].float().cpu() / scale)
            at += hi - lo
    return {i: torch.cat(v) for i, v in outs.items()}


CUTS = lambda n0, n1: [[(0, 0, 2), (1, 0, 1)], [(0, 2, 19), (1, 1, 2)], [(1, 2, 3), (0, 19, n0 - 11)], [(0, n0 - 11, n0 - 9), (1, 3, 4)],
                       [(0, n0 - 9, n0 - 8), (1, 4, n1)]] + [[(0, p, p + 1)] for p in range(n0 - 8, n0)]  # noqa: E731


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,nkv,d,window,pool,bs", [(4, 2, 24, 40, 5, 16), (3, 1, 16, 9, 1, 8), (6, 6, 20, 64, 16, 32), (5, 1, 12, 33, 7, 8),
                                                     (2, 2, 64, 128, 32, 16), (2, 1, 8, 1, 1, 8), (2, 1, 8, 300, 3, 16)])
def test_window_and_pooled_blocks_share_one_softmax(nh, nkv, d, window, pool, bs, dtype):
    """Two sequences, whole in one step and then cut (two tokens, across page borders, the last tokens one by one): the values
    are the keys before their norm, the pooled means are those of the keys as the pages hold them."""
    lens = [300, 45]
    rows, qw, kw, m, want, table, pages = pooled_case(nh, nkv, d, window, pool, bs, lens, dtype, seed=nh * 100 + d)
    whole = run_pooled(rows, qw, kw, m, table, pages, bs, dtype, [[(0, 0, 300), (1, 0, 45)]], tiled=False)
    cut = run_pooled(rows, qw, kw, m, table, pages, bs, dtype, CUTS(300, 45), tiled=False, out_cols=(nh * d + 24, 8, 0.7))
    for i in (0, 1):
        assert rel_err(whole[i], want[i]) < TOL[dtype], i
        assert rel_err(cut[i], want[i]) < TOL[dtype], i
        if dtype is torch.float32:
            assert rel_err(cut[i], whole[i]) < 1e-6


@pytest.mark.parametrize("nh,nkv,d,window,pool,bs", [(4, 2, 32, 40, 5, 16), (8, 1, 64, 100, 12, 16), (6, 3, 96, 80, 10, 64), (16, 8, 128, 256, 32, 16),
                                                     (2, 1, 32, 1, 1, 16), (2, 2, 64, 700, 3, 32), (6, 2, 64, 64, 64, 64)])
def test_the_matrix_core_kernels_see_what_the_general_kernel_sees(nh, nkv, d, window, pool, bs):
    """bfloat16 through the tiled kernel (prompts, portions, tokens beside portions) and the split-context kernel (steps of
    single tokens), into columns of wider rows: against the plain implementation, as close as the general kernel is."""
    from mini_engine_amd.ops import kernels as K

    lens = [600, 77]
    rows, qw, kw, m, want, table, pages = pooled_case(nh, nkv, d, window, pool, bs, lens, torch.bfloat16, seed=nh + d + window)
    # the tiled kernel's blocks of 128 query columns, then those of 256 (which a step takes by its size: both are forced here)
    for limits in ((1e30, 1e30), (0.0, 0.0)):
        before = K.set_prefill_wide_limits(*limits)
        try:
            whole = run_pooled(rows, qw, kw, m, table, pages, bs, torch.bfloat16, [[(0, 0, 600), (1, 0, 77)]], tiled=True)
            cut = run_pooled(rows, qw, kw, m, table, pages, bs, torch.bfloat16, CUTS(599, 76) + [[(0, 599, 600), (1, 76, 77)]], tiled=True,
                             out_cols=(nh * d + 32, 16, 0.7))
        finally:
            K.set_prefill_wide_limits(*before)
        for i in (0, 1):
            assert rel_err(whole[i], want[i]) < TOL[torch.bfloat16], (i, limits)
            assert rel_err(cut[i], want[i]) < TOL[torch.bfloat16], (i, limits)


@pytest.mark.parametrize("tiled", [False, True])
@pytest.mark.parametrize("behind", [-1, 0, 1, 2, 3, 7, 8, 250])
def test_a_key_at_the_windows_edge_and_in_a_pooled_block(behind, tiled):
    """One key that outweighs all others, ``behind`` positions beyond the window of the last query (-1: the window's last key),
    window 40, blocks of 6, the query at position 299: behind the window it is seen only once its block is wholly behind it
    (its block's mean then carries the softmax), and not at all before that. In a prompt, and decoded alone."""
    nh, nkv, d, window, pool, bs, n = 2, 1, 32, 40, 6, 16, 300
    dtype = torch.bfloat16 if tiled else torch.float32
    kpos = n - 1 - (window - 1) - behind - 1 if behind >= 0 else n - window
    rows, qw, kw, m, want, table, pages = pooled_case(nh, nkv, d, window, pool, bs, [n], dtype, seed=behind + 5, mark=(0, n - 1, kpos, True))
    unmarked = pooled_case(nh, nkv, d, window, pool, bs, [n], dtype, seed=behind + 5, mark=(0, n - 1, kpos, False))[4]
    seen = (n - 1 - kpos < window) or (kpos // pool * pool + pool - 1 <= n - 1 - window)
    moved = float((want[0][-1, :d] - unmarked[0][-1, :d]).abs().max()) > 0.5 * float(unmarked[0][-1, :d].abs().max())
    assert moved == seen  # the mark decides head 0's output where it is seen, and changes nothing where it is not
    for cuts in ([[(0, 0, n)]], [[(0, 0, n - 3)], [(0, n - 3, n - 1)], [(0, n - 1, n)]]):
        got = run_pooled(rows, qw, kw, m, table, pages, bs, dtype, cuts, tiled=tiled)
        assert rel_err(got[0], want[0]) < TOL[dtype]


# ------------------------------------------------------------------------------------- the generalized delta rule
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,d,rank", [(2, 16, 8), (3, 24, 12), (1, 40, 20), (4, 12, 4), (2, 64, 32), (1, 128, 16), (2, 200, 5)])
def test_delta_rule_against_the_plain_recurrence(heads, d, rank, dtype):
    """Three sequences: whole in one step, and cut into steps (two tokens, one token, a sequence left out of a step), in state
    slots that were used before; the state after the last step is the plain one."""
    from mini_engine_amd.ops import kernels as K

    g = torch.Generator().manual_seed(heads * 100 + d)
    hd = heads * d
    lens = [70, 9, 33]
    width = 5 * hd + rank
    cols = {r: i * hd for i, r in enumerate(("r", "k", "v", "g", "a", "w1"))}
    rows = [(torch.randn(n, width, generator=g) * (1.0 if d < 100 else 0.5)).to(dtype) for n in lens]
    w2 = (0.5 * torch.randn(hd, rank, generator=g)).to(dtype)
    w0, ab, nw = torch.randn(hd, generator=g), torch.randn(hd, generator=g), 1 + 0.2 * torch.randn(hd, generator=g)
    sel = torch.eye(width, dtype=F64)
    w = {f"m.{r}": sel[c : c + (rank if r == "w1" else hd)] for r, c in cols.items()}
    w.update({"m.w2": w2.to(F64), "m.w0": w0.to(F64), "m.a.b": ab.to(F64), "m.norm": nw.to(F64), "m.o": torch.eye(hd, dtype=F64)})
    # (the gate's sigmoid is part of the plain function: it reads the same column)
    want = [plain.delta_rule(r.to(F64), w, "m", {"heads": heads, "dim": d}, 1e-5) for r in rows]
    coef = math.exp(-0.5)

    def run(cuts, slots):
        state = torch.randn(5, heads, d, d, generator=g).cuda()  # what earlier requests left in the slots
        outs, began = {i: [] for i in range(3)}, set()
        for step in cuts:
            for i, lo, hi in step:
                if i not in began:  # a request's state begins at zero (the state manager clears the slot it hands out)
                    state[slots[i]].zero_()
                    began.add(i)
            proj = torch.cat([rows[i][lo:hi] for i, lo, hi in step]).cuda().contiguous()
            item_start = torch.tensor([0] + list(torch.tensor([hi - lo for _, lo, hi in step]).cumsum(0)), dtype=torch.int32).cuda()
            state_slots = torch.tensor([slots[i] for i, _, _ in step], dtype=torch.int32).cuda()
            out = torch.full((proj.shape[0], hd + 16), 7.0, dtype=dtype).cuda()
            K.delta_rule(proj, cols, w2.cuda(), w0.cuda(), ab.cuda(), nw.cuda(), state, item_start, state_slots, heads, d, 1e-5, coef, out=out,
                         out_col=8, out_scale=1.3)
            assert bool((out[:, :8] == 7.0).all()) and bool((out[:, 8 + hd :] == 7.0).all())
            at = 0
            for i, lo, hi in step:
                outs[i].append(out[at : at + hi - lo, 8 : 8 + hd].float().cpu() / 1.3)
                at += hi - lo
        return {i: torch.cat(v) for i, v in outs.items()}, state.cpu()

    slots = [3, 0, 4]
    whole, s_whole = run([[(0, 0, 70), (1, 0, 9), (2, 0, 33)]], slots)
    cuts = [[(0, 0, 2), (1, 0, 1)], [(0, 2, 3), (1, 1, 9), (2, 0, 2)], [(0, 3, 40)], [(2, 2, 33), (0, 40, 42)]] + [[(0, p, p + 1)] for p in range(42, 70)]
    cut, s_cut = run(cuts, slots)
    tol = 6e-2 if dtype is torch.bfloat16 else 3e-4  # (a float32 recurrence over 70 tokens, sums over up to 200 rows of state)
    for i in range(3):
        assert rel_err(whole[i], want[i][0]) < tol, i
        assert rel_err(cut[i], want[i][0]) < tol, i
        if dtype is torch.float32:
            assert rel_err(cut[i], whole[i]) < 1e-5
        for s in (s_whole, s_cut):
            assert rel_err(s[slots[i]].reshape(heads, d * d), want[i][1].reshape(heads, d * d)) < tol


def test_the_state_carries_what_a_token_far_back_wrote():
    """A head whose decay is (almost) none and whose removal rate is (almost) none keeps k v^T of the first token for good:
    300 tokens later a query along that key reads that value, through steps of every size."""
    from mini_engine_amd.ops import kernels as K

    heads, d, rank, n = 1, 32, 4, 300
    g = torch.Generator().manual_seed(3)
    hd = d
    cols = {r: i * hd for i, r in enumerate(("r", "k", "v", "g", "a", "w1"))}
    x = torch.zeros(n, 5 * hd + rank)
    e = torch.zeros(d)
    e[0] = 1.0
    noise = torch.randn(n, d, generator=g)
    noise[:, 0] = 0.0  # every later key is orthogonal to the first
    x[:, cols["k"] : cols["k"] + d] = noise
    x[0, cols["k"] : cols["k"] + d] = 4 * e
    x[:, cols["v"] : cols["v"] + d] = 0.1 * torch.randn(n, d, generator=g)
    value = torch.randn(d, generator=g)
    x[0, cols["v"] : cols["v"] + d] = value
    x[:, cols["r"] : cols["r"] + d] = 0.01 * torch.randn(n, d, generator=g)
    x[n - 1, cols["r"] : cols["r"] + d] = e
    x[:, cols["g"] : cols["g"] + d] = 8.0   # gates open
    x[:, cols["a"] : cols["a"] + d] = -30.0  # nothing removed
    w2, w0 = torch.zeros(hd, rank), torch.full((hd,), -30.0)  # decay exp(-c sigmoid(-30)): none
    ab, nw = torch.zeros(hd), torch.ones(hd)
    sel = torch.eye(5 * hd + rank, dtype=F64)
    w = {f"m.{r}": sel[c : c + (rank if r == "w1" else hd)] for r, c in cols.items()}
    w.update({"m.w2": w2.to(F64), "m.w0": w0.to(F64), "m.a.b": ab.to(F64), "m.norm": nw.to(F64), "m.o": torch.eye(hd, dtype=F64)})
    want, _ = plain.delta_rule(x.to(F64), w, "m", {"heads": heads, "dim": d}, 1e-5)
    unit = value / value.pow(2).mean().sqrt()
    assert rel_err(want[-1:].float(), (4 * unit).unsqueeze(0) / 4) < 0.05  # the last output is the first token's value, normed
    for cuts in ([(0, n)], [(0, 7), (7, 9), (9, 250)] + [(p, p + 1) for p in range(250, n)]):
        state = torch.zeros(2, heads, d, d).cuda()
        outs = []
        for lo, hi in cuts:
            item_start = torch.tensor([0, hi - lo], dtype=torch.int32).cuda()
            outs.append(K.delta_rule(x[lo:hi].cuda().contiguous(), cols, w2.cuda(), w0.cuda(), ab.cuda(), nw.cuda(), state, item_start,
                                     torch.tensor([1], dtype=torch.int32).cuda(), heads, d, 1e-5, math.exp(-0.5)).cpu())
        assert rel_err(torch.cat(outs), want) < 1e-4
        assert float(state[0].abs().max()) == 0.0  # the other slot is nobody's


# ------------------------------------------------------------------------------------- routed experts
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hidden,ff,experts,top,count,keep,tokens,shared", [
    (96, 40, 6, 2, 3, 2, 37, 24), (128, 32, 4, 3, 1, 1, 150, 0), (128, 48, 8, 1, 8, 3, 3, 72), (100, 24, 4, 4, 2, 2, 1, 8),
    (128, 64, 6, 2, 2, 1, 300, 64), (64, 16, 12, 3, 4, 2, 64, 0), (80, 20, 8, 8, 4, 4, 5, 20)])
def test_scored_router_groups_limits_and_the_shared_expert(hidden, ff, experts, top, count, keep, tokens, shared, dtype):
    """Sigmoid scores, groups scored by their two best, the picks' scores over their sum times a scale, experts that clamp before
    the activation, and the shared expert's gate: the routed part, and the gate that the same launch leaves for the shared one."""
    from mini_engine_amd.ops import kernels as K

    g = torch.Generator().manual_seed(hidden + experts + top)
    h = torch.randn(tokens, hidden, generator=g).to(dtype)
    limit, scale = 0.9, 1.7
    w = {"m.router": (0.3 * torch.randn(experts, hidden, generator=g)).to(torch.bfloat16)}
    for e in range(experts):
        w.update({f"m.e{e}.{n}": (0.2 * torch.randn((hidden, ff) if n == "down" else (ff, hidden), generator=g)).to(dtype) for n in ("gate", "up", "down")})
    mlp = {"router": {"experts": experts, "top": top, "groups": {"count": count, "keep": keep}, "scale": scale}, "expert": {"ff": ff, "limit": limit}}
    router = w["m.router"].float()
    if shared:
        w["m.shared.sg"] = (0.3 * torch.randn(1, hidden, generator=g)).to(torch.bfloat16)
        router = torch.cat((router, w["m.shared.sg"].float()))
    gaps: list = []
    want = plain.routed_experts(h.to(F64), {k: v.to(F64) for k, v in w.items()}, "m", mlp, gaps)
    sure = gaps[0] > 1e-3  # (a pick decided by less is a rounding's to make)
    gate_up = torch.stack([torch.cat((w[f"m.e{e}.gate"], w[f"m.e{e}.up"])) for e in range(experts)]).cuda()
    down = torch.stack([w[f"m.e{e}.down"] for e in range(experts)]).cuda()
    got = K.routed_ff_scored(h.cuda(), router.cuda(), gate_up, down, top, "clamped_sigmoid", limit, "sigmoid_normalized", count, keep, scale,
                             shared=bool(shared))
    parts, gate = got if shared else (got, None)
    assert parts.parts.shape == (top, tokens, hidden)
    assert rel_err(parts.parts.sum(0)[sure], want[sure]) < TOL[dtype]
    if shared:
        assert rel_err(gate.unsqueeze(0), torch.sigmoid(h.to(F64) @ w["m.shared.sg"].to(F64).T).T) < 1e-5
        # the shared expert's activation with a limit of its own, every row times its gate
        gu = torch.randn(tokens, 2 * shared, generator=g).to(dtype)
        out = K.gated_rows(gu.cuda(), gate, "clamped_sigmoid", 0.6)
        a, b = gu[:, :shared].to(F64).clamp(max=0.6), gu[:, shared:].to(F64).clamp(-0.6, 0.6)
        assert rel_err(out, a * torch.sigmoid(1.702 * a) * (b + 1) * gate.cpu().to(F64).unsqueeze(1)) < TOL[dtype]


# --------------------------------------------------------------------------------- models through the engine
def assert_logits_close(got, want, dtype, what, loose=1.0):
    """float32: the bound of the other models' tests. bfloat16, row by row: no element further off than 4% of the row's
    largest logit and a root-mean-square error of at most 3% of the row's root mean square; one row in twenty (at least
    one) may miss that."""
    if dtype == "float32":
        return th.assert_logits_close(got, want, dtype, what)
    err = (got - want).abs()
    bad = (err.max(dim=-1).values > 0.04 * loose * want.abs().max(dim=-1).values) | (
        err.pow(2).mean(dim=-1).sqrt() > 0.03 * loose * want.pow(2).mean(dim=-1).sqrt())
    if int(bad.sum()) > max(1, got.shape[0] // 20):
        pos = int(bad.nonzero()[0])
        raise AssertionError(f"{what}: {int(bad.sum())} rows off, the first at {pos} of {got.shape[0]}: error {err[pos].max().item():.3e}, the row's "
                             f"largest logit {want[pos].abs().max().item():.3e}")


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {n: bh.write_folder(str(tmp_path_factory.mktemp(f"bezurax_{n}")), cfg, seed=61 + i) for i, (n, cfg) in enumerate(bh.configs().items())}


def requests_for(cfg, seed, lengths=(1, 23, 97, 150, 61)):
    g = torch.Generator().manual_seed(seed)
    return {f"r{i}": torch.randint(0, cfg["vocab"], (n,), generator=g).tolist() for i, n in enumerate(lengths)}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E"])
def test_every_way_of_cutting_gives_the_plain_logits(folders, name, dtype):
    """Whole prompts; most of a prompt and its tail token by token (replayed graphs); portions down to two tokens; up to
    four live requests in a pool whose pages and state slots are used again: all against the plain implementation."""
    from mini_engine_amd.engine.trace import TraceSession, build_session

    cfg = bh.configs()[name]
    reqs = requests_for(cfg, seed=7)
    weights = bh.read_weights(folders[name])
    want = bh.plain_logits(cfg, weights, reqs)
    # bfloat16: a router's pick between two experts whose scores nearly tie is decided by a rounding, and what the token
    # then leaves in the cache and the state reaches every later one: rows are compared up to a sequence's first such pick
    # (and rows whose plain logits do not bear a rounding of the normed activations are left out as well)
    keep = {rid: torch.ones(len(t), dtype=torch.bool) for rid, t in reqs.items()}
    if dtype == "bfloat16":
        for rid, t in reqs.items():
            keep[rid] = bh.rows_that_bear_rounding(cfg, weights, t)
            keep[rid][bh.rows_before_a_close_call(cfg, weights, t):] = False
    assert sum(int(k.sum()) for k in keep.values()) >= 12  # (float32 compares every row; few rows of the configurations with
    # many experts a layer come before a close call)
    bs = bh.BLOCK_SIZES[name]
    biggest = max(th.round_up(len(t)) for t in reqs.values())
    for build, max_tokens, live in ((th.whole, biggest, 4), (lambda r: th.tail_one_by_one(r, tail=60), biggest, 4),
                                    (th.portions, biggest, 4), (lambda r: th.mixed(r, 448, seed=3, max_live=3), 448, 3)):
        session = TraceSession(build_session(folders[name], dtype, max_tokens, block_size=bs, max_live=live))
        steps = build(reqs)
        got = th.collect(steps, th.replay_in_process(session, steps))
        for rid in reqs:
            assert got[rid].shape == want[rid].shape
            if keep[rid].any():
                assert_logits_close(got[rid][keep[rid]], want[rid][keep[rid]], dtype, f"{name} {dtype} {rid}")
    assert len({int(t) for t in want["r3"].argmax(-1)}) > 10


def test_float32_logits_do_not_depend_on_the_cut_or_the_company(folders):
    from mini_engine_amd.engine.trace import TraceSession, build_session

    cfg = bh.configs()["A"]
    reqs = requests_for(cfg, seed=9, lengths=(130, 45, 77))
    outs = []
    for build in (th.whole, th.portions, lambda r: th.mixed(r, 320, seed=5, max_live=3)):
        session = TraceSession(build_session(folders["A"], "float32", 320, block_size=16, max_live=3))
        steps = build(reqs)
        outs.append(th.collect(steps, th.replay_in_process(session, steps)))
    for rid in reqs:
        for other in outs[1:]:
            assert rel_err(other[rid], outs[0][rid]) < 2e-5


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_from_a_short_prompt(folders, dtype):
    """Three tokens of prompt, then 300 tokens one by one through replayed graphs: the window passes over decoded tokens,
    pooled blocks are completed by decoded tokens, over many page borders. bfloat16 (heads of 64: the matrix-core kernels)
    is held against float32 where the plain logits bear a rounding."""
    from mini_engine_amd.engine.trace import TraceSession, build_session

    name = "C" if dtype == "float32" else "D"
    cfg = bh.configs()[name]
    reqs = requests_for(cfg, seed=13, lengths=(303,))
    weights = bh.read_weights(folders[name])
    want = bh.plain_logits(cfg, weights, reqs)
    session = TraceSession(build_session(folders[name], dtype, 320, block_size=bh.BLOCK_SIZES[name], max_live=2))
    steps = th.tail_one_by_one(reqs, tail=300)
    got = th.collect(steps, th.replay_in_process(session, steps))
    if dtype == "float32":
        th.assert_logits_close(got["r0"], want["r0"], "float32", "long decoding")
    else:
        keep = bh.rows_that_bear_rounding(cfg, weights, reqs["r0"])
        keep[bh.rows_before_a_close_call(cfg, weights, reqs["r0"]):] = False
        assert int(keep.sum()) > 10
        assert_logits_close(got["r0"][keep], want["r0"][keep], dtype, "long decoding")
    assert session.engine.runner.graph_replays >= 299


def marked_model(window: int, pool: int, d: int = 16):
    """One layer whose left mixer alone speaks (the right one's scale is nought, no feed-forward): every query points along e;
    the key of token 1 (the mark) points along e, every other token's key is orthogonal to it. The values are the keys, so a
    sequence whose last token sees the mark (in its window, or in a pooled block) reads e, and any other reads none of it."""
    vocab, width = 40, 32
    cfg = bh.model(vocab, width, 1e-6, 2, 1.0, [bh.layer(bh.left(2, 1, d, 2.0, window, pool), bh.right(1, 8, 4), 1.0, 0.0)])
    t = {k: torch.zeros(v.shape) for k, v in bh.random_tensors(cfg, 0).items()}
    g = torch.Generator().manual_seed(0)
    e = torch.ones(d) / math.sqrt(d)
    embed = torch.randn(vocab, width, generator=g)
    embed[:, 0] = 0.0
    embed[:, 1] = 3.0  # a constant that every token carries: what the queries read
    embed[1, 2:] = 0.0
    embed[1, 0] = 9.0  # the mark
    t["embed"] = embed
    for n in ("l0.norm1", "final.norm", "l0.mix.left.q.norm", "l0.mix.left.k.norm", "l0.mix.right.norm"):
        t[n] = torch.ones(t[n].shape)
    noise = 0.3 * torch.randn(d, width - 2, generator=g)
    t["l0.mix.left.k"][:, 2:] = noise - e[:, None] * (e @ noise)[None, :]
    t["l0.mix.left.k"][:, 0] = 5.0 * e
    t["l0.mix.left.q"][:, 1] = torch.cat((e, e)) * 6.0
    t["l0.mix.left.o"] = torch.randn(width, 2 * d, generator=g)
    return cfg, t


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_marked_token_decides_the_logits_where_the_mask_shows_it(tmp_path, dtype):
    """Window 40, blocks of 6, 202 tokens: the mark as the window's last key, just behind it in a block that is not yet wholly
    behind it (seen by nobody), in the newest block that is, far back just behind a page's border, and nowhere. Whole, in
    portions and decoded: the logits follow the plain implementation's, which differ widely between these."""
    from mini_engine_amd.engine.trace import TraceSession, build_session

    window, pool, n = 40, 6, 202
    cfg, t = marked_model(window, pool, d=32 if dtype == "bfloat16" else 16)
    vocab = cfg["vocab"]
    folder = bh.write_folder(str(tmp_path / "marked"), cfg, tensors={k: v.to(torch.bfloat16) for k, v in t.items()})
    base = torch.randint(2, vocab, (n,), generator=torch.Generator().manual_seed(1)).tolist()
    last = n - 1
    edge = last - window  # the newest position outside the last token's window: 161, in the block 156..161, wholly behind it
    reqs = {}
    for name, mark in (("in", edge + 1), ("pooled", edge), ("far", 17), ("first", 0), ("none", None)):
        toks = list(base)
        if mark is not None:
            toks[mark] = 1
        reqs[name] = toks
    # two tokens on, the last token's window ends at 163: 162 and 163 lie in a block (162..167) that is not behind it
    reqs["unseen"] = list(base) + base[:2]
    reqs["unseen"][edge + 1] = 1
    weights = bh.read_weights(folder)
    want = bh.plain_logits(cfg, weights, reqs)
    size = lambda x: float(x.abs().max())  # noqa: E731
    for name in ("in", "pooled", "far", "first"):
        assert size(want[name][-1] - want["none"][-1]) > 0.3 * size(want["none"][-1]), name
    blank = list(base) + base[:2]
    assert size(want["unseen"][-1] - bh.plain_logits(cfg, weights, {"b": blank})["b"][-1]) < 1e-9
    assert size(want["unseen"][-3] - want["none"][-1]) > 0.3 * size(want["none"][-1])  # (two tokens earlier it was seen)
    for build in (th.whole, lambda r: th.tail_one_by_one(r, tail=50), th.portions):
        session = TraceSession(build_session(folder, dtype, 256, block_size=16, max_live=2))
        steps = build(reqs)
        got = th.collect(steps, th.replay_in_process(session, steps))
        for rid in reqs:
            # (bfloat16: keys that are orthogonal to the queries only until they are rounded make scores of their rounding, which
            # a scale of 2 sharpens: twice the other tests' bound, against marks that move the logits by more than their size)
            assert_logits_close(got[rid], want[rid], dtype, f"marked token {rid}", loose=2.0)


@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_through_the_scheduler(folders, name):
    """Unequal prompts through ``LLMEngine.generate``: a token budget that cuts prompts into portions, a pool that fits two
    of the three requests at a time. float32 picks the plain implementation's tokens."""
    from mini_engine_amd import EngineConfig, LLMEngine, SamplingParams

    cfg = bh.configs()[name]
    w = bh.read_weights(folders[name])
    prompts = list(requests_for(cfg, seed=17, lengths=(40, 9, 75)).values())
    new = 12
    want = []
    for p in prompts:
        toks = list(p)
        for _ in range(new):
            toks.append(int(plain.forward(cfg, w, toks)[-1].argmax()))
        want.append(toks[len(p):])
    bs = bh.BLOCK_SIZES[name]
    engine = LLMEngine.from_pretrained(folders[name], EngineConfig(dtype="float32", block_size=bs, num_blocks=160 // bs,
                                                                   max_num_seqs=3, max_num_batched_tokens=32, max_model_len=128,
                                                                   enable_prefix_caching=False))
    got = engine.generate(prompts, SamplingParams(max_tokens=new, ignore_eos=True))
    assert got == want
