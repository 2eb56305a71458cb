"""Sevadra on the GPU: models of the tests' own sizes through the engine's step function, cache and state manager, cut in every
way, against the plain implementation; each mechanism alone in a model of one layer; weights made so that a lost key shows."""

from __future__ import annotations

import json
import os

import pytest
import torch

import plain_sevadra as plain
import sevadra_helpers as sh
import trace_helpers as th

pytestmark = pytest.mark.gpu

SEEDS = {"A": 3, "B": 4, "C": 1, "D": 1}  # (seeds whose routers decide nothing by a hair for the first dozens of tokens)
LENGTHS = {"long": 150, "mid": 61, "short": 5, "one": 1, "pair": 2, "other": 37}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("sevadra")
    return {name: sh.write_folder(str(root / name), cfg, SEEDS[name]) for name, cfg in sh.configs().items()}


def session(folder: str, dtype: str, max_tokens: int, block_size: int = 16, max_live: int = 4):
    from mini_engine_amd.engine.trace import TraceSession, build_session

    return TraceSession(build_session(folder, dtype, max_tokens, block_size=block_size, max_live=max_live))


def read_cfg(folder: str) -> dict:
    with open(os.path.join(folder, "config.json")) as f:
        return json.load(f)


def assert_close(got: torch.Tensor, want: torch.Tensor, dtype: str, what: str) -> None:
    """float32: no element further off than 2e-5 of its row's largest logit (the rows' logits reach dozens; float32 sums of a few
    hundred terms stay an order of magnitude below that, a key that is lost or seen twice lies orders above). bfloat16, row by row:
    the root mean square of the error (its mean over the row taken off, which no softmax sees) at most 3% of the root mean square of
    the logits, and no element further off than 4% of the row's largest logit (measured on these models of three to five layers, each
    of which rounds a dozen intermediate results: up to 1.8% and 1.4%)."""
    assert got.shape == want.shape, (what, got.shape, want.shape)
    diff = got - want
    if dtype == "float32":
        err = diff.abs().amax(dim=-1)
        bad = err > 2e-5 * want.abs().amax(dim=-1) + 1e-5
    else:
        err = (diff - diff.mean(dim=-1, keepdim=True)).pow(2).mean(dim=-1).sqrt()
        bad = (err > 0.03 * want.pow(2).mean().sqrt()) | (diff.abs().amax(dim=-1) > 0.04 * want.abs().amax(dim=-1))
    if bad.any():
        pos = int(bad.nonzero()[0])
        raise AssertionError(f"{what}: first wrong position {pos} of {got.shape[0]}: error {err[pos].item():.3e} (largest element "
                             f"{diff[pos].abs().max().item():.3e}), the row's largest logit {want[pos].abs().max().item():.3e}")


def check(got: dict, want: dict, dtype: str, what: str, trusted: dict | None = None) -> None:
    for rid, logits in want.items():
        if trusted is None:
            assert_close(got[rid], logits, dtype, f"{what} {rid}")
        elif trusted[rid].any():
            rows = trusted[rid].nonzero().flatten()
            assert_close(got[rid][rows], logits[rows], dtype, f"{what} {rid} (rows {rows.tolist()[:3]}..)")


def trusted_rows(cfg, weights, requests, dtype):
    """float32: every row. bfloat16: the rows before a router decides by a hair (a rounding may pick another expert there) that
    bear a rounding of the stream."""
    if dtype == "float32":
        return None
    out = {}
    for rid, toks in requests.items():
        mask = sh.rows_that_bear_rounding(cfg, weights, toks)
        mask[sh.rows_before_a_close_call(cfg, weights, toks):] = False
        out[rid] = mask
    return out


# ---------------------------------------------------------------- whole models, cut in every way
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_every_cut_of_the_requests_gives_the_plain_logits(folders, name, dtype):
    folder, cfg = folders[name], read_cfg(folders[name])
    weights = sh.read_weights(folder)
    requests = sh.requests_for(cfg, LENGTHS, seed=7)
    want = sh.plain_logits(cfg, weights, requests)
    trusted = trusted_rows(cfg, weights, requests, dtype)
    assert trusted is None or sum(int(m.sum()) for m in trusted.values()) >= 60  # (the bfloat16 runs still compare something)
    bs = sh.BLOCK_SIZES[name]
    cuts = {
        "whole": th.whole(requests),
        "decoded": th.tail_one_by_one(requests, tail=20),
        "portions": th.portions(requests),
        "portions of two and three": th.portions(requests, sizes=(2, 3, 2, 2, 5, 2)),
        # four live requests at most, in a pool of 320 tokens: the pages and slots of requests that ended are used again
        "mixed": th.mixed(requests, max_tokens=320, seed=3, max_live=4),
    }
    for what, steps in cuts.items():
        s = session(folder, dtype, 320, block_size=bs, max_live=4)
        got = th.collect(steps, th.replay_in_process(s, steps))
        check(got, want, dtype, f"{name} {dtype} {what}", trusted)


@pytest.mark.parametrize("name", ["A", "C"])
def test_long_decoding(folders, name):
    """Eight tokens at once, then hundreds one by one: the states, the convolutions' rows and the pages carry every token."""
    folder, cfg = folders[name], read_cfg(folders[name])
    weights = sh.read_weights(folder)
    requests = sh.requests_for(cfg, {"r": 330}, seed=11)
    want = sh.plain_logits(cfg, weights, requests)
    steps = th.tail_one_by_one(requests, tail=322)
    got = th.collect(steps, th.replay_in_process(session(folder, "float32", 384, block_size=sh.BLOCK_SIZES[name]), steps))
    check(got, want, "float32", f"{name} long decoding")


def test_a_batch_of_unequal_requests_against_each_alone(folders):
    """One step holds portions of four requests of very different lengths; then every request decodes beside the others."""
    folder, cfg = folders["A"], read_cfg(folders["A"])
    weights = sh.read_weights(folder)
    requests = sh.requests_for(cfg, {"a": 97, "b": 3, "c": 40, "d": 18}, seed=5)
    want = sh.plain_logits(cfg, weights, requests)
    heads = {"a": 90, "b": 1, "c": 33, "d": 16}
    steps = [{"step": 0, "entries": [{"id": r, "tokens": t[: heads[r]], "want": list(range(heads[r]))} for r, t in requests.items()], "end": []}]
    at = dict(heads)
    while any(at[r] < len(requests[r]) for r in requests):
        entries = [{"id": r, "tokens": [requests[r][at[r]]], "want": [0]} for r in requests if at[r] < len(requests[r])]
        for e in entries:
            at[e["id"]] += 1
        steps.append({"step": len(steps), "entries": entries, "end": [r for r in requests if at[r] == len(requests[r]) and any(e["id"] == r for e in entries)]})
    got = th.collect(steps, th.replay_in_process(session(folder, "float32", 320), steps))
    check(got, want, "float32", "a batch of unequal requests")


# ---------------------------------------------------------------- each mechanism alone: models of one or two layers
def one_layer_models() -> dict[str, dict]:
    att = sh.attention(4, 2, 16, 24, 0.3, sh.rot(10000.0, 8, (4.0, 1.0, 4.0, 32)), conv=4)
    return {
        "attention with convolutions and a rotation of half a head": sh.model(90, 64, 1e-5, 0, [sh.layer(att)]),
        "attention without convolution and rotation": sh.model(90, 64, 1e-5, 0, [sh.layer(sh.attention(2, 2, 32, 32, 0.2))]),
        "a pair of capped attention and time mixing": sh.model(90, 64, 1e-5, 0, [sh.layer(sh.parallel((4, 1, 16, 16, 0.4, 1.0), (4, 16, 8), 0.5, 1.5))]),
        "time mixing beside a silent attention": sh.model(90, 64, 1e-5, 0, [sh.layer(sh.parallel((1, 1, 16, 16, 0.4, 5.0), (2, 32, 4), 0.0, 1.0))]),
        "time mixing over one head of 128 and over heads of 32": sh.model(90, 64, 1e-5, 0, [
            sh.layer(sh.parallel((2, 1, 16, 16, 0.4, 5.0), (1, 128, 8), 0.3, 1.0)), sh.layer(sh.parallel((2, 2, 16, 16, 0.4, 5.0), (3, 32, 5), 0.5, 0.8))]),
        "latent attention": sh.model(90, 64, 1e-5, 0, [sh.layer(sh.latent(3, 16, 8, 24, 40, 0.25, 10000.0))]),
        "latent attention over another layer's latents": sh.model(90, 64, 1e-5, 0, [sh.layer(sh.latent(3, 16, 8, 24, 40, 0.25, 10000.0)),
                                                                                    sh.layer(sh.latent(5, 8, 8, 16, 40, 0.3, 10000.0, kv_from=0))]),
        "a dense feed-forward": sh.model(90, 64, 1e-5, 0, [sh.layer(sh.attention(2, 2, 32, 32, 0.2), sh.dense(96))]),
        "routed experts with identity experts and a shared one": sh.model(90, 64, 1e-5, 0, [sh.layer(sh.attention(2, 2, 32, 32, 0.2), sh.moe(5, 3, 3, 48, shared=32))]),
        "routed experts alone": sh.model(90, 64, 1e-5, 0, [sh.layer(sh.attention(2, 2, 32, 32, 0.2), sh.moe(7, 0, 2, 24))]),
        "a token input": sh.model(90, 64, 1e-5, 12, [sh.layer(sh.attention(2, 2, 32, 32, 0.2)), sh.layer(sh.attention(2, 2, 32, 32, 0.2))]),
    }


@pytest.mark.parametrize("what", list(one_layer_models()))
def test_each_mechanism_alone(tmp_path, what):
    cfg = one_layer_models()[what]
    folder = sh.write_folder(str(tmp_path / "m"), cfg, seed=4)
    weights = sh.read_weights(folder)
    requests = sh.requests_for(cfg, {"a": 75, "b": 1, "c": 9}, seed=9)
    want = sh.plain_logits(cfg, weights, requests)
    for cut, steps in (("whole", th.whole(requests)), ("decoded", th.tail_one_by_one(requests, tail=12)),
                       ("portions", th.portions(requests, sizes=(2, 5, 3, 2, 11)))):
        got = th.collect(steps, th.replay_in_process(session(folder, "float32", 192), steps))
        check(got, want, "float32", f"{what}, {cut}")


# ---------------------------------------------------------------- weights made so that a lost key shows
def far_key_model(kind: str, width: int = 32, vocab: int = 40):
    """A model of one layer whose keys all lie across a direction u, but for the token 1's, which lies along it; the token 2's query
    points along u with a large score scale. Wherever token 2 stands, the softmax is carried by wherever token 1 stood, however
    far back and on whichever page. (The sizes make q the input itself and k its first half: the weights are selections.)"""
    d = width // 2
    g = torch.Generator().manual_seed(3)
    if kind == "attention":
        cfg = sh.model(vocab, width, 1e-6, 0, [sh.layer(sh.attention(2, 1, d, d, 6.0))])
    else:
        cfg = sh.model(vocab, width, 1e-6, 0, [sh.layer(sh.parallel((2, 1, d, d, 6.0, 40.0), (1, 8, 2), 1.0, 0.05))])
    tensors = sh.random_tensors(cfg, seed=2)
    u = torch.randn(d, generator=g)
    u = u / u.norm()
    embed = torch.randn(vocab, width, generator=g)
    embed[:, :d] -= (embed[:, :d] @ u)[:, None] * u[None, :]  # every key across u
    embed[1, :d] = 4 * u  # token 1: its key along u
    embed[2, :d] = 0  # token 2: no key to speak of, its second head's query along u
    embed[2, d:] = 4 * u
    p = "l0.mix" if kind == "attention" else "l0.mix.left"
    eye = torch.eye(width)
    tensors["embed"] = embed.to(torch.bfloat16)
    tensors[p + ".q"] = eye.to(torch.bfloat16)
    tensors[p + ".k"] = eye[:d].to(torch.bfloat16)
    tensors[p + ".q.norm"] = torch.ones(width, dtype=torch.bfloat16)
    tensors[p + ".k.norm"] = torch.ones(d, dtype=torch.bfloat16)
    return cfg, tensors


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", ["attention", "capped attention with a sink"])
def test_a_far_key_carries_the_softmax(tmp_path, kind, dtype):
    cfg, tensors = far_key_model("attention" if kind == "attention" else "pair")
    folder = sh.write_folder(str(tmp_path / "m"), cfg, tensors=tensors)
    weights = sh.read_weights(folder)
    g = torch.Generator().manual_seed(1)
    for key_at in (0, 15, 16, 17, 200):  # the first token, a page's last and first slots, far back
        toks = (torch.randint(3, 40, (420,), generator=g)).tolist()
        toks[key_at] = 1
        for q_at in (key_at + 1 if key_at else 1, 250, 400, 419):
            toks[q_at] = 2
        requests = {"r": toks}
        want = sh.plain_logits(cfg, weights, requests)
        probe = plain.forward(cfg, {k: (v if k != "embed" else torch.cat((v[:1], v[3:4], v[2:])))
                                    for k, v in weights.items()}, toks).to(torch.float32)
        assert (probe[419] - want["r"][419]).abs().max() > 0.05 * want["r"][419].abs().max()  # (the key does carry the row)
        for cut, steps in (("whole", th.whole(requests)), ("decoded", th.tail_one_by_one(requests, tail=25)),
                           ("portions", th.portions(requests, sizes=(64, 2, 17, 100, 3)))):
            got = th.collect(steps, th.replay_in_process(session(folder, dtype, 448), steps))
            if dtype == "float32":
                check(got, want, dtype, f"{kind}, key at {key_at}, {cut}")
            else:  # (the rows whose softmax the one key carries: the other rows' sharp scores do not bear a rounding)
                rows = [i for i, t in enumerate(toks) if t == 2]
                assert_close(got["r"][rows], want["r"][rows], dtype, f"{kind}, key at {key_at}, {cut}")


# ---------------------------------------------------------------- generation through the engine's own entry point
@pytest.mark.parametrize("name", ["A", "D"])
def test_greedy_generation_through_the_engine_and_its_scheduler(folders, name):
    from mini_engine_amd import EngineConfig, LLMEngine, SamplingParams

    folder, cfg = folders[name], read_cfg(folders[name])
    weights = sh.read_weights(folder)
    prompts = list(sh.requests_for(cfg, {"a": 23, "b": 4, "c": 1, "d": 40, "e": 9, "f": 15}, seed=2).values())
    new = 12
    expected = []
    for p in prompts:
        toks = list(p)
        for _ in range(new):
            toks.append(int(plain.forward(cfg, weights, toks)[-1].argmax()))
        expected.append(toks[len(p):])
    for graphs in (True, False):
        engine = LLMEngine.from_pretrained(folder, EngineConfig(dtype="float32", num_blocks=40, block_size=sh.BLOCK_SIZES[name], max_num_seqs=4,
                                                                max_num_batched_tokens=48, cuda_graphs=graphs))
        got = engine.generate(prompts, SamplingParams(max_tokens=new))
        assert got == expected, f"{name}, graphs {graphs}: {got} vs {expected}"
