"""Zatinex in the engine against the plain implementation (plain_zatinex.py): each mechanism's
kernels, each mixer alone in a one-layer model, whole prompts, decoding, portions, mixed batches,
reused pages and state rows, far tokens, page borders, generation through the entry points."""

import copy
import json
import math
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import helpers
import plain_zatinex as plain
from test_zatinex import SMALL, YARN, _attention, _config, _gla, _latent, _with_ff

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# max |engine - plain| over max |plain logits|: float32 sums where the plain side has float64;
# bfloat16 rounds activations between the products (the plain side gets the rounded matrices)
TOL = {"float32": 5e-5, "bfloat16": 6e-2}

CONFIGS = {
    "A": SMALL,
    # corners: a key head for every query head, one head, keys as wide as values, every column
    # turning, no interpolation, no convolution, one tap, two taps, tau 1, a gla layer first, a
    # latent layer without a feed-forward, two layers that read one layer's latents, diff 0
    "B": _config(72, 97, [
        _gla(1, 40, 48, 1.0),
        _latent(1, 24, 4, 20, 8, 28, base=50.0),
        _with_ff(_attention(2, 2, 12, 12, rot={"dims": 12, "base": 100.0}, diff=0.0), 20),
        _with_ff(_latent(3, 8, 4, 12, 16, 28, base=50.0, kv_from=1, scale=0.5), 12),
        _attention(3, 1, 20, 8, conv=1, diff=0.7, scale=0.3),
        _latent(2, 16, 4, 8, 9, 28, base=50.0, kv_from=1),
        _with_ff(_attention(1, 1, 16, 40, conv=2, rot={"dims": 2, "base": 7.0, "scaling": {"factor": 2.0, "original": 16, "fast": 4.0, "slow": 1.0}}), 10)],
        eps=1e-3),
    # wider, for bfloat16: heads of 64
    "C": _config(128, 300, [
        _with_ff(_attention(4, 2, 64, 64, conv=3, rot={"dims": 32, "base": 1e4, "scaling": YARN}, diff=0.45), 96),
        _gla(2, 64, 64, 8.0),
        _with_ff(_latent(4, 32, 16, 48, 48, 64, base=1e5), 96),
        _with_ff(_gla(4, 32, 32, 12.0), 64),
        _with_ff(_latent(2, 64, 16, 64, 32, 64, base=1e5, kv_from=2), 64)]),
}
SEEDS = {"A": 3, "B": 4, "C": 5}
RANKS = {"A": 4, "B": 3, "C": 16}


def _folder(path, config, weights):
    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    json.dump(config, open(os.path.join(path, "config.json"), "w"))
    save_file({k: v.contiguous() for k, v in weights.items()}, os.path.join(path, "model.safetensors"))
    return path


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name, config in CONFIGS.items():
        weights = plain.random_weights(config, SEEDS[name], sharp=2.0, decay_rank=RANKS[name])
        out[name] = (_folder(str(tmp_path_factory.mktemp("zat" + name)), config, weights), config, weights)
    return out


def _engine(folder, dtype, n_pages, page_size=16, max_requests=4, **kw):
    from mlx_lm_amd.engine import Engine
    from mlx_lm_amd.utils import load_model

    model, _ = load_model(folder, dtype=dtype)
    return Engine(model, dtype=dtype, page_size=page_size, n_pages=n_pages, max_requests=max_requests, **kw)


def _plain(weights, config, tokens, dtype):
    w = helpers.round_matrices_to_bf16(weights) if dtype == "bfloat16" else weights
    return plain.model(w, config, tokens)


def _close(got, want, dtype, what=""):
    scale = want.abs().max().item()
    err = (got.double().cpu() - want).abs().amax(-1) / scale
    assert err.max().item() <= TOL[dtype], f"{what}: max error {err.max().item():.3e} of the scale at {int(err.argmax())}"


def _run(engine, rid, tokens, cuts):
    from mlx_lm_amd.engine import StepEntry

    engine.add_request(rid)
    rows, i = [], 0
    for n in cuts:
        part = tokens[i : i + n]
        rows.append(engine.step([StepEntry(rid, part, list(range(len(part))))]).clone())
        i += n
    assert i == len(tokens)
    engine.end_request(rid)
    return torch.cat(rows)


def _ints(values):
    return torch.tensor(values, dtype=torch.int32).cuda()


# -- each mechanism's kernels alone -------------------------------------------------------


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_heads_normed_turned_and_placed(dtype):
    """Heads of 12 columns out of a float32 row, normed over all 12 with one weight, the first 8
    turning in pairs (2i, 2i + 1) with interpolated frequencies, written 16 apart in another order."""
    from mlx_lm_amd.ops import kernels
    from mlx_lm_amd.parts.rotary import rotary_table

    g = torch.Generator().manual_seed(0)
    T, H, d, pad = 9, 3, 12, 5
    src = torch.randn(T, pad + H * d + 3, generator=g).cuda()
    w = (1 + 0.3 * torch.randn(d, generator=g)).cuda()
    rot = {"dims": 8, "base": 50.0, "scaling": YARN}
    inv_freq, mult = rotary_table(8, 50.0, YARN, "cuda")
    pos = torch.tensor([0, 1, 2, 700, 701, 5, 6, 7, 8])
    place = [2, 0, 1]
    dst = torch.full((T, H * 16 + 8), 7.0, dtype=dtype, device="cuda")
    kernels.head_prepare(dst, src, pad, H, d, dst_stride=16, dst_fill=16, norm_dim=d, norm_weight=w, eps=1e-4, rot_dims=8,
                         inv_freq=inv_freq, rot_mult=mult, positions=pos.to(torch.int32).cuda(), dst_head=_ints(place))
    heads = src[:, pad : pad + H * d].double().cpu().view(T, H, d)
    f, m = plain.rotary_frequencies(rot)
    want = plain.rotate_pairs(plain.rms_norm(heads, w.double().cpu(), 1e-4), pos, f, m)
    got = dst.double().cpu()[:, : H * 16].view(T, H, 16)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    for h in range(H):
        assert (got[:, place[h], :d] - want[:, h]).abs().max() <= tol
        assert (got[:, place[h], d:] == 0).all()  # the padding is cleared
    assert (dst[:, H * 16 :] == 7.0).all()
    # a part that is normed, beside a part that turns (the latent and the shared key part)
    dst2 = torch.empty(T, 16, dtype=dtype, device="cuda")
    inv4, _ = rotary_table(4, 9.0, None, "cuda")
    kernels.head_prepare(dst2, src, 1, 1, 14, dst_stride=16, dst_fill=16, norm_dim=10, norm_weight=w[:10].contiguous(), eps=1e-4,
                         rot_off=10, rot_dims=4, inv_freq=inv4, positions=pos.to(torch.int32).cuda())
    row = src[:, 1:15].double().cpu()
    f4, _ = plain.rotary_frequencies({"dims": 4, "base": 9.0})
    want2 = torch.cat([plain.rms_norm(row[:, :10], w[:10].double().cpu(), 1e-4), plain.rotate_pairs(row[:, 10:], pos, f4, 1.0)], -1)
    assert (dst2.double().cpu()[:, :14] - want2).abs().max() <= tol and (dst2[:, 14:] == 0).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_two_maps_joined_and_heads_gated(dtype):
    from mlx_lm_amd.ops import kernels

    g = torch.Generator().manual_seed(1)
    T, H, hd, dv = 6, 3, 32, 20
    att = torch.randn(T, 2 * H * hd, generator=g).to(dtype).cuda()
    first, second = [4, 0, 3], [5, 1, 2]
    out = torch.zeros(T, H * dv + 4, dtype=dtype, device="cuda")
    kernels.diff_combine(out, att, hd, _ints(first), _ints(second), 0.37, 0.6, 1e-3, dv)
    a = att.double().cpu().view(T, 2 * H, hd)[..., :dv]
    want = torch.stack([plain.rms_norm(a[:, first[h]] - 0.37 * a[:, second[h]], None, 1e-3) * 0.6 for h in range(H)], 1)
    tol = 1e-5 if dtype == torch.float32 else 3e-2
    assert (out.double().cpu()[:, : H * dv].view(T, H, dv) - want).abs().max() <= tol
    x = torch.randn(T, H * hd, generator=g).to(dtype).cuda()
    gate = torch.randn(T, H + 2, generator=g).cuda()
    before = x.double().cpu().view(T, H, hd)
    kernels.head_gate(x, hd, H, gate[:, 1:])
    want = before * torch.sigmoid(gate[:, 1 : 1 + H].double().cpu())[:, :, None]
    assert (x.double().cpu().view(T, H, hd) - want).abs().max() <= tol


@pytest.mark.parametrize("taps", [1, 2, 4, 7])
def test_the_convolution_on_the_way_into_the_heads(taps):
    """``head_prepare`` with a convolution ahead: two requests in portions of 2, 1, 1, 6 and 3 tokens
    (shorter than the taps, so old inputs stay in the state; single tokens, where the kernel moves
    the state up itself), the first tokens of a request seeing zeros; then the heads' norm."""
    from mlx_lm_amd.ops import kernels

    H, d, n = 3, 10, 13
    C = H * d + 4  # (channels beyond the heads: the state's rows are as wide as the projection)
    g = torch.Generator().manual_seed(taps)
    u = [torch.randn(n, C, generator=g) for _ in range(2)]
    w = torch.randn(C, taps, generator=g)
    nw = 1 + 0.3 * torch.randn(d, generator=g)
    state = torch.zeros(3, 5 + (taps - 1) * C).cuda()
    want = [plain.rms_norm(plain.causal_conv(x.double(), w.double())[:, : H * d].reshape(n, H, d), nw.double(), 1e-4) for x in u]
    at, got = 0, [[], []]
    for m in (2, 1, 1, 6, 3):
        rows = torch.cat([u[0][at : at + m], u[1][at : at + m]]).cuda()
        req, starts, slots = _ints([0] * m + [1] * m), _ints([0, m]), _ints([2, 1])
        conv = kernels.ConvolutionAhead(w.cuda(), state, 5, req, starts, slots, single=m == 1)
        out = torch.empty(2 * m, H * d, device="cuda")
        kernels.head_prepare(out, rows, 0, H, d, norm_dim=d, norm_weight=nw.cuda(), eps=1e-4, conv=conv)
        if m > 1:
            kernels.conv_state_update(rows, 0, taps, C, state, 5, starts, _ints([m, m]), slots, 2)
        got[0].append(out[:m].cpu()), got[1].append(out[m:].cpu())
        at += m
    for r in range(2):
        assert (torch.cat(got[r]).double().view(n, H, d) - want[r]).abs().max() <= 2e-5
    assert (state[0] == 0).all() and (state[:, :5] == 0).all()


def _scan_channels(q, k, v, log_a, S):
    """``S = diag(a_t) S + k_t v_t^T; o_t = S^T q_t`` of one head, float64."""
    out = []
    for t in range(q.shape[0]):
        S = log_a[t].exp()[:, None] * S + k[t][:, None] * v[t][None]
        out.append(S.t() @ q[t])
    return torch.stack(out), S


@pytest.mark.parametrize("chunked", [False, True, "spans"])
@pytest.mark.parametrize("N,P,H", [(8, 8, 4), (24, 16, 2), (5, 24, 3), (64, 64, 2), (40, 48, 1), (128, 128, 1), (6, 10, 2),
                                   (200, 100, 1), (48, 32, 6)])
def test_a_state_that_decays_by_key_channel_in_portions_of_two_requests(N, P, H, chunked):
    """Two requests side by side, three steps; decays given as logits (some so low that a channel
    forgets within a token, some so high that it keeps everything), the output normed with a
    weight and gated.  Token by token, in chunks, and in spans side by side."""
    from mlx_lm_amd.ops import kernels

    g = torch.Generator().manual_seed(N + P)
    lens = [[5, 2], [1, 9], [2, 1]] if not chunked else [[70, 2], [1, 129], [65, 1]]
    n = [sum(x[0] for x in lens), sum(x[1] for x in lens)]
    q = [torch.randn(m, H, N, generator=g).double() for m in n]
    k = [torch.randn(m, H, N, generator=g).double() for m in n]
    v = [torch.randn(m, H, P, generator=g).double() for m in n]
    z = [torch.randn(m, H, N, generator=g).double() * 4 + 2 for m in n]
    for zz in z:
        zz[:, :, 0], zz[:, :, -1] = -60.0, 40.0
    gate = [torch.randn(m, H, P, generator=g).double() for m in n]
    nw = (1 + 0.3 * torch.randn(P, generator=g))
    tau, eps = 2.5, 1e-4
    state = torch.full((4, 7 + H * N * P), 3.0).cuda()
    state[[2, 0], 7:] = 0
    want = []
    for r in range(2):
        heads = []
        for h in range(H):
            log_a = torch.nn.functional.logsigmoid(z[r][:, h]) / tau
            o, _ = _scan_channels(q[r][:, h], k[r][:, h] * N ** -0.5, v[r][:, h], log_a, torch.zeros(N, P, dtype=torch.float64))
            heads.append(plain.rms_norm(o, nw.double(), eps) * gate[r][:, h] * torch.sigmoid(gate[r][:, h]))
        want.append(torch.stack(heads, 1))
    at, got = [0, 0], [[], []]
    for step in lens:
        rows = lambda xs: torch.cat([xs[r][at[r] : at[r] + step[r]].flatten(1) for r in range(2)]).float().cuda()  # noqa: E731
        out = torch.empty(sum(step), H * P, device="cuda")
        spans = None
        if chunked == "spans":
            req, first, lo = [], [], []
            for r_, m_ in enumerate(step):
                first.append(len(req))
                req += [r_] * ((m_ + 63) // 64)
                lo += list(range(0, m_, 64))
            spans = (64, len(req), _ints(req), _ints(lo), _ints(first), lambda shape, dt: torch.empty(shape, dtype=dt, device="cuda"))
        kernels.state_scan(out, rows(q), rows(k), rows(v), state, 7, _ints([0, step[0]]), _ints(step), _ints([2, 0]), 2, H, H, N, P,
                           channel_decay=rows(z), channel_logit_mult=1.0 / tau, k_mult=N ** -0.5, unit_rms=True, eps=eps,
                           norm_weight=nw.cuda(), gate=rows(gate), chunked=bool(chunked), spans=spans)
        got[0].append(out[: step[0]].cpu()), got[1].append(out[step[0] :].cpu())
        at = [at[0] + step[0], at[1] + step[1]]
    for r in range(2):
        w = want[r].flatten(1)
        assert (torch.cat(got[r]).double() - w).abs().max() <= 5e-5 * w.abs().max()
    assert (state[[1, 3]] == 3.0).all() and (state[:, :7] == 3.0).all()


def test_a_token_far_back_in_a_state_that_decays_by_channel():
    """Half of the key channels keep nearly everything and the query of the last of 1,200 tokens
    lies along the key of token 3 on those: the output is that token's value, and the state after
    the last token agrees; the other half forgets quickly."""
    from mlx_lm_amd.ops import kernels

    n, N, P = 1200, 16, 8
    g = torch.Generator().manual_seed(2)
    q, k, v = torch.randn(n, N, generator=g) * 0.1, torch.randn(n, N, generator=g) * 0.01, torch.randn(n, P, generator=g)
    k[3] = torch.randn(N, generator=g) * 3.0
    q[n - 1] = k[3] * 4.0
    log_a = torch.cat([torch.full((n, N // 2), -1.0 / 8192), torch.full((n, N // 2), -0.7)], 1)
    want, S = _scan_channels(q.double(), k.double(), v.double(), log_a.double(), torch.zeros(N, P, dtype=torch.float64))
    lean = (q[n - 1, : N // 2].double() @ k[3, : N // 2].double()) * math.exp(-(n - 4) / 8192)
    assert lean > 10 * (want[n - 1] - lean * v[3].double()).abs().max()
    state = torch.zeros(1, N * P).cuda()
    out = torch.empty(n, P, device="cuda")
    cut = 1190
    for a, b in ((0, cut), (cut, n - 1), (n - 1, n)):
        kernels.state_scan(out[a:b], q[a:b].cuda(), k[a:b].cuda(), v[a:b].cuda(), state, 0, _ints([0]), _ints([b - a]), _ints([0]),
                           1, 1, 1, N, P, channel_decay=log_a[a:b].contiguous().cuda(), chunked=b - a > 8)
    assert (out.double().cpu() - want).abs().max() <= 1e-4 * want.abs().max()
    assert (state.double().cpu().view(N, P) - S).abs().max() <= 1e-4 * S.abs().max()


# -- each mixer alone, in a model of one layer ----------------------------------------------


ALONE = {
    "attention": [_attention(4, 2, 16, 24, conv=3, rot={"dims": 8, "base": 300.0, "scaling": YARN}, diff=0.35)],
    "attention, a head, no convolution": [_attention(1, 1, 8, 8, rot={"dims": 8, "base": 10.0}, diff=0.2, scale=0.7)],
    "attention, seven taps, no rotation": [_attention(6, 2, 24, 16, conv=7, diff=0.6)],
    "gla": [_gla(3, 16, 24, 4.0)],
    "gla, wide": [_gla(2, 80, 40, 1.0)],
    "latent": [_latent(3, 16, 8, 24, 20, 40, base=300.0)],
    "latent and a reader": [_latent(2, 8, 6, 12, 10, 18, base=20.0, scale=0.9), _latent(4, 12, 6, 8, 14, 18, base=20.0, kv_from=0)],
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(ALONE))
def test_a_mixer_alone(tmp_path, name, dtype):
    """Whole, the last tokens one by one, in portions of changing size and of two tokens; portions
    shorter than the convolution's taps among them."""
    config = _config(48, 61, copy.deepcopy(ALONE[name]))
    weights = plain.random_weights(config, 7, sharp=2.0, decay_rank=5)
    folder = _folder(str(tmp_path / "m"), config, weights)
    n = 100
    tokens = helpers.random_tokens(n, 61, seed=len(name))
    want = _plain(weights, config, tokens, dtype)
    eng = _engine(folder, dtype, n_pages=8)
    _close(_run(eng, "whole", tokens, [n]), want, dtype, name + " whole")
    _close(_run(eng, "decoded", tokens, [n - 40] + [1] * 40), want, dtype, name + " decoded")
    _close(_run(eng, "portions", tokens, helpers.cuts_changing(n)), want, dtype, name + " in portions")
    _close(_run(eng, "twos", tokens[:40], [2] * 20), want[:40], dtype, name + " in twos")
    _close(_run(eng, "ones", tokens[:20], [1] * 20), want[:20], dtype, name + " from the first token one by one")
    eng.cache.check()


def test_the_plain_side_notices_what_the_comparisons_are_for(models):
    """With these weights a key head taken for another, the maps swapped, the convolution's taps
    in reverse, a rotation of the wrong layout, a decay per head instead of per channel or a
    reader that makes latents of its own move the logits by far more than the float32 tolerance."""
    _, config, weights = models["A"]
    tokens = helpers.random_tokens(90, config["vocab"], seed=1)
    base = plain.model(weights, config, tokens)
    scale = base.abs().max().item()

    def moved(change):
        c, w = copy.deepcopy(config), dict(weights)
        change(c, w)
        return (plain.model(w, c, tokens) - base)[40:].abs().max().item() / scale

    def key_heads(c, w):
        w["l1.mix.k"] = w["l1.mix.k"].view(3, 2, 16, 64)[[1, 2, 0]].reshape(96, 64)

    def maps(c, w):
        w["l1.mix.q"] = w["l1.mix.q"].view(6, 2, 16, 64)[:, [1, 0]].reshape(192, 64)

    def taps(c, w):
        w["l1.mix.v.conv"] = w["l1.mix.v.conv"].flip(1)

    def decay(c, w):
        w["l2.mix.a2"] = w["l2.mix.a2"].view(2, 24, 4).mean(1, keepdim=True).expand(2, 24, 4).reshape(48, 4)

    def gate(c, w):
        w["l3.mix.g"] = w["l3.mix.g"].flip(0)

    def latents(c, w):
        w["l0.mix.dkv.norm"] = w["l0.mix.dkv.norm"].flip(0)

    for change in (key_heads, maps, taps, decay, gate, latents):
        assert moved(change) > 100 * TOL["float32"], change.__name__


# -- whole, decoded, portions ----------------------------------------------------------


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,n", [("A", 150), ("B", 130), ("C", 200)])
def test_whole_decoded_and_portions(models, dtype, name, n):
    folder, config, weights = models[name]
    tokens = helpers.random_tokens(n, config["vocab"], seed=n)
    want = _plain(weights, config, tokens, dtype)
    eng = _engine(folder, dtype, n_pages=(n + 15) // 16 + 2)
    _close(_run(eng, "whole", tokens, [n]), want, dtype, "whole")
    _close(_run(eng, "decoded", tokens, [n - 90] + [1] * 90), want, dtype, "last 90 one by one")
    _close(_run(eng, "portions", tokens, helpers.cuts_changing(n)), want, dtype, "portions of changing size")
    _close(_run(eng, "twos", tokens[:64], [2] * 32), want[:64], dtype, "portions of two tokens")
    eng.cache.check()
    assert eng.cache.free_pages() == eng.cache.n_pages


def test_portions_give_what_the_whole_prompt_gives(models):
    """However a prompt is cut (at a page's border, one token before and after it, token by
    token), the logits agree with the uncut prompt's to rounding: the engine against itself."""
    folder, config, _ = models["A"]
    tokens = helpers.random_tokens(140, config["vocab"], seed=8)
    eng = _engine(folder, "float32", n_pages=12)
    whole = _run(eng, "w", tokens, [140])
    for cuts in (helpers.cuts_changing(140), [1] * 140, [16, 16, 1, 15, 17, 15, 2, 58], [15, 2, 31, 33, 59], [137, 3]):
        got = _run(eng, "c", tokens, cuts)
        assert (got - whole).abs().max().item() <= 2e-5 * whole.abs().max().item(), cuts[:6]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens_and_long_decode(models, dtype):
    """Every token one by one from the first: 400 of them, recorded decode steps replayed, page
    after page taken, the states carried 400 times."""
    folder, config, weights = models["C"]
    n = 400
    tokens = helpers.random_tokens(n, config["vocab"], seed=77)
    want = _plain(weights, config, tokens, dtype)
    eng = _engine(folder, dtype, n_pages=n // 16 + 1)
    got = _run(eng, "r", tokens, [1] * n)
    _close(got[:8], want[:8], dtype, "first tokens")
    _close(got, want, dtype, "decoding every token")


def _far_model(kind):
    """One mixer and an embedding whose column 0 marks the token ids below 4 (keys to be found) and
    whose column 1 marks the ids 4 to 7 (queries that look for them); only position 3 and the last
    carry such ids."""
    if kind == "attention":
        layers = [_attention(2, 1, 16, 16, diff=0.25, scale=1.0)]
    else:
        layers = [_latent(2, 16, 4, 16, 12, 24, base=1e4, scale=1.0)]
    config = _config(32, 40, layers)
    w = plain.random_weights(config, 11, sharp=1.0)
    w["embed"][:8] *= 0.05
    w["embed"][:, :2] = 0.0
    w["embed"][:4, 0], w["embed"][4:8, 1] = 6.0, 6.0
    return config, w


@pytest.mark.parametrize("kind", ["attention", "latent"])
def test_a_key_far_back(tmp_path, kind):
    """900 tokens; the scores of the marked tokens stand out (the marking column is scaled in the
    query and key projections), so the last position reads position 3 among hundreds: in a prompt,
    in a portion's last row, and decoded alone."""
    config, w = _far_model(kind)
    p = "l0.mix."
    if kind == "attention":
        for name, col in (("q", 1), ("k", 0)):
            w[p + name][:, :2] = 0.0
            w[p + name][0::16, col] = 3.0  # the first column of every map of every head follows the mark
        w[p + "q.b"][:] = 0
        w[p + "k.b"][:] = 0
        w[p + "q.norm"][:], w[p + "k.norm"][:] = 1.0, 1.0
        w[p + "q.norm"][0] = 6.0
    else:
        w[p + "dq"][:, :2], w[p + "dkv"][:, :2] = 0.0, 0.0
        w[p + "dq"][0, 1], w[p + "dkv"][0, 0] = 3.0, 3.0
        w[p + "uq"][:, 0], w[p + "uk"][:, 0] = 0.0, 0.0
        w[p + "uq"][0::20, 0], w[p + "uk"][0::16, 0] = 4.0, 4.0
    n = 900
    tokens = [8 + t for t in helpers.random_tokens(n, 32, seed=5)]
    tokens[3], tokens[n - 1] = 2, 5
    want = plain.model(w, config, tokens)
    other = list(tokens)
    other[3] = 20  # without the marked token the last position reads something else
    moved = (plain.model(w, config, other)[n - 1] - want[n - 1]).abs().max() / want.abs().max()
    assert moved > 0.05, float(moved)
    folder = _folder(str(tmp_path / "m"), config, w)
    eng = _engine(folder, "float32", n_pages=n // 16 + 2)
    for cuts in ([n], [n - 7, 7], [n - 1, 1], [500, 2, 397, 1]):
        got = _run(eng, "r", tokens, cuts)
        _close(got[n - 1 :], want[n - 1 :], "float32", f"{kind}: the last of {cuts}")
        _close(got, want, "float32", f"{kind}: {cuts}")


# -- batches -------------------------------------------------------------------------------


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_mixed_batches_equal_each_request_alone(models, dtype, name):
    """Up to four live requests of unequal lengths, portions beside single tokens, requests that
    sit a step out; state rows (the decaying states, the convolutions' last inputs) and pages of
    finished requests are used again by later ones, and what freed pages hold is never read."""
    from mlx_lm_amd.engine import StepEntry

    folder, config, weights = models[name]
    lengths = [70, 9, 131, 40, 3, 97, 55]
    tokens, steps = helpers.mixed_trace({"vocab_size": config["vocab"]}, 21, lengths, n_live=4)
    eng = _engine(folder, dtype, n_pages=helpers.held(lengths, 4) // 16, max_requests=4)
    got = {rid: [] for rid in tokens}
    for s in steps:
        entries = []
        for e in s["entries"]:
            if not eng.has_request(e["id"]):
                eng.add_request(e["id"])
            entries.append(StepEntry(e["id"], e["tokens"], e["want"]))
        logits = eng.step(entries).clone()
        at = 0
        for e in entries:
            got[e.request_id].append(logits[at : at + len(e.want)])
            at += len(e.want)
        for rid in s["end"]:
            eng.end_request(rid)
        eng.cache.poison_free_pages()
    for rid, toks in tokens.items():
        _close(torch.cat(got[rid]), _plain(weights, config, toks, dtype), dtype, f"request {rid} in mixed batches")
    eng.cache.check()
    assert eng.cache.free_pages() == eng.cache.n_pages


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_twenty_requests_decode_together(models, dtype):
    from mlx_lm_amd.engine import StepEntry

    folder, config, weights = models["C"]
    lengths = [5 + 7 * i for i in range(20)]
    tokens = [helpers.random_tokens(n + 12, config["vocab"], seed=200 + n) for n in lengths]
    eng = _engine(folder, dtype, n_pages=sum((n + 12 + 15) // 16 for n in lengths), max_requests=20)
    for i, (n, toks) in enumerate(zip(lengths, tokens)):
        eng.add_request(i)
        eng.step([StepEntry(i, toks[:n], [])])
    got = [[] for _ in lengths]
    for step in range(12):
        logits = eng.step([StepEntry(i, [tokens[i][n + step]], [0]) for i, n in enumerate(lengths)]).clone()
        for i in range(len(lengths)):
            got[i].append(logits[i])
    for i, n in enumerate(lengths):
        _close(torch.stack(got[i]), _plain(weights, config, tokens[i], dtype)[n:], dtype, f"request {i} among twenty")


def _drawn_config(seed):
    g = torch.Generator().manual_seed(seed)

    def pick(options):
        return options[int(torch.randint(0, len(options), (), generator=g))]

    layers, latents = [], []
    for i in range(pick([1, 2, 3, 4, 5])):
        kind = pick(["attention", "gla", "latent"])
        if kind == "attention":
            kv, dim = pick([1, 2, 3]), pick([8, 12, 16, 32, 40, 64])
            rot = pick([None, dim, dim // 2 // 2 * 2, 2])
            rot = {"dims": rot, "base": pick([10.0, 1e4, 1e6])} if rot else None
            if rot and pick([0, 1]):
                rot["scaling"] = {"factor": pick([2.0, 4.0, 16.0]), "original": pick([16, 64, 512]), "fast": pick([8.0, 32.0]), "slow": pick([1.0, 2.0])}
            entry = _attention(kv * pick([1, 2, 4]), kv, dim, pick([8, 16, 24, 48, 80]), conv=pick([None, 1, 2, 3, 4, 5]), rot=rot,
                               diff=pick([0.0, 0.2, 0.5, 0.8]), scale=pick([None, 0.05, 0.4]))
        elif kind == "gla":
            heads, vdim = pick([1, 2, 4]), pick([8, 16, 32, 40])
            entry = _gla(heads, pick([8, 16, 24, 32, 64]), vdim, pick([1.0, 2.0, 16.0, 64.0]))
        else:
            reads = pick(latents + [None]) if latents else None
            if reads is not None:
                src = layers[reads]["mixer"]
                entry = _latent(pick([1, 2, 4]), pick([8, 16, 24]), src["rot_dim"], pick([8, 16, 40]), pick([8, 12, 32]), src["kv_rank"],
                                base=src["rot"]["base"], kv_from=reads, scale=pick([None, 0.3]))
            else:
                entry = _latent(pick([1, 2, 4]), pick([8, 16, 24]), pick([2, 4, 8, 16]), pick([8, 16, 40]), pick([8, 12, 32]),
                                pick([8, 20, 48, 64]), base=pick([10.0, 1e4, 1e6]), scale=pick([None, 0.3]))
                latents.append(i)
        if pick([0, 1, 1]):
            entry = _with_ff(entry, pick([4, 8, 20, 64]))
        layers.append(entry)
    return _config(pick([16, 40, 64, 104, 256]), pick([17, 100, 257, 1000]), layers, eps=pick([1e-6, 1e-5, 1e-2]))


@pytest.mark.parametrize("seed", range(10))
def test_drawn_configurations(tmp_path, seed):
    """Every size, the layers' order and constants drawn: whole, in portions, and two requests
    side by side, in float32."""
    from mlx_lm_amd.engine import StepEntry

    config = _drawn_config(seed)
    weights = plain.random_weights(config, 100 + seed, sharp=2.0, decay_rank=1 + seed % 7)
    folder = _folder(str(tmp_path / "m"), config, weights)
    a, b = helpers.random_tokens(120, config["vocab"], seed=seed), helpers.random_tokens(75, config["vocab"], seed=50 + seed)
    wa, wb = plain.model(weights, config, a), plain.model(weights, config, b)
    eng = _engine(folder, "float32", n_pages=16)
    _close(_run(eng, "whole", a, [120]), wa, "float32", f"seed {seed} whole: {json.dumps(config)}")
    eng.add_request("a"), eng.add_request("b")
    ga, gb, ia, ib = [], [], 0, 0
    for ca, cb in ((50, 2), (1, 40), (1, 1), (38, 1), (2, 30), (28, 1)):
        out = eng.step([StepEntry("a", a[ia : ia + ca], list(range(ca))), StepEntry("b", b[ib : ib + cb], list(range(cb)))]).clone()
        ga.append(out[:ca]), gb.append(out[ca:])
        ia, ib = ia + ca, ib + cb
    _close(torch.cat(ga), wa, "float32", f"seed {seed}, first of two")
    _close(torch.cat(gb), wb, "float32", f"seed {seed}, second of two")


def test_recorded_steps_equal_eager_steps(models):
    """Decode steps replayed from recorded graphs against the same steps run eagerly, bit for bit."""
    from mlx_lm_amd.engine import StepEntry

    folder, config, _ = models["A"]
    seqs = {"a": helpers.random_tokens(60, config["vocab"], 1), "b": helpers.random_tokens(45, config["vocab"], 2)}
    results = {}
    for use_graphs in (True, False):
        eng = _engine(folder, "bfloat16", n_pages=10, use_graphs=use_graphs)
        assert eng.use_graphs == use_graphs  # every part launches kernels only
        for r in seqs:
            eng.add_request(r)
        out = [eng.step([StepEntry("a", seqs["a"][:20], [19]), StepEntry("b", seqs["b"][:5], [4])]).clone()]
        for i in range(40):
            out.append(eng.step([StepEntry("a", [seqs["a"][20 + i]], [0]), StepEntry("b", [seqs["b"][5 + i]], [0])]).clone())
        if use_graphs:
            assert helpers.decode_graphs(eng, 2)[0].graph is not None
        results[use_graphs] = torch.cat(out)
    assert torch.equal(results[True], results[False])


# -- generation through the entry points -----------------------------------------------------


def test_greedy_generation_through_the_scheduler(models):
    from mlx_lm_amd import batch_generate, load, stream_generate

    folder, config, weights = models["A"]
    model, tok = load(folder, dtype="float32")
    prompts = [helpers.random_tokens(n, config["vocab"], seed=n) for n in (23, 5, 61)]
    want = [plain.greedy(weights, config, p, 10) for p in prompts]
    got = [r.token for r in stream_generate(model, tok, prompts[0], max_tokens=10, prefill_step_size=7)]
    assert got == want[0]
    batch = batch_generate(model, tok, prompts, max_tokens=10)
    assert [[int(t) for t in text.split()] for text in batch.texts] == want


def test_command_line_and_trace_replay(tmp_path, models):
    """``python -m mlx_lm_amd generate`` on a folder of this design, and the replay program on that
    folder: a prompt in two steps beside a second request that starts later."""
    folder, config, weights = models["B"]
    prompt = [3, 1, 4, 1, 5, 9, 2, 6]
    want = plain.greedy(weights, config, prompt, 25)
    env = dict(os.environ, PYTHONPATH=ROOT)
    out = subprocess.run(
        [sys.executable, "-m", "mlx_lm_amd", "generate", "--model", folder, "--prompt-ids", ",".join(map(str, prompt)),
         "--max-tokens", "25", "--dtype", "float32", "--verbose", "F", "--num-pages", "8", "--prefill-step-size", "3"],
        capture_output=True, text=True, env=env, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    assert out.stdout.strip() == " ".join(map(str, want))
    a, b = helpers.random_tokens(50, config["vocab"], seed=9), helpers.random_tokens(20, config["vocab"], seed=10)
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": a[:31], "want": [30]}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": a[31:], "want": [0, 18]}, {"id": "y", "tokens": b, "want": [19]}], "end": ["x", "y"]}]
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32",
                           "--out", str(tmp_path / "out"), "--max-tokens", "128"],
                          input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert "done 0" in proc.stdout and "done 1" in proc.stdout
    wa, wb = plain.model(weights, config, a), plain.model(weights, config, b)
    first = np.fromfile(tmp_path / "out" / "0.f32", dtype="<f4").reshape(-1, config["vocab"])
    second = np.fromfile(tmp_path / "out" / "1.f32", dtype="<f4").reshape(-1, config["vocab"])
    _close(torch.from_numpy(first), wa[30:31], "float32", "the replay's first step")
    _close(torch.from_numpy(second), torch.stack([wa[31], wa[49], wb[19]]), "float32", "the replay's second step")
