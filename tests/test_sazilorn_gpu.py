"""Sazilorn in the engine against the plain implementation (plain_sazilorn.py): each mechanism's
kernels, each mixer alone in a one-layer model, whole prompts, decoding, portions, mixed batches,
reused pages and state rows, far tokens, the edges of the distance buckets, generation through the
entry points."""

import copy
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import helpers
import plain_sazilorn as plain
from test_pafutar_gpu import _paged
from test_sazilorn import SMALL, _attention, _config, _dense, _hgrn2, _moe, _parallel, _softmax

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# max |engine - plain| over max |plain logits|: float32 sums where the plain side has float64;
# bfloat16 rounds activations between the products (the plain side gets the rounded matrices)
TOL = {"float32": 5e-5, "bfloat16": 6e-2}

CONFIGS = {
    "A": SMALL,
    # corners: one head, a key head for every query head, keys wider and narrower than values, one
    # tap, an expert a token of two, no shared expert, a decay of one, a table of two rows reaching
    # to 3, a table that reaches beyond the positions, scales of 1, a layer without a feed-forward
    "B": _config(72, 97, 300, 1, [
        _attention(1, 1, 40, 8, 2, 3, scale=1.0),
        _moe(_parallel(_softmax(3, 3, 12, 20, softcap=1.0), 2, 12, 40, [1.0, 0.25], left_scale=1.0, right_scale=1.0), 2, 1, 8, scale=1.0),
        _hgrn2(1, 40, 8),
        _dense(_attention(4, 2, 8, 24, 7, 1000), 12),
        _moe(_hgrn2(3, 8, 24), 4, 4, 12, shared=20)], eps=1e-3),
    # wider, for bfloat16: heads of 64
    "C": _config(128, 300, 512, 2, [
        _dense(_parallel(_softmax(4, 2, 64, 64, softcap=15.0), 2, 64, 32, [0.7, 0.995]), 96),
        _moe(_hgrn2(2, 32, 64), 6, 2, 32, shared=32, scale=1.7),
        _dense(_attention(4, 2, 64, 64, 24, 100), 96),
        _moe(_parallel(_softmax(2, 1, 64, 32, softcap=30.0), 4, 16, 16, [0.9, 0.95, 0.99, 0.5]), 4, 2, 48),
        _hgrn2(4, 16, 32)]),
}
SEEDS = {"A": 3, "B": 4, "C": 5}


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
        weights = plain.random_weights(config, SEEDS[name], sharp=2.0)
        out[name] = (_folder(str(tmp_path_factory.mktemp("saz" + name)), config, weights), config, weights)
    return out


def _engine(folder, dtype, n_pages, page_size=16, max_requests=4, **kw):
    from mlx_lm_amd.engine import Engine
    from mlx_lm_amd.utils import load_model

    model, _ = load_model(folder, dtype=dtype)
    return Engine(model, dtype=dtype, page_size=page_size, n_pages=n_pages, max_requests=max_requests, **kw)


def _rounded(weights, config):
    """What the engine's bfloat16 path holds: the tensors it keeps as matrices rounded, the others as they are."""
    from mlx_lm_amd.config import get_model_classes

    Model, Args = get_model_classes(config)
    roles = Model(Args.from_dict(config)).decoder.expected_tensors()
    return {k: v.to(torch.bfloat16).float() if roles[k].role == "matrix" else v for k, v in weights.items()}


CLOSE_CALL = 0.01  # a choice score this near the next one's may fall the other way once activations are rounded to bfloat16


class _Want:
    """The plain logits of a sequence and, for bfloat16, the positions at which some layer's choice
    of experts is a close call: there the rounded engine may rightly choose otherwise, which moves
    that position's logits by far more than rounding, so such positions are not compared."""

    def __init__(self, logits, sure):
        self.logits, self.sure = logits, sure

    def __getitem__(self, rows):
        return _Want(self.logits[rows], self.sure[rows])


def _plain(weights, config, tokens, dtype):
    if dtype != "bfloat16":
        return plain.model(weights, config, tokens)
    margins = []
    logits = plain.model(_rounded(weights, config), config, tokens, margins=margins)
    sure = torch.ones(len(tokens), dtype=torch.bool)
    for m in margins:
        sure &= m > CLOSE_CALL
    assert sure.any() and (len(tokens) < 50 or sure.float().mean() > 0.5), "most positions are compared"
    return _Want(logits, sure)


def _close(got, want, dtype, what=""):
    sure = None
    if isinstance(want, _Want):
        want, sure = want.logits, want.sure
    scale = want.abs().max().item()
    err = (got.double().cpu() - want).abs().amax(-1) / scale
    if sure is not None:
        err = err[sure]
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


# -- each mechanism's kernels alone -------------------------------------------------------


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [64, 200, 1032, 2304, 8200])
def test_one_norm_and_the_streams_copies(width, dtype):
    from mlx_lm_amd.ops import kernels

    g = torch.Generator().manual_seed(width)
    x = (torch.randn(7, width + 8, generator=g) * 3).cuda()[:, :width]  # (rows further apart than they are wide)
    w = (1 + 0.2 * torch.randn(width, generator=g)).cuda()
    out = torch.empty(7, width, dtype=dtype, device="cuda")
    out32, a, b = (torch.empty(7, width, device="cuda") for _ in range(3))
    kernels.norm_fanout(out, x, w, 1e-3, out32=out32, copy_a=a, copy_b=b)
    want = plain.rms_norm(x.double().cpu(), w.double().cpu(), 1e-3)
    assert (out32.double().cpu() - want).abs().max() <= 1e-5 * want.abs().max()
    assert (out.double().cpu() - want).abs().max() <= (1e-5 if dtype == torch.float32 else 1e-2) * want.abs().max()
    assert torch.equal(a, x) and torch.equal(b, x)
    kernels.norm_fanout(out, x, w, 1e-3)  # (every extra output is optional)
    assert (out.double().cpu() - want).abs().max() <= (1e-5 if dtype == torch.float32 else 1e-2) * want.abs().max()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("taps,width", [(1, 64), (2, 72), (4, 1032), (7, 2304)])
def test_the_convolution_on_the_mixers_input_across_steps(taps, width, dtype):
    """Two requests in state rows 3 and 1 (behind 5 floats of someone else's): a portion of each, a
    second portion shorter than the taps, then tokens one by one, in which the norm's kernel runs the
    convolution and moves the state itself; against ``h + conv(h)`` over each whole sequence."""
    from mlx_lm_amd.ops import kernels

    g = torch.Generator().manual_seed(taps)
    lens, offset = [9 + taps, 12], 8
    x = [torch.randn(n + 6, width, generator=g) * 2 for n in lens]
    gamma = 1 + 0.2 * torch.randn(width, generator=g)
    w = torch.randn(width, taps, generator=g) * 0.5
    want = []
    for xs in x:
        h = plain.rms_norm(xs.double(), gamma.double(), 1e-4)
        want.append(h + plain.causal_conv(h, w.double()))
    state = torch.zeros(5, offset + (taps - 1) * width + 3, device="cuda")
    slot_ids = torch.tensor([3, 1], dtype=torch.int32).cuda()
    got, fed = [[], []], [0, 0]
    for cuts in ((lens[0] - 2, lens[1] - 3), (2, 3), (1, 1), (1, 1), (1, 1), (1, 1), (1, 1), (1, 1)):
        rows = torch.cat([x[r][fed[r]:fed[r] + n] for r, n in enumerate(cuts)]).cuda()
        T = rows.shape[0]
        token_req = torch.tensor([r for r, n in enumerate(cuts) for _ in range(n)], dtype=torch.int32).cuda()
        starts = torch.tensor([0, cuts[0]], dtype=torch.int32).cuda()
        seq_lens = torch.tensor(list(cuts), dtype=torch.int32).cuda()
        out, mixed = torch.empty(T, width, dtype=dtype, device="cuda"), torch.empty(T, width, dtype=dtype, device="cuda")
        canon = kernels.InputConvolution(w.cuda(), state, offset, token_req, starts, slot_ids, mixed)
        if max(cuts) == 1:
            kernels.norm_fanout(out, rows, gamma.cuda(), 1e-4, canon=canon)
        else:
            h32 = torch.empty(T, width, device="cuda")
            kernels.norm_fanout(out, rows, gamma.cuda(), 1e-4, out32=h32)
            kernels.canon_rows(h32, canon)
            if taps > 1:
                kernels.conv_state_update(h32, 0, taps, width, state, offset, starts, seq_lens, slot_ids, 2)
        at = 0
        for r, n in enumerate(cuts):
            got[r].append(mixed[at:at + n].double().cpu())
            at, fed[r] = at + n, fed[r] + n
    for r in range(2):
        err = (torch.cat(got[r]) - want[r]).abs().max() / want[r].abs().max()
        assert err <= (1e-5 if dtype == torch.float32 else 1e-2), (r, float(err))
    assert (state[[0, 2, 4]] == 0).all() and (state[:, :offset] == 0).all() and (state[:, offset + (taps - 1) * width:] == 0).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_norm_over_all_heads_as_they_are_placed(dtype):
    """Heads of 12 columns normed over the whole projection of 5 heads (a weight for every column),
    written 16 apart; beside heads that are only placed."""
    from mlx_lm_amd.ops import kernels

    g = torch.Generator().manual_seed(3)
    T, H, d, pad = 7, 5, 12, 4
    src = (torch.randn(T, pad + H * d + 9, generator=g) * 3).cuda()
    w = (1 + 0.3 * torch.randn(H * d, generator=g)).cuda()
    dst = torch.full((T, H * 16 + 8), 7.0, dtype=dtype, device="cuda")
    plainly = torch.full((T, 16), 7.0, dtype=dtype, device="cuda")
    kernels.head_prepare_many((dst, src, pad, H, d, dict(dst_stride=16, dst_fill=16, norm_whole=H * d, norm_weight=w, eps=1e-3)),
                              (plainly, src, pad + H * d, 1, 9, dict(dst_stride=16, dst_fill=16)))
    want = plain.rms_norm(src[:, pad:pad + H * d].double().cpu(), w.double().cpu(), 1e-3).view(T, H, d)
    got = dst.double().cpu()[:, :H * 16].view(T, H, 16)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert (got[:, :, :d] - want).abs().max() <= tol * want.abs().max() and (got[:, :, d:] == 0).all()
    assert (dst[:, H * 16:] == 7.0).all()
    assert (plainly.double().cpu()[:, :9] - src[:, pad + H * d:].double().cpu()).abs().max() <= tol * 10


@pytest.mark.parametrize("n", [1, 2, 7, 33])
def test_the_sum_over_depth(n):
    from mlx_lm_amd.ops import kernels

    g = torch.Generator().manual_seed(n)
    kept = torch.randn(n + 2, 11, 72, generator=g).cuda()
    a = torch.randn(n, generator=g).cuda()
    out = torch.full((11, 72), 9.0, device="cuda")
    kernels.depth_average(out, kept, a, n)
    want = torch.einsum("j,jtc->tc", a.double().cpu(), kept[:n].double().cpu())
    assert (out.double().cpu() - want).abs().max() <= 1e-5 * want.abs().max()


def test_activations_gates_and_the_norm_over_all_heads():
    from mlx_lm_amd.ops import kernels

    g = torch.Generator().manual_seed(0)
    T, n, cols = 9, 44, 150
    u0 = (torch.randn(T, cols, generator=g) * 3)
    u = u0.clone().cuda()
    kernels.silu_columns(u, 5, 71)
    want = u0.double().clone()
    want[:, 5:76] = plain.silu(want[:, 5:76])
    assert (u.double().cpu() - want).abs().max() <= 1e-6
    # the forget gate with its floor: logits of -30 .. 30, floors from 0 to nearly 1
    u0[:, 60:60 + n] = torch.linspace(-30, 30, T * n).view(T, n)
    lower = torch.cat([torch.tensor([0.0, 0.999999]), torch.rand(n - 2, generator=g)])
    u = u0.clone().cuda()
    keys = torch.zeros(T, n + 3, device="cuda")[:, :n]
    kernels.forget_gate(u, 3, 60, n, lower.cuda(), keys)
    f = lower.double() + (1 - lower.double()) * torch.sigmoid(u0[:, 60:60 + n].double())
    assert (keys.double().cpu() - (1 - f)).abs().max() <= 1e-7
    rest = (1 - lower.double()) * torch.sigmoid(-u0[:, 60:60 + n].double())  # 1 - f, written without the difference
    assert ((keys.double().cpu() - rest).abs() / rest).max() <= 1e-5  # (no cancellation where f is close to one)
    assert ((u[:, 60:60 + n].double().cpu() - f.log()).abs() / (1 + f.log().abs())).max() <= 2e-7
    assert (u[:, 3:3 + n].double().cpu() - plain.silu(u0[:, 3:3 + n].double())).abs().max() <= 1e-6
    assert torch.equal(u[:, :3].cpu(), u0[:, :3]) and torch.equal(u[:, 60 + n:].cpu(), u0[:, 60 + n:])
    # one norm over the whole row, then the sigmoid gate
    y, gate, w = torch.randn(T, 100, generator=g) * 5, torch.randn(T, 100, generator=g) * 2, 1 + 0.3 * torch.randn(100, generator=g)
    want = plain.rms_norm(y.double(), w.double(), 1e-4) * torch.sigmoid(gate.double())
    for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 1e-2)):
        out = torch.zeros(T, 104, dtype=dtype, device="cuda")
        kernels.normed_gate(out[:, :100], y.cuda(), gate.cuda(), w.cuda(), 1e-4)
        assert (out[:, :100].double().cpu() - want).abs().max() <= tol * want.abs().max()
        assert (out[:, 100:] == 0).all()


@pytest.mark.parametrize("n_out,top", [(8, 3), (5, 1), (3, 3), (70, 6), (200, 70)])
def test_the_routers_weights_renormalised_and_scaled(n_out, top):
    from mlx_lm_amd.ops import kernels

    g = torch.Generator().manual_seed(n_out)
    T = 13
    z = torch.randn(T, n_out, generator=g) * 2
    corr = torch.randn(n_out, generator=g) * 0.1
    idx = torch.zeros(T, top, dtype=torch.int32, device="cuda")
    weight = torch.zeros(T, top, device="cuda")
    kernels.router_choice(idx, weight, z.cuda(), corr.cuda(), top, renormalize=True, weight_scale=2.5)
    s = torch.softmax(z.double(), -1)
    want_idx = torch.topk(s + corr.double(), top, dim=-1).indices
    picked = torch.gather(s, 1, want_idx)
    want = picked / (picked.sum(-1, keepdim=True) + 1e-20) * 2.5
    assert torch.equal(idx.cpu().long(), want_idx)
    assert (weight.double().cpu() - want).abs().max() <= 1e-6
    # the same in the launch that also makes the shared expert's activations
    F = 24
    zu = torch.cat([z, torch.randn(T, 2 * F, generator=g)], 1).cuda()
    act = torch.empty(T, F, device="cuda")
    kernels.route_and_gate(idx.zero_(), weight.zero_(), act, zu, corr.cuda(), top, n_out, renormalize=True, weight_scale=2.5)
    assert torch.equal(idx.cpu().long(), want_idx) and (weight.double().cpu() - want).abs().max() <= 1e-6
    assert (act.double().cpu() - plain.silu(zu[:, n_out:n_out + F].double().cpu()) * zu[:, n_out + F:].double().cpu()).abs().max() <= 1e-5
    # not renormalised, as before
    kernels.router_choice(idx, weight, z.cuda(), corr.cuda(), top)
    assert (weight.double().cpu() - picked).abs().max() <= 1e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_the_gate_through_the_tanh_form_of_gelu(dtype):
    from mlx_lm_amd.ops import kernels

    g = torch.Generator().manual_seed(1)
    gu = (torch.randn(6, 2 * 40, generator=g) * 3).to(dtype)
    out = torch.empty(6, 40, dtype=dtype, device="cuda")
    kernels.silu_mul(out, gu.cuda(), "gelu_tanh")
    want = plain.gelu_tanh(gu[:, :40].double()) * gu[:, 40:].double()
    assert (out.double().cpu() - want).abs().max() <= (1e-5 if dtype == torch.float32 else 2e-2) * want.abs().max()
    kernels.silu_mul(out, gu.cuda())
    want = plain.silu(gu[:, :40].double()) * gu[:, 40:].double()
    assert (out.double().cpu() - want).abs().max() <= (1e-5 if dtype == torch.float32 else 2e-2) * want.abs().max()


@pytest.mark.parametrize("kernel,dtype,d", [("tile", torch.float32, 48), ("tile", torch.bfloat16, 24), ("row", torch.float32, 40),
                                            ("row", torch.bfloat16, 80), ("prefill", torch.bfloat16, 64),
                                            ("prefill", torch.bfloat16, 128), ("prefill", torch.bfloat16, 32),
                                            ("prefill", torch.bfloat16, 256), ("decode", torch.bfloat16, 64),
                                            ("decode", torch.float32, 64), ("decode", torch.bfloat16, 128)])
@pytest.mark.parametrize("softcap,rows,far", [(5.0, 0, 0), (0.0, 12, 50), (0.0, 32, 520.0), (2.0, 7, 1000), (0.0, 2, 3)])
def test_attention_kernels_with_capped_scores_and_a_distance_table(kernel, dtype, d, softcap, rows, far):
    """Queries at positions 530 .. of a request that holds 530 + n keys; scores capped, a term by
    bucketed distance added, a gate on the output.  Keys that stand out for the first query: one
    far back among hundreds, and the first and the last distance of a bucket in the table's
    logarithmic part (taken for the neighbouring bucket, either moves the output)."""
    from mlx_lm_amd.ops import kernels

    H, G, offset = 4, 2, 530
    n_q = {"tile": 16, "row": 3, "prefill": 150, "decode": 3}[kernel]
    n = offset + n_q
    g = torch.Generator().manual_seed(d + rows + int(softcap))
    q = torch.randn(n_q, H, d, generator=g).to(dtype)
    k = torch.randn(n, G, d, generator=g).to(dtype)
    v = torch.randn(n, G, d, generator=g).to(dtype)
    gate = torch.randn(n_q, H * d, generator=g).to(dtype)
    scale = 1.0 / d**0.5
    stand_out = [2]
    table = None
    if rows:
        rel = torch.randn(rows, H, generator=g) * 2.0
        buckets = [plain.distance_bucket(m, rows, far) for m in range(n)]
        table = torch.stack([rel[b] for b in buckets]).t().contiguous()[:, : min(n, int(far) + 1)]
        # distances from the first query at which the bucket changes, in the logarithmic part
        edges = [m for m in range(rows // 2 + 1, offset) if buckets[m] != buckets[m - 1]]
        for m in edges[-2:]:
            stand_out += [offset - m, offset - m + 1]
    for j in stand_out:
        k[j, G - 1] = (q[0, H - 1].float() * (1.5 if not softcap else 3.0)).to(dtype)
    s = torch.einsum("ihd,jhd->hij", q.double(), k.double().repeat_interleave(H // G, dim=1)) * scale
    if softcap:
        s = softcap * torch.tanh(s / softcap)
    i, j = torch.arange(n_q)[:, None] + offset, torch.arange(n)[None, :]
    if rows:
        full = torch.stack([rel[b] for b in buckets]).t().double()  # [H, distance]
        s = s + full[:, (i - j).clamp(min=0)]
    p = torch.softmax(s.masked_fill((j > i).unsqueeze(0), float("-inf")), dim=-1)
    want = torch.einsum("hij,jhd->ihd", p, v.double().repeat_interleave(H // G, dim=1)).reshape(n_q, H * d)
    want = want * torch.sigmoid(gate.double())
    if not rows:
        assert p[H - 1, 0, 2] > 0.02  # the first query reads the far key (capped: among others of the cap's height)

    kv, block_table = _paged(k, v, 16, dtype, seed=d)
    qd = q.reshape(n_q, H * d).cuda()
    out = torch.empty_like(qd)
    zeros = torch.zeros(n_q, dtype=torch.int32, device="cuda")
    positions = (torch.arange(n_q, dtype=torch.int32) + offset).cuda()
    terms = kernels.ScoreTerms(gate=gate.cuda(), softcap=softcap, distance_bias=table.cuda() if rows else None)
    items = torch.arange(n_q, dtype=torch.int32).cuda()
    if kernel == "tile":
        tiles = torch.tensor([[0, n_q]], dtype=torch.int32).cuda()
        kernels.attn_tile(out, qd, kv, block_table, zeros, positions, tiles, 1, H, scale, 0, terms)
    elif kernel == "prefill":
        tiles = torch.tensor([[128, n_q - 128], [0, 128]], dtype=torch.int32).cuda()
        kernels.attn_prefill(out, qd, kv, block_table, zeros, positions, tiles, 2, H, scale, 0, terms)
    else:
        n_splits = 3
        part_o = torch.empty(n_q * H * n_splits * d, device="cuda")
        part_ml = torch.empty(n_q * H * n_splits * 2, device="cuda")
        if kernel == "row":
            kernels.attn_row(out, qd, kv, block_table, zeros, positions, items, n_q, H, scale, 0, n_splits, part_o, part_ml, terms)
        else:
            kernels.attn_decode(out, qd, kv, block_table, zeros, positions, items, n_q, H, scale, 0, n_splits, part_o, part_ml,
                                n_waves=4, join_in_kernel=2, terms=terms)
    err = (out.double().cpu() - want).abs().max().item()
    assert err <= (2e-5 if dtype == torch.float32 else 2.5e-2) * want.abs().max().item(), err


# -- each mixer alone in a one-layer model ---------------------------------------------------


ALONE = {
    "parallel": _parallel(_softmax(4, 2, 16, 24, softcap=4.0), 3, 8, 16, [0.5, 0.97, 0.9]),
    "parallel_wide": _dense(_parallel(_softmax(2, 1, 64, 64, softcap=50.0, scale=0.2), 2, 64, 64, [0.8, 0.999]), 32),
    # (sizes that are multiples of nothing: the state row's floats behind the convolution's start anywhere)
    "parallel_odd": _parallel(_softmax(3, 1, 10, 6, softcap=2.0), 1, 5, 3, [0.7]),
    "parallel_odder": _parallel(_softmax(1, 1, 5, 6, softcap=2.0), 1, 5, 3, [0.7]),  # (the right one's columns start at 22)
    "hgrn2": _hgrn2(3, 24, 16),
    "hgrn2_odd": _hgrn2(1, 5, 3),
    "hgrn2_experts": _moe(_hgrn2(2, 64, 64), 6, 2, 24, shared=8),
    "attention": _attention(6, 2, 16, 24, 10, 40),
    "attention_dense": _dense(_attention(2, 2, 64, 32, 33, 90.5, scale=0.3), 40),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(ALONE))
def test_a_mixer_alone(tmp_path, name, dtype):
    """One layer: whole, the last tokens one by one, and portions; 300 tokens, so that the
    recurrences run in chunks and spans and the prompt's attention in large tiles."""
    if "_odd" in name and dtype == "bfloat16":
        pytest.skip("a norm over three columns turns bfloat16's rounding into errors of any size: float32 only")
    config = _config(64, 90, 320, 3, [copy.deepcopy(ALONE[name])])
    weights = plain.random_weights(config, 7, sharp=2.0)
    folder = _folder(str(tmp_path / "m"), config, weights)
    n = 300
    tokens = helpers.random_tokens(n, config["vocab"], seed=1)
    want = _plain(weights, config, tokens, dtype)
    eng = _engine(folder, dtype, n_pages=n // 16 + 2)
    _close(_run(eng, "whole", tokens, [n]), want, dtype, f"{name} whole")
    _close(_run(eng, "decoded", tokens, [n - 40] + [1] * 40), want, dtype, f"{name} decoded")
    _close(_run(eng, "portions", tokens, helpers.cuts_changing(n)), want, dtype, f"{name} in portions")


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
    token, shorter than the convolution's taps), the logits agree with the uncut prompt's to
    rounding: the engine against itself."""
    folder, config, _ = models["A"]
    tokens = helpers.random_tokens(140, config["vocab"], seed=8)
    eng = _engine(folder, "float32", n_pages=12)
    whole = _run(eng, "w", tokens, [140])
    for cuts in (helpers.cuts_changing(140), [1] * 140, [16, 16, 1, 15, 17, 15, 2, 58], [15, 2, 31, 33, 59], [137, 3],
                 [2, 1, 3, 2, 64, 65, 3]):
        got = _run(eng, "c", tokens, cuts)
        assert (got - whole).abs().max().item() <= 2e-5 * whole.abs().max().item(), cuts[:6]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens_and_long_decode(models, dtype):
    """Every token one by one from the first: 400 of them, recorded decode steps replayed, page
    after page taken, the states and the convolutions' inputs carried 400 times."""
    folder, config, weights = models["C"]
    n = 400
    tokens = helpers.random_tokens(n, config["vocab"], seed=77)
    want = _plain(weights, config, tokens, dtype)
    eng = _engine(folder, dtype, n_pages=n // 16 + 1)
    got = _run(eng, "r", tokens, [1] * n)
    _close(got[:8], want[:8], dtype, "first tokens")
    _close(got, want, dtype, "decoding every token")


@pytest.mark.parametrize("kind", ["attention", "parallel"])
def test_a_key_far_back(tmp_path, kind):
    """900 tokens; the embedding's column 0 marks the token ids below 4 (keys to be found), column 1
    the ids 4 to 7 (queries that look for them), and the query and key projections follow those
    columns, so the last position reads position 3 among hundreds: in a prompt, in a portion's last
    row, and decoded alone."""
    if kind == "attention":
        layers = [_attention(2, 1, 16, 16, 12, 700, scale=1.0)]
    else:
        layers = [_parallel(_softmax(2, 1, 16, 16, softcap=40.0, scale=1.0), 1, 8, 8, [0.9])]
    config = _config(32, 40, 1000, 2, layers)
    w = plain.random_weights(config, 11)
    w["embed"][:8] *= 0.05
    w["embed"][:, :2] = 0.0
    w["embed"][:4, 0], w["embed"][4:8, 1] = 6.0, 6.0
    w["pos"][:, :2] = 0.0
    w["pos"] *= 0.2
    w["l0.norm1"][:], w["l0.canon1"][:] = 0.0, 0.0
    p = "l0.mix." + ("" if kind == "attention" else "left.")
    for name, col in (("q", 1), ("k", 0)):
        w[p + name][:, :2] = 0.0
        w[p + name][0::16, col] = 3.0  # the first column of every head follows the mark
    if kind == "attention":
        w[p + "q.norm"][:], w[p + "k.norm"][:] = 1.0, 1.0
        w[p + "q.norm"][0::16], w[p + "k.norm"][0::16] = 4.0, 4.0
        w[p + "rel"] *= 0.3
    n = 900
    tokens = [8 + t for t in helpers.random_tokens(n, 32, seed=5)]
    tokens[3], tokens[n - 1] = 2, 5
    want = plain.model(w, config, tokens)
    other = list(tokens)
    other[3] = 20  # without the marked token the last position reads something else
    moved = (plain.model(w, config, other)[n - 1] - want[n - 1]).abs().max() / want.abs().max()
    assert moved > 0.02, float(moved)
    folder = _folder(str(tmp_path / "m"), config, w)
    eng = _engine(folder, "float32", n_pages=n // 16 + 2)
    for cuts in ([n], [n - 7, 7], [n - 1, 1], [500, 2, 397, 1]):
        got = _run(eng, "r", tokens, cuts)
        _close(got[n - 1 :], want[n - 1 :], "float32", f"{kind}: the last of {cuts}")
        _close(got, want, "float32", f"{kind}: {cuts}")


def test_a_bucket_s_edge_in_prompts_and_in_decoding(tmp_path):
    """One attention layer whose distance table decides everything: the scores of queries and keys are nearly
    nothing (a scale of 0.01), a row of the table stands 8 above its neighbours.  The rows that a position reads change
    with every token, at distances in the table's plain part, in its logarithmic part and beyond
    its reach: whole, in portions cut at those distances, and token by token."""
    config = _config(32, 50, 200, 1, [_attention(2, 2, 8, 8, 10, 60, scale=0.01)])
    w = plain.random_weights(config, 2)
    rel = torch.zeros(10, 2)
    rel[6, 0], rel[9, 0], rel[3, 1], rel[8, 1] = 8.0, 8.0, 8.0, 8.0
    w["l0.mix.rel"] = rel
    n = 150
    tokens = helpers.random_tokens(n, 50, seed=3)
    want = plain.model(w, config, tokens)
    moved = copy.deepcopy(config)
    moved["layers"][0]["mixer"]["bias_max"] = 58  # two distances change their row
    assert (plain.model(w, moved, tokens) - want).abs().max() / want.abs().max() > 1e-3
    firsts = [m for m in range(1, 80) if plain.distance_bucket(m, 10, 60) != plain.distance_bucket(m - 1, 10, 60)]
    eng = _engine(_folder(str(tmp_path / "m"), config, w), "float32", n_pages=n // 16 + 2)
    cuts = [firsts[5], 1, 1] + [b - a for a, b in zip(firsts[5:], firsts[6:])]
    cuts = cuts[:-1] + [n - sum(cuts[:-1])]
    for c in ([n], cuts, [n - 70] + [1] * 70):
        _close(_run(eng, "r", tokens, c), want, "float32", f"cut {c[:8]}")


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

    def softmax(**more):
        kv = pick([1, 2, 3])
        return _softmax(kv * pick([1, 2, 4]), kv, pick([8, 12, 16, 32, 40, 64]), pick([8, 16, 24, 48, 80]), scale=pick([None, 0.05, 0.4]), **more)

    layers = []
    for i in range(pick([1, 2, 3, 4, 5])):
        kind = pick(["parallel", "hgrn2", "attention"])
        if kind == "parallel":
            heads = pick([1, 2, 3])
            entry = _parallel(softmax(softcap=pick([0.5, 5.0, 30.0])), heads, pick([8, 16, 24]), pick([8, 16, 40]),
                              [pick([0.3, 0.9, 0.99, 1.0]) for _ in range(heads)], pick([0.5, 1.0]), pick([0.8, 1.3]))
        elif kind == "hgrn2":
            entry = _hgrn2(pick([1, 2, 4]), pick([8, 16, 24, 64]), pick([8, 16, 32, 40]))
        else:
            rows = pick([2, 5, 8, 32])
            entry = {"type": "attention", "mixer": softmax(bias_rows=rows, bias_max=pick([rows // 2 + 1, 20, 64.5, 500]))}
        ff = pick(["none", "dense", "moe", "moe"])
        if ff == "dense":
            entry = _dense(entry, pick([4, 8, 20, 64]))
        elif ff == "moe":
            experts = pick([2, 3, 8, 17])
            entry = _moe(entry, experts, pick([1, 2, experts]), pick([4, 8, 20]), shared=pick([None, 8, 12]), scale=pick([1.0, 2.5]))
        layers.append(entry)
    return _config(pick([16, 40, 64, 104, 256]), pick([17, 100, 257, 1000]), 256, pick([1, 2, 3, 5]), layers, eps=pick([1e-6, 1e-5, 1e-2]))


@pytest.mark.parametrize("seed", range(10))
def test_drawn_configurations(tmp_path, seed):
    """Every size, the layers' order and constants drawn: whole, in portions, and two requests
    side by side, in float32."""
    from mlx_lm_amd.engine import StepEntry

    config = _drawn_config(seed)
    weights = plain.random_weights(config, 100 + seed, sharp=2.0)
    folder = _folder(str(tmp_path / "m"), config, weights)
    a, b = helpers.random_tokens(120, config["vocab"], seed=seed), helpers.random_tokens(75, config["vocab"], seed=50 + seed)
    wa, wb = plain.model(weights, config, a), plain.model(weights, config, b)
    eng = _engine(folder, "float32", n_pages=16)
    _close(_run(eng, "whole", a, [120]), wa, "float32", f"seed {seed} whole: {json.dumps(config)}")
    _close(_run(eng, "portions", a, helpers.cuts_changing(120)), wa, "float32", f"seed {seed} portions: {json.dumps(config)}")
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
