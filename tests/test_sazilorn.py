"""Sazilorn without a GPU: the registry, the plan run by run, refusals, the size read from a
checkpoint's shapes, the distance buckets, and properties of the plain implementation
(plain_sazilorn.py) that the GPU tests lean on."""

import copy
import math

import pytest
import torch

import plain_sazilorn as plain
from mlx_lm_amd.config import CacheNeed, StateNeed, get_model_classes


def _softmax(heads, kv_heads, dim, vdim, scale=None, **more):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale or dim ** -0.5, **more}


def _parallel(left, heads, dim, vdim, decay, left_scale=0.7, right_scale=1.1):
    return {"type": "parallel", "mixer": {"left": left, "left_scale": left_scale, "right_scale": right_scale,
                                          "right": {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay}}}


def _hgrn2(heads, dim, vdim):
    return {"type": "hgrn2", "mixer": {"heads": heads, "dim": dim, "vdim": vdim}}


def _attention(heads, kv_heads, dim, vdim, rows, far, scale=None):
    return {"type": "attention", "mixer": _softmax(heads, kv_heads, dim, vdim, scale, bias_rows=rows, bias_max=far)}


def _dense(entry, ff):
    return dict(entry, mlp={"kind": "dense", "ff": ff})


def _moe(entry, experts, top, ff, shared=None, scale=1.5):
    return dict(entry, mlp={"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "scale": scale},
                            "shared": {"ff": shared} if shared else None})


def _config(width, vocab, positions, taps, layers, eps=1e-5):
    for entry in layers:
        entry.setdefault("mlp", None)
    return {"architecture": "Sazilorn", "vocab": vocab, "width": width, "max_positions": positions, "norm": {"eps": eps},
            "canon": {"taps": taps}, "layers": layers}


SMALL = _config(64, 130, 400, 4, [
    _moe(_hgrn2(2, 24, 16), 5, 2, 24, shared=16),
    _dense(_parallel(_softmax(4, 2, 16, 24, softcap=8.0), 3, 8, 16, [0.5, 0.97, 0.9]), 40),
    _dense(_attention(6, 3, 16, 8, 12, 50), 24),
    _parallel(_softmax(2, 2, 24, 24, softcap=3.0, scale=0.3), 1, 16, 24, [0.999]),
    _moe(_attention(2, 1, 32, 32, 9, 33.5), 3, 1, 16)])


def test_the_registry_finds_the_design_by_its_architecture_key():
    Model, Args = get_model_classes(SMALL)
    assert Model.__module__.endswith("models.sazilorn")
    with pytest.raises(ValueError):
        get_model_classes({"architecture": "Sazilorm"})


def test_the_plan_run_by_run():
    Model, Args = get_model_classes(SMALL)
    model = Model(Args.from_dict(SMALL))
    D, taps = 64, 4
    canon = (taps - 1) * D
    assert [(r.layer, r.cache, r.writes_cache, r.state) for r in model.decoder.schedule] == [
        (0, 0, True, 1), (1, 2, True, 3), (2, 4, True, 5), (3, 6, True, 7), (4, 8, True, 9)]
    needs = model.decoder.cache_needs()
    assert needs[0] == StateNeed((2 * 24 * 16,), "float32") and needs[1] == StateNeed((canon,), "float32")
    # pages in the next head size the attention kernels take; the linear attention's matrices behind the convolution's inputs
    assert needs[2] == CacheNeed(2, 32, 0) and needs[3] == StateNeed((canon + 3 * 8 * 16,), "float32")
    assert needs[4] == CacheNeed(3, 16, 0) and needs[5] == StateNeed((canon,), "float32")
    assert needs[6] == CacheNeed(2, 32, 0) and needs[7] == StateNeed((canon + 16 * 24,), "float32")
    assert needs[8] == CacheNeed(1, 32, 0)
    names = model.decoder.expected_tensors()
    assert names["l2.mix.rel"].shape == (12, 6) and names["l2.mix.q.norm"].shape == (96,) and names["l2.mix.k.norm"].shape == (48,)
    assert names["l3.dwa"].shape == (5,) and names["l0.canon1"].shape == (64, 4) and names["l1.mix.right.norm"].shape == (48,)
    assert "l3.mlp.gate" not in names and "l4.mlp.shared.gate" not in names and "l0.mlp.shared.gate" in names
    # one tap keeps nothing: only a parallel layer's run has a state slot then
    one = copy.deepcopy(SMALL)
    one["canon"]["taps"] = 1
    runs = Model(Args.from_dict(one)).decoder.schedule
    assert [r.state is not None for r in runs] == [False, True, False, True, False]


def test_the_plains_weights_carry_the_names_the_model_expects():
    Model, Args = get_model_classes(SMALL)
    w = plain.random_weights(SMALL, 0)
    args = Args.from_dict(SMALL)
    names = Model(args).decoder.expected_tensors()
    assert set(names) == set(w)
    assert all(tuple(names[k].shape) == tuple(w[k].shape) for k in w)
    for scheme in "ab":
        random = Model.random_weights(args, 1, scheme)
        assert {k: tuple(v.shape) for k, v in random.items()} == {k: tuple(v.shape) for k, v in w.items()}


def test_the_tables_rows_come_from_the_checkpoint_where_the_config_is_silent():
    _, Args = get_model_classes(SMALL)
    c = copy.deepcopy(SMALL)
    del c["layers"][2]["mixer"]["bias_rows"]
    got = Args.sizes_from_tensors(c, {"l2.mix.rel": (12, 6), "l4.mix.rel": (7, 2)})
    assert got["layers"][2]["mixer"]["bias_rows"] == 12 and got["layers"][4]["mixer"]["bias_rows"] == 9
    assert "bias_rows" not in c["layers"][2]["mixer"]


def test_what_cannot_run_is_refused():
    Model, Args = get_model_classes(SMALL)
    for change in (lambda c: c["layers"][0].update(type="window"), lambda c: c["layers"][1]["mlp"].update(kind="sparse"),
                   lambda c: c.pop("norm"), lambda c: c["canon"].update(taps=0), lambda c: c.update(max_positions=0),
                   lambda c: c.update(layers=[])):
        c = copy.deepcopy(SMALL)
        change(c)
        with pytest.raises(ValueError):
            Args.from_dict(c)
    for change in (lambda c: c["layers"][1]["mixer"]["right"].update(decay=[0.5]), lambda c: c["layers"][2]["mixer"].update(kv_heads=4),
                   lambda c: c["layers"][2]["mixer"].update(bias_max=5), lambda c: c["layers"][2]["mixer"].pop("bias_rows")):
        c = copy.deepcopy(SMALL)
        change(c)
        with pytest.raises(ValueError):
            Model(Args.from_dict(c))


@pytest.mark.parametrize("rows,far", [(12, 50), (30, 110), (9, 33.5), (7, 400), (2, 3)])
def test_distance_buckets(rows, far):
    from mlx_lm_amd.parts.scored_attention import distance_bucket

    half = rows // 2
    got = [distance_bucket(n, rows, far) for n in range(1000)]
    assert got == [plain.distance_bucket(n, rows, far) for n in range(1000)]
    assert got[:half] == list(range(half)) and got[half] == half  # a row of its own up to half the table, ln(1) = 0
    assert all(a <= b for a, b in zip(got, got[1:])) and max(got) == rows - 1
    assert all(b == rows - 1 for n, b in enumerate(got) if n >= far)
    # written out once more: the first distance of every later row
    for row in range(half + 1, rows - 1):
        first = got.index(row) if row in got else None
        if first is not None:
            assert math.log(first / half) / math.log(far / half) * (rows - half) >= row - half - 1e-9


def test_the_plain_side_notices_what_the_comparisons_are_for():
    """Changes that a faulty engine could make move the plain logits by far more than the GPU
    tests' tolerances: the cap, the distance term, a bucket's row, the floor of the forget gate,
    the depth weights, the convolution's oldest tap, the renormalised weights and their constant."""
    w = plain.random_weights(SMALL, 3, sharp=3.0)
    tokens = [int(t) for t in torch.randint(0, 130, (60,), generator=torch.Generator().manual_seed(0))]
    base = plain.model(w, SMALL, tokens)
    scale = base.abs().max()

    def moved(config=None, **tensors):
        w2 = dict(w)
        w2.update(tensors)
        return ((plain.model(w2, config or SMALL, tokens) - base).abs().max() / scale).item()

    def with_(path, value):
        c = copy.deepcopy(SMALL)
        node = c
        for key in path[:-1]:
            node = node[key]
        node[path[-1]] = value
        return c

    assert moved(with_(("layers", 1, "mixer", "left", "softcap"), 0.0)) > 1e-3
    rel = w["l2.mix.rel"].clone()
    rel[11] += 1.0  # the last row: distances from 50 on
    assert moved(**{"l2.mix.rel": rel}) > 1e-3
    assert moved(with_(("layers", 2, "mixer", "bias_max"), 49)) > 1e-4
    assert moved(**{"l0.mix.lower": w["l0.mix.lower"] * 0.5}) > 1e-3
    dwa = w["l3.dwa"].clone()
    dwa[0] += 0.2  # the embedding's share, four layers on
    assert moved(**{"l3.dwa": dwa}) > 1e-3
    canon = w["l1.canon1"].clone()
    canon[:, 0] = 0.0  # the oldest tap
    assert moved(**{"l1.canon1": canon}) > 1e-3
    assert moved(with_(("layers", 0, "mlp", "router", "scale"), 1.0)) > 1e-3
    assert moved(with_(("layers", 1, "mixer", "right", "decay"), [0.5, 0.97, 0.8])) > 1e-4
    assert moved(with_(("layers", 3, "mixer", "right_scale"), 1.0)) > 1e-4


def test_the_plain_recurrences_by_their_closed_forms():
    """The two linear attentions against sums written out: ``o_t = sum_(j <= t) decay^(t - j) (q_t . k_j) v_j``
    and ``o_t = sum_j (q_t * prod_(j < i <= t) f_i * (1 - f_j)) v_j`` per channel."""
    g = torch.Generator().manual_seed(1)
    D, T = 16, 9
    h = torch.randn(T, D, generator=g, dtype=torch.float64)
    w = {k: torch.randn(s, generator=g, dtype=torch.float64) * 0.4 for k, s in
         {"q": (8, D), "k": (8, D), "v": (6, D), "g": (6, D), "o": (D, 6), "norm": (6,)}.items()}
    m = {"heads": 2, "dim": 4, "vdim": 3, "decay": [0.8, 0.3]}
    got = plain.lightning_attention(h, w, "", m, 1e-5)
    q, k, v = (plain.silu(h @ w[x].t()) for x in "qkv")
    o = torch.zeros(T, 6, dtype=torch.float64)
    for head in range(2):
        for t in range(T):
            for j in range(t + 1):
                o[t, 3 * head:3 * head + 3] += m["decay"][head] ** (t - j) * (q[t, 4 * head:4 * head + 4] @ k[j, 4 * head:4 * head + 4]) * v[j, 3 * head:3 * head + 3]
    want = (plain.rms_norm(o, w["norm"], 1e-5) * torch.sigmoid(h @ w["g"].t())) @ w["o"].t()
    assert torch.allclose(got, want, atol=1e-12)
    w2 = {"q": w["q"], "f": w["k"], "f.b": torch.randn(8, generator=g, dtype=torch.float64), "lower": torch.rand(8, generator=g, dtype=torch.float64),
          "v": w["v"], "norm": torch.randn(3, generator=g, dtype=torch.float64), "o": w["o"]}
    got = plain.hgrn2_mixer(h, w2, "", {"heads": 2, "dim": 4, "vdim": 3}, 1e-5)
    f = w2["lower"] + (1 - w2["lower"]) * torch.sigmoid(h @ w2["f"].t() + w2["f.b"])
    q = plain.silu(h @ w2["q"].t())
    v = h @ w2["v"].t()
    o = torch.zeros(T, 2, 3, dtype=torch.float64)
    for head in range(2):
        cols = slice(4 * head, 4 * head + 4)
        for t in range(T):
            for j in range(t + 1):
                keep = torch.ones(4, dtype=torch.float64)
                for i in range(j + 1, t + 1):
                    keep = keep * f[i, cols]
                o[t, head] += (q[t, cols] * keep * (1 - f[j, cols])).sum() * v[j, 3 * head:3 * head + 3]
    want = plain.rms_norm(o, w2["norm"], 1e-5).reshape(T, 6) @ w2["o"].t()
    assert torch.allclose(got, want, atol=1e-12)
