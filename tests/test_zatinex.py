"""Zatinex without a GPU: the registry, the plan run by run, refusals, sizes read from a
checkpoint's shapes, and properties of the plain implementation (plain_zatinex.py) that the GPU
tests lean on."""

import copy
import math

import pytest
import torch

import plain_zatinex as plain
from mlx_lm_amd.config import CacheNeed, StateNeed, get_model_classes


def _attention(heads, kv_heads, dim, vdim, conv=None, rot=None, diff=0.4, scale=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "diff": diff, "scale": scale or dim ** -0.5}
    if conv:
        m["conv"] = conv
    if rot:
        m["rot"] = rot
    return {"type": "attention", "mixer": m}


def _gla(heads, dim, vdim, tau):
    return {"type": "gla", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau}}


def _latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, base=10000.0, kv_from=None, scale=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
         "scale": scale or (dim + rot_dim) ** -0.5, "rot": {"dims": rot_dim, "base": base}}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m}


def _with_ff(entry, ff):
    entry = dict(entry)
    entry["mlp"] = {"kind": "dense", "ff": ff}
    return entry


def _config(width, vocab, layers, eps=1e-5):
    for entry in layers:
        entry.setdefault("mlp", None)
    return {"architecture": "Zatinex", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}


YARN = {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0}
SMALL = _config(64, 130, [
    _with_ff(_latent(3, 16, 8, 24, 20, 40, base=300.0), 40),
    _attention(6, 3, 16, 24, conv=4, rot={"dims": 8, "base": 500.0, "scaling": YARN}, diff=0.3),
    _with_ff(_gla(2, 24, 16, 4.0), 24),
    _with_ff(_latent(2, 8, 8, 16, 12, 40, base=300.0, kv_from=0), 16),
    _gla(4, 8, 8, 1.0)])


def test_the_registry_finds_the_design_by_its_architecture_key():
    Model, Args = get_model_classes(SMALL)
    assert Model.__module__.endswith("models.zatinex")
    with pytest.raises(ValueError):
        get_model_classes({"architecture": "Zatinox"})


def test_the_plan_run_by_run():
    Model, Args = get_model_classes(SMALL)
    model = Model(Args.from_dict(Args.sizes_from_tensors(SMALL, {"l2.mix.a1": (4, 64), "l4.mix.a1": (5, 64)})))
    runs = model.decoder.schedule
    # the attention layer keeps pages and its convolution's inputs; the fourth layer reads the first one's pages
    assert [(r.layer, r.cache, r.writes_cache, r.state) for r in runs] == [
        (0, 0, True, None), (1, 1, True, 2), (2, 3, True, None), (3, 0, False, None), (4, 4, True, None)]
    needs = model.decoder.cache_needs()
    assert needs[0] == CacheNeed(1, 64, 0)  # one key head of kv_rank + rot_dim = 48 columns, in the next size the kernels take
    assert needs[1] == CacheNeed(6, 32, 0)  # two maps of three key heads, max(16, 24) in the next size
    assert needs[2] == StateNeed(((4 - 1) * (2 * 6 * 16 + 2 * 3 * 16 + 3 * 24),), "float32")
    assert needs[3] == StateNeed((2 * 24 * 16,), "float32") and needs[4] == StateNeed((4 * 8 * 8,), "float32")
    names = model.decoder.expected_tensors()
    assert names["l2.mix.a1"].shape == (4, 64) and names["l4.mix.a2"].shape == (32, 5)
    assert "l3.mix.dkv" not in names and "l0.mix.dkv" in names and "l1.mix.q.conv" in names
    assert "l1.norm2" not in names and "l0.mlp.gate" in names


def test_the_plains_weights_carry_the_names_the_model_expects():
    Model, Args = get_model_classes(SMALL)
    w = plain.random_weights(SMALL, 0, decay_rank=4)
    cfg = Args.sizes_from_tensors(SMALL, {k: tuple(v.shape) for k, v in w.items()})
    names = Model(Args.from_dict(cfg)).decoder.expected_tensors()
    assert set(names) == set(w)
    assert all(tuple(names[k].shape) == tuple(w[k].shape) for k in w)
    random = Model.random_weights(Args.from_dict(cfg), 1, "b")
    assert {k: tuple(v.shape) for k, v in random.items()} == {k: tuple(v.shape) for k, v in w.items()}


def test_what_cannot_run_is_refused():
    _, Args = get_model_classes(SMALL)
    for change in (lambda c: c["layers"][0].update(type="window"), lambda c: c["layers"][0]["mlp"].update(kind="moe"),
                   lambda c: c["layers"][3]["mixer"].update(kv_from=2), lambda c: c["layers"][3]["mixer"].update(kv_from=3),
                   lambda c: c["layers"][3]["mixer"].update(kv_rank=48), lambda c: c.pop("norm"),
                   lambda c: c["layers"][0]["mixer"]["rot"].update(dims=4)):
        c = copy.deepcopy(SMALL)
        change(c)
        with pytest.raises(ValueError):
            Args.from_dict(c)


def test_the_rotary_table_follows_the_interpolation_by_wavelength():
    from mlx_lm_amd.parts.rotary import rotary_table

    rot = {"dims": 16, "base": 500.0, "scaling": YARN}
    f, mult = rotary_table(16, 500.0, YARN)
    want, want_mult = plain.rotary_frequencies(rot)
    assert torch.allclose(f.double(), want, rtol=1e-6) and abs(mult - want_mult) < 1e-12
    plain_f = torch.tensor([500.0 ** (-2.0 * i / 16) for i in range(8)], dtype=torch.float64)
    # fast pairs keep their frequency, slow ones are divided by the factor, some lie between
    ratio = want / plain_f
    assert ratio[0] == 1.0 and abs(ratio[-1] - 1 / 8) < 1e-12 and ((ratio < 1) & (ratio > 1 / 8)).any()
    assert abs(mult - (0.1 * math.log(8.0) + 1)) < 1e-12
    g, one = rotary_table(8, 300.0)
    assert one == 1.0 and torch.allclose(g.double(), torch.tensor([300.0 ** (-i / 4) for i in range(4)], dtype=torch.float64), rtol=1e-6)


def test_the_plain_side_is_causal_and_leans_on_every_mechanism():
    w = {k: v.double() for k, v in plain.random_weights(SMALL, 3, sharp=2.0).items()}
    tokens = torch.randint(0, 130, (40,), generator=torch.Generator().manual_seed(1)).tolist()
    base = plain.forward(SMALL, w, tokens)
    other = plain.forward(SMALL, w, tokens[:25] + [(t + 1) % 130 for t in tokens[25:]])
    assert torch.equal(base[:25], other[:25]) and (base[25:] - other[25:]).abs().max() > 0.1
    scale = base.abs().max()

    def moved(change):
        c, ww = copy.deepcopy(SMALL), dict(w)
        change(c, ww)
        return ((plain.forward(c, ww, tokens) - base).abs().max() / scale).item()

    # each of these is a fault that an engine could have; all move the logits by far more than a tolerance of 5e-5
    assert moved(lambda c, ww: c["layers"][1]["mixer"].update(diff=0.31)) > 1e-3
    assert moved(lambda c, ww: c["layers"][1]["mixer"]["rot"].pop("scaling")) > 1e-3
    assert moved(lambda c, ww: c["layers"][1]["mixer"].pop("conv")) > 1e-2
    assert moved(lambda c, ww: c["layers"][2]["mixer"].update(tau=4.5)) > 1e-4
    assert moved(lambda c, ww: c["layers"][0]["mixer"]["rot"].update(base=310.0)) > 1e-4
    assert moved(lambda c, ww: ww.update({"l3.mix.g": ww["l3.mix.g"] * 0})) > 1e-3
    assert moved(lambda c, ww: ww.update({"l1.mix.lq1": ww["l1.mix.lq1"] * 0})) > 1e-4


def test_the_convolution_and_the_recurrence_against_sums_written_out():
    g = torch.Generator().manual_seed(0)
    u, taps = torch.randn(9, 3, generator=g).double(), torch.randn(3, 4, generator=g).double()
    y = plain.causal_conv(u, taps)
    for t in range(9):
        want = sum(taps[:, j] * u[t - 3 + j] for j in range(4) if t - 3 + j >= 0)
        assert torch.allclose(y[t], want)
    # gated linear attention: o_t = sum_(j <= t) (q_t * prod_(j < s <= t) alpha_s) . k_j  v_j
    cfg = _config(16, 20, [_gla(1, 4, 3, 2.0)])
    w = {k: v.double() for k, v in plain.random_weights(cfg, 1).items()}
    h = torch.randn(6, 16, generator=g).double()
    p = "l0.mix."
    q, k, v = h @ w[p + "q"].t() * 0.5, h @ w[p + "k"].t(), h @ w[p + "v"].t()
    alpha = torch.sigmoid((h @ w[p + "a1"].t()) @ w[p + "a2"].t() + w[p + "a2.b"]).pow(0.5)
    o = torch.stack([sum(((q[t] * alpha[j + 1 : t + 1].prod(0)) @ k[j]) * v[j] for j in range(t + 1)) for t in range(6)])
    gate = h @ w[p + "g"].t()
    want = (plain.rms_norm(o, w[p + "norm"], 1e-5) * gate * torch.sigmoid(gate)) @ w[p + "o"].t()
    assert torch.allclose(plain.gated_linear_attention(h, w, p, cfg["layers"][0]["mixer"], 1e-5), want, atol=1e-10)
