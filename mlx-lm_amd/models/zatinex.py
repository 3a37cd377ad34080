"""Zatinex: arguments, plan, tensor names, random weights.

A decoder-only design of pre-norm layers, ``h += mixer(N(h)); h += ff(N(h))`` with RMS norms,
whose layers mix tokens in one of three ways:

* ``attention``: differential attention (two softmax maps over the same values, one taken off
  the other) with grouped key heads, biases, a short causal convolution behind the projections,
  RMS-normed queries and keys and a partial rotation with interpolated frequencies
  (``parts/differential_attention.py``);
* ``gla``: gated linear attention, a matrix state per head that decays per key channel
  (``parts/linear_state.py:GatedLinearAttention``);
* ``latent_attention``: attention whose keys and values are read out of a small latent per
  token, with an output gate per head; a layer may read the latents that an earlier layer cached
  (``kv_from``) instead of making its own (``parts/latent_attention.py``).

The feed-forward is a dense gated one (``gated_mlp``); a layer may have none.  Token embedding,
no position table, a final RMS norm and an untied head.

config.json names the design under ``architecture`` and gives every size and constant: ``vocab``,
``width``, ``norm.eps`` and ``layers``, a list of ``{"type": ..., "mixer": {...}, "mlp": {"kind":
"dense", "ff": n} or null}``; ``max_positions`` is optional (the design has no table that bounds
it).  Mixer keys: ``attention``: ``heads, kv_heads, dim, vdim, scale, diff, conv`` (taps, optional),
``rot: {dims, base, scaling: {factor, original, fast, slow}}``; ``gla``: ``heads, dim, vdim, tau``
(the width of the decay's narrow middle is ``decay_rank``, or, as in the design's own files, what
the shape of ``a1`` says: ``sizes_from_tensors``); ``latent_attention``: ``heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, rot:
{dims, base}, kv_from`` (optional).  Tensors: ``embed``, ``l<i>.norm1``, ``l<i>.norm2``,
``l<i>.mix.*``, ``l<i>.mlp.{gate,up,down}``, ``final.norm``, ``head``; linear weights ``[out, in]``.
"""

from dataclasses import dataclass, field
from typing import Any, Dict, List

import torch

from ..config.base import BaseModelArgs
from ..config.plan import LayerSpec, ModelPlan, PartSpec, RunEntry
from ..parts.model import DecoderModel

MIXERS = ("attention", "gla", "latent_attention")
FEED_FORWARDS = ("dense",)
DEFAULT_POSITIONS = 1 << 15  # nothing in the design bounds a sequence; the cache's tables need a bound
DEFAULT_DECAY_RANK = 16


@dataclass
class ModelArgs(BaseModelArgs):
    """Keys of a Zatinex config.json; what the engine cannot run is refused here."""

    architecture: str
    vocab: int
    width: int
    layers: List[Dict[str, Any]]
    norm: Dict[str, Any] = field(default_factory=dict)
    max_positions: int = DEFAULT_POSITIONS

    def __post_init__(self):
        for key in ("vocab", "width", "max_positions"):
            if not isinstance(getattr(self, key), int) or getattr(self, key) <= 0:
                raise ValueError(f"{key} must be a positive integer, got {getattr(self, key)!r}")
        if not self.layers:
            raise ValueError("a model needs at least one layer")
        if "eps" not in self.norm:
            raise ValueError("norm.eps is missing")
        for i, entry in enumerate(self.layers):
            if entry.get("type") not in MIXERS:
                raise ValueError(f"layer {i}: mixer type {entry.get('type')!r} is not implemented (known: {MIXERS})")
            mlp = entry.get("mlp")
            if mlp is not None and mlp.get("kind") not in FEED_FORWARDS:
                raise ValueError(f"layer {i}: feed-forward kind {mlp.get('kind')!r} is not implemented (known: {FEED_FORWARDS})")
            m = entry.get("mixer") or {}
            if entry["type"] == "latent_attention":
                rot = m.get("rot") or {}
                if int(rot.get("dims", m.get("rot_dim", 0))) != int(m.get("rot_dim", 0)):
                    raise ValueError(f"layer {i}: the rotated key part has rot_dim columns, all of which turn")
                if "kv_from" in m:
                    j = m["kv_from"]
                    src = self.layers[j] if isinstance(j, int) and 0 <= j < i else None
                    if src is None or src.get("type") != "latent_attention" or "kv_from" in src["mixer"]:
                        raise ValueError(f"layer {i}: kv_from {j!r} must name an earlier latent-attention layer with latents of its own")
                    for key in ("kv_rank", "rot_dim", "rot"):
                        if src["mixer"].get(key) != m.get(key):
                            raise ValueError(f"layer {i}: its {key} differs from layer {j}'s, whose latents it reads")

    @property
    def eps(self):
        return float(self.norm["eps"])

    @staticmethod
    def sizes_from_tensors(config, shapes):
        """``config`` with the sizes that only a checkpoint's tensor shapes give: the width of a
        ``gla`` layer's decay middle (rows of ``a1``) and, where ``conv`` is not given, the taps of an
        attention layer's convolution (columns of ``q.conv``)."""
        import copy

        config = copy.deepcopy(config)
        for i, entry in enumerate(config.get("layers") or []):
            m = entry.get("mixer")
            if not isinstance(m, dict):
                continue
            a1, conv = shapes.get(f"l{i}.mix.a1"), shapes.get(f"l{i}.mix.q.conv")
            if entry.get("type") == "gla" and "decay_rank" not in m and a1 is not None:
                m["decay_rank"] = int(a1[0])
            if entry.get("type") == "attention" and "conv" not in m and conv is not None:
                m["conv"] = int(conv[1])
        return config


class Model:
    """The Zatinex model: a ``DecoderModel`` built from the plan below."""

    def __init__(self, args: ModelArgs):
        self.args = args
        self.model_type = "zatinex"
        self.decoder = DecoderModel(self.plan(args))

    @property
    def layers(self):
        return self.decoder.layers

    @staticmethod
    def mixer_spec(args, entry, p):
        D, eps, m = args.width, args.eps, entry["mixer"]
        rot = m.get("rot") or {}
        if entry["type"] == "attention":
            return PartSpec("differential_attention", {
                "width": D, "n_heads": m["heads"], "n_kv_heads": m.get("kv_heads", m["heads"]), "key_dim": m["dim"],
                "value_dim": m.get("vdim", m["dim"]), "scale": m.get("scale", m["dim"] ** -0.5), "diff": m["diff"], "eps": eps,
                "taps": int(m.get("conv") or 0), "rot_dims": int(rot.get("dims", 0)), "rot_base": float(rot.get("base", 10000.0)),
                "rot_scaling": rot.get("scaling")}, p)
        if entry["type"] == "gla":
            return PartSpec("gated_linear_attention", {
                "width": D, "n_heads": m["heads"], "key_dim": m["dim"], "value_dim": m.get("vdim", m["dim"]),
                "tau": m["tau"], "eps": eps, "decay_rank": int(m.get("decay_rank", DEFAULT_DECAY_RANK))}, p)
        return PartSpec("latent_attention", {
            "width": D, "n_heads": m["heads"], "key_dim": m["dim"], "rot_dim": m["rot_dim"], "value_dim": m["vdim"],
            "q_rank": m["q_rank"], "kv_rank": m["kv_rank"], "scale": m.get("scale", (m["dim"] + m["rot_dim"]) ** -0.5),
            "eps": eps, "rot_base": float(rot.get("base", 10000.0)), "rot_scaling": rot.get("scaling"),
            "own_latent": "kv_from" not in m}, p)

    @staticmethod
    def plan(args: ModelArgs) -> ModelPlan:
        D, eps = args.width, args.eps

        def norm(name):
            return PartSpec("rmsnorm", {"width": D, "eps": eps, "weight_name": name})

        layers, schedule, slot, slot_of = [], [], 0, {}
        for i, entry in enumerate(args.layers):
            p = f"l{i}."
            mixer = Model.mixer_spec(args, entry, p + "mix.")
            parts = dict(mixer_norm=norm(p + "norm1"), mixer=mixer)
            mlp = entry.get("mlp")
            if mlp is not None:
                parts["ffn_norm"] = norm(p + "norm2")
                parts["ffn"] = PartSpec("gated_mlp", {"width": D, "inner": mlp["ff"]}, p + "mlp.")
            layers.append(LayerSpec("pre_norm", parts))
            m = entry["mixer"]
            if entry["type"] == "latent_attention" and "kv_from" in m:
                schedule.append(RunEntry(layer=i, cache=slot_of[m["kv_from"]], writes_cache=False))
                continue
            slot_of[i] = slot
            # an attention layer with a convolution keeps pages and the convolution's last inputs: two slots
            if entry["type"] == "attention" and int(m.get("conv") or 0) > 1:
                schedule.append(RunEntry(layer=i, cache=slot, state=slot + 1))
                slot += 2
            else:
                schedule.append(RunEntry(layer=i, cache=slot))
                slot += 1
        return ModelPlan(
            width=D, vocab_size=args.vocab, max_positions=args.max_positions,
            embedding=PartSpec("token", {"vocab_size": args.vocab, "width": D, "weight_name": "embed"}),
            embedding_positions=None, layers=layers, schedule=schedule, final_norm=norm("final.norm"),
            head=PartSpec("linear", {"vocab_size": args.vocab, "width": D, "weight_name": "head"}))

    def sanitize(self, weights):
        return dict(weights)

    @staticmethod
    def random_weights(args: ModelArgs, seed, scheme="a"):
        """Seeded tensors under the checkpoint's names.  Scheme ``a``: norm weights 1, biases 0.
        Scheme ``b``: all of them drawn."""
        if scheme not in ("a", "b"):
            raise ValueError(f"unknown random-weight scheme '{scheme}'")
        g = torch.Generator().manual_seed(int(seed))
        D = args.width

        def normal(shape, std, mean=0.0):
            return torch.randn(shape, generator=g, dtype=torch.float32) * std + mean

        def vector(n, mean, std):
            return normal((n,), std, mean) if scheme == "b" else torch.full((n,), float(mean))

        t = {"embed": normal((args.vocab, D), 1.0)}
        for i, entry in enumerate(args.layers):
            p, m, q = f"l{i}.", entry["mixer"], f"l{i}.mix."
            t[p + "norm1"] = vector(D, 1.0, 0.1)
            if entry["type"] == "attention":
                H, G, d, dv = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m.get("vdim", m["dim"])
                for name, n in (("q", 2 * H * d), ("k", 2 * G * d), ("v", G * dv)):
                    t[q + name], t[q + name + ".b"] = normal((n, D), D ** -0.5), vector(n, 0.0, 0.1)
                    taps = int(m.get("conv") or 0)
                    if taps >= 1:
                        t[q + name + ".conv"] = normal((n, taps), taps ** -0.5)
                t[q + "q.norm"], t[q + "k.norm"] = vector(d, 1.0, 0.1), vector(d, 1.0, 0.1)
                for name in ("lq1", "lk1", "lq2", "lk2"):
                    t[q + name] = normal((d,), 0.1)
                t[q + "o"] = normal((D, H * dv), (H * dv) ** -0.5)
            elif entry["type"] == "gla":
                H, d, dv = m["heads"], m["dim"], m.get("vdim", m["dim"])
                rank = int(m.get("decay_rank", DEFAULT_DECAY_RANK))
                for name, n in (("q", H * d), ("k", H * d), ("v", H * dv), ("g", H * dv)):
                    t[q + name] = normal((n, D), D ** -0.5)
                t[q + "o"], t[q + "norm"] = normal((D, H * dv), (H * dv) ** -0.5), vector(dv, 1.0, 0.1)
                t[q + "a1"], t[q + "a2"] = normal((rank, D), D ** -0.5), normal((H * d, rank), rank ** -0.5)
                t[q + "a2.b"] = normal((H * d,), 1.0, 2.0)
            else:
                H, d, dr, dv, Q, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["q_rank"], m["kv_rank"]
                t[q + "dq"], t[q + "dq.norm"] = normal((Q, D), D ** -0.5), vector(Q, 1.0, 0.1)
                t[q + "uq"] = normal((H * (d + dr), Q), Q ** -0.5)
                if "kv_from" not in m:
                    t[q + "dkv"], t[q + "dkv.norm"] = normal((R + dr, D), D ** -0.5), vector(R, 1.0, 0.1)
                t[q + "uk"], t[q + "uv"] = normal((H * d, R), R ** -0.5), normal((H * dv, R), R ** -0.5)
                t[q + "g"], t[q + "o"] = normal((H, D), D ** -0.5), normal((D, H * dv), (H * dv) ** -0.5)
            mlp = entry.get("mlp")
            if mlp is not None:
                F = mlp["ff"]
                t[p + "norm2"] = vector(D, 1.0, 0.1)
                t[p + "mlp.gate"], t[p + "mlp.up"] = normal((F, D), D ** -0.5), normal((F, D), D ** -0.5)
                t[p + "mlp.down"] = normal((D, F), F ** -0.5)
        t["final.norm"] = vector(D, 1.0, 0.1)
        t["head"] = normal((args.vocab, D), D ** -0.5)
        return t
