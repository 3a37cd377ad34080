"""Sazilorn: arguments, plan, tensor names, random weights.

A decoder-only design whose layers run their two sublayers side by side on one norm and pass on
a weighted sum of every earlier layer's result.  Token embedding plus a learned position vector;
layers

    ``u = N(x; 1 + w)``,  ``Y_(i+1) = x + mixer(u + conv(u)) + ff(u)``,  ``x <- sum_(j <= i+1) a_i[j] Y_j``

with an RMS norm whose tensor holds the scale's difference from one, a short causal convolution over time on what
the mixer reads, and ``Y_0`` the embedding's output; the model's norm and an untied head.  Mixers:

* ``parallel``: two mixers on the same input, summed with two constants: softmax attention with
  grouped key heads, capped scores (``softcap * tanh(s / softcap)``) and a sigmoid gate on the
  concatenated heads (``scored_attention``), beside linear attention with a fixed decay per
  head, silu on queries, keys and values, one norm over all heads and a sigmoid gate
  (``lightning_attention``);
* ``hgrn2``: linear attention with a forget gate per key channel that has a floor, and whose complement is the key
  (``forget_gate_attention``);
* ``attention``: softmax attention with grouped key heads, queries and keys normed over their
  whole projection, and a learned bias by bucketed distance (``scored_attention``).

No mixer rotates anything: positions enter through the embedding and the distance bias only.
Feed-forwards: ``dense`` (``down(gelu_tanh(gate u) * (up u))``) or ``moe`` (gated silu experts chosen
per token by ``softmax + correction``, weighted by the renormalised softmax times a constant, and
a shared expert); a layer may have none.

config.json names the design under ``architecture`` and gives every size and constant: ``vocab``,
``width``, ``max_positions``, ``norm.eps``, ``canon.taps`` and ``layers``, a list of ``{"type",
"mixer": {...}, "mlp": {"kind": "dense", "ff"} | {"kind": "moe", "expert": {ff}, "router":
{experts, top, scale}, "shared": {ff} or null} | null}``.  Tensors: ``embed``, ``pos``,
``l<i>.norm1``, ``l<i>.canon1``, ``l<i>.dwa``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``,
``head``; linear weights ``[out, in]``.
"""

from dataclasses import dataclass, field
from typing import Any, Dict, List

import torch

from ..config.base import BaseModelArgs
from ..config.plan import LayerSpec, ModelPlan, PartSpec, RunEntry
from ..parts.model import DecoderModel

MIXERS = ("parallel", "hgrn2", "attention")
FEED_FORWARDS = ("dense", "moe")


@dataclass
class ModelArgs(BaseModelArgs):
    """Keys of a Sazilorn config.json; what the engine cannot run is refused here."""

    architecture: str
    vocab: int
    width: int
    max_positions: int
    layers: List[Dict[str, Any]]
    norm: Dict[str, Any] = field(default_factory=dict)
    canon: Dict[str, Any] = field(default_factory=dict)

    def __post_init__(self):
        for key in ("vocab", "width", "max_positions"):
            if not isinstance(getattr(self, key), int) or getattr(self, key) <= 0:
                raise ValueError(f"{key} must be a positive integer, got {getattr(self, key)!r}")
        if not self.layers:
            raise ValueError("a model needs at least one layer")
        if "eps" not in self.norm:
            raise ValueError("norm.eps is missing")
        if not isinstance(self.taps, int) or self.taps < 1:
            raise ValueError(f"canon.taps must be a positive integer, got {self.taps!r}")
        for i, entry in enumerate(self.layers):
            if entry.get("type") not in MIXERS:
                raise ValueError(f"layer {i}: mixer type {entry.get('type')!r} is not implemented (known: {MIXERS})")
            mlp = entry.get("mlp")
            if mlp is not None and mlp.get("kind") not in FEED_FORWARDS:
                raise ValueError(f"layer {i}: feed-forward kind {mlp.get('kind')!r} is not implemented (known: {FEED_FORWARDS})")

    @property
    def eps(self):
        return float(self.norm["eps"])

    @property
    def taps(self):
        return self.canon.get("taps", 1)

    @staticmethod
    def sizes_from_tensors(config, shapes):
        """``config`` with the one size that only a checkpoint's tensor shapes give: the rows of an
        ``attention`` layer's distance table (``rel``)."""
        import copy

        config = copy.deepcopy(config)
        for i, entry in enumerate(config.get("layers") or []):
            m, rel = entry.get("mixer"), shapes.get(f"l{i}.mix.rel")
            if isinstance(m, dict) and entry.get("type") == "attention" and "bias_rows" not in m and rel is not None:
                m["bias_rows"] = int(rel[0])
        return config


class Model:
    """The Sazilorn model: a ``DecoderModel`` built from the plan below."""

    def __init__(self, args: ModelArgs):
        self.args = args
        self.model_type = "sazilorn"
        self.decoder = DecoderModel(self.plan(args))

    @property
    def layers(self):
        return self.decoder.layers

    @staticmethod
    def mixer_spec(args, entry, p):
        D, eps, m = args.width, args.eps, entry["mixer"]

        def softmax(a, q, **more):
            return PartSpec("scored_attention", {
                "width": D, "n_heads": a["heads"], "n_kv_heads": a.get("kv_heads", a["heads"]), "key_dim": a["dim"],
                "value_dim": a.get("vdim", a["dim"]), "scale": a.get("scale", a["dim"] ** -0.5), "eps": eps, **more}, q)

        if entry["type"] == "hgrn2":
            return PartSpec("forget_gate_attention", {"width": D, "n_heads": m["heads"], "key_dim": m["dim"],
                                                      "value_dim": m.get("vdim", m["dim"]), "eps": eps}, p)
        if entry["type"] == "attention":
            return softmax(m, p, whole_norm=True, bias_rows=m["bias_rows"], bias_far=float(m["bias_max"]),
                           max_positions=args.max_positions)
        left, right = m["left"], m["right"]
        attention = softmax(left, p + "left.", softcap=float(left.get("softcap", 0.0)), gate=True)
        lightning = PartSpec("lightning_attention", {
            "width": D, "n_heads": right["heads"], "key_dim": right["dim"], "value_dim": right.get("vdim", right["dim"]),
            "decay": list(right["decay"]), "eps": eps}, p + "right.")
        return PartSpec("parallel", {"left": attention, "right": lightning, "left_scale": m.get("left_scale", 1.0),
                                     "right_scale": m.get("right_scale", 1.0)}, p)

    @staticmethod
    def feed_forward_spec(args, mlp, p):
        if mlp["kind"] == "dense":
            return PartSpec("gated_mlp", {"width": args.width, "inner": mlp["ff"], "activation": "gelu_tanh"}, p)
        router, shared = mlp["router"], mlp.get("shared") or {}
        return PartSpec("gated_experts", {
            "width": args.width, "n_experts": router["experts"], "inner": (mlp.get("expert") or {}).get("ff", 0),
            "top": router["top"], "shared_inner": shared.get("ff", 0), "renormalize": True,
            "weight_scale": float(router.get("scale", 1.0))}, p)

    @staticmethod
    def plan(args: ModelArgs) -> ModelPlan:
        D, eps, n = args.width, args.eps, len(args.layers)

        def norm(name):
            return PartSpec("rmsnorm", {"width": D, "eps": eps, "weight_name": name, "offset": 1.0})

        layers, schedule, slot = [], [], 0
        for i, entry in enumerate(args.layers):
            p = f"l{i}."
            if entry["type"] == "attention" and "bias_rows" not in entry["mixer"]:
                raise ValueError(f"layer {i}: the rows of its distance table are not known (bias_rows, or the shape of {p}mix.rel)")
            parts = dict(norm=norm(p + "norm1"), mixer=Model.mixer_spec(args, entry, p + "mix."))
            if entry.get("mlp") is not None:
                parts["ffn"] = Model.feed_forward_spec(args, entry["mlp"], p + "mlp.")
            layers.append(LayerSpec("shared_norm", parts, {"input_taps": args.taps, "depth": i, "depth_total": n, "prefix": p}))
            # the run's state slot: the convolution's last inputs and, in a parallel layer, the linear attention's matrices
            keeps = args.taps > 1 or entry["type"] == "parallel"
            schedule.append(RunEntry(layer=i, cache=slot, state=slot + 1 if keeps else None))
            slot += 2 if keeps else 1
        return ModelPlan(
            width=D, vocab_size=args.vocab, max_positions=args.max_positions,
            embedding=PartSpec("token", {"vocab_size": args.vocab, "width": D, "weight_name": "embed"}),
            embedding_positions=PartSpec("learned", {"max_positions": args.max_positions, "width": D, "weight_name": "pos"}),
            layers=layers, schedule=schedule, final_norm=norm("final.norm"),
            head=PartSpec("linear", {"vocab_size": args.vocab, "width": D, "weight_name": "head"}))

    def sanitize(self, weights):
        return dict(weights)

    @staticmethod
    def random_weights(args: ModelArgs, seed, scheme="a"):
        """Seeded tensors under the checkpoint's names.  Scheme ``a``: norm weights and corrections
        0 (plain norms 1), the depth weights pass the last result on alone.  Scheme ``b``: all drawn."""
        if scheme not in ("a", "b"):
            raise ValueError(f"unknown random-weight scheme '{scheme}'")
        g = torch.Generator().manual_seed(int(seed))
        D = args.width

        def normal(shape, std, mean=0.0):
            return torch.randn(shape, generator=g, dtype=torch.float32) * std + mean

        def vector(n, mean, std):
            return normal((n,), std, mean) if scheme == "b" else torch.full((n,), float(mean))

        def softmax_attention(t, q, a, gate):
            H, G, d, dv = a["heads"], a.get("kv_heads", a["heads"]), a["dim"], a.get("vdim", a["dim"])
            t[q + "q"], t[q + "k"] = normal((H * d, D), D ** -0.5), normal((G * d, D), D ** -0.5)
            t[q + "v"], t[q + "o"] = normal((G * dv, D), D ** -0.5), normal((D, H * dv), (H * dv) ** -0.5)
            if gate:
                t[q + "g"] = normal((H * dv, D), D ** -0.5)
            return H, G, d, dv

        def gated(t, q, F):
            t[q + "gate"], t[q + "up"], t[q + "down"] = normal((F, D), D ** -0.5), normal((F, D), D ** -0.5), normal((D, F), F ** -0.5)

        t = {"embed": normal((args.vocab, D), 1.0), "pos": normal((args.max_positions, D), 0.3)}
        for i, entry in enumerate(args.layers):
            p, m = f"l{i}.", entry["mixer"]
            t[p + "norm1"] = vector(D, 0.0, 0.1)
            t[p + "canon1"] = normal((D, args.taps), 0.3)
            if scheme == "b":
                t[p + "dwa"] = normal((i + 2,), 0.3, 0.2)
                t[p + "dwa"][-1] += 0.6
            else:
                t[p + "dwa"] = torch.tensor([0.0] * (i + 1) + [1.0])
            q = p + "mix."
            if entry["type"] == "parallel":
                softmax_attention(t, q + "left.", m["left"], True)
                r, right = q + "right.", m["right"]
                H, d, dv = right["heads"], right["dim"], right.get("vdim", right["dim"])
                for name, rows in (("q", H * d), ("k", H * d), ("v", H * dv), ("g", H * dv)):
                    t[r + name] = normal((rows, D), D ** -0.5)
                t[r + "o"], t[r + "norm"] = normal((D, H * dv), (H * dv) ** -0.5), vector(H * dv, 1.0, 0.1)
            elif entry["type"] == "hgrn2":
                H, d, dv = m["heads"], m["dim"], m.get("vdim", m["dim"])
                t[q + "q"], t[q + "f"], t[q + "v"] = normal((H * d, D), D ** -0.5), normal((H * d, D), D ** -0.5), normal((H * dv, D), D ** -0.5)
                t[q + "f.b"] = normal((H * d,), 1.0, 1.0) if scheme == "b" else torch.full((H * d,), 1.0)
                t[q + "lower"] = torch.rand((H * d,), generator=g) * 0.9 if scheme == "b" else torch.full((H * d,), 0.5)
                t[q + "norm"], t[q + "o"] = vector(dv, 1.0, 0.1), normal((D, H * dv), (H * dv) ** -0.5)
            else:
                H, G, d, dv = softmax_attention(t, q, m, False)
                t[q + "q.norm"], t[q + "k.norm"] = vector(H * d, 1.0, 0.1), vector(G * d, 1.0, 0.1)
                t[q + "rel"] = normal((m["bias_rows"], H), 0.5)
            mlp = entry.get("mlp")
            if mlp is not None and mlp["kind"] == "dense":
                gated(t, p + "mlp.", mlp["ff"])
            elif mlp is not None:
                q, router = p + "mlp.", mlp["router"]
                for e in range(router["experts"]):
                    gated(t, f"{q}e{e}.", mlp["expert"]["ff"])
                t[q + "router"], t[q + "correction"] = normal((router["experts"], D), D ** -0.5), vector(router["experts"], 0.0, 0.02)
                if (mlp.get("shared") or {}).get("ff"):
                    gated(t, q + "shared.", mlp["shared"]["ff"])
        t["final.norm"] = vector(D, 0.0, 0.1)
        t["head"] = normal((args.vocab, D), D ** -0.5)
        return t
