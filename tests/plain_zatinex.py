"""Zatinex, plainly: one function per mechanism, whole sequences, float64, no cache.

Written from the design's equations only; nothing here is shared with the engine.  ``config`` is
the config.json as a dict, ``w`` maps tensor names to float64 tensors, tokens are a list of ints.

    x_p      = embed[t_p]
    layer:     x += mixer(N(x; w1));  x += ff(N(x; w2))          (ff may be absent)
    N(x; w)  = x / sqrt(mean(x^2) + eps) * w
    logits   = head N(x; wf)
"""

import math

import torch

F64 = torch.float64


def rms_norm(x, weight, eps):
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def rotary_frequencies(rot):
    """``(f_i for i < dims/2, factor for cos and sin)``.  With ``scaling`` the frequencies whose
    wavelength is long against ``original`` are divided by ``factor``, short ones stay, a ramp
    between; cos and sin grow by ``0.1 ln(factor) + 1``."""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if not sc:
        return torch.tensor(f, dtype=F64), 1.0
    factor, original = float(sc["factor"]), float(sc["original"])

    def dim_of(turns):
        return dims * math.log(original / (2 * math.pi * turns)) / (2 * math.log(base))

    lo = max(math.floor(dim_of(float(sc["fast"]))), 0)
    hi = min(math.ceil(dim_of(float(sc["slow"]))), dims - 1)
    out = []
    for i, fi in enumerate(f):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(fi / factor * ramp + fi * (1.0 - ramp))
    return torch.tensor(out, dtype=F64), 0.1 * math.log(factor) + 1.0


def rotate_pairs(x, positions, freqs, mult):
    """``x`` ``[T, ..., n]``: columns ``2i`` and ``2i + 1`` of the first ``2 len(freqs)`` turn by
    ``position * freqs[i]``; the rest pass."""
    n = 2 * len(freqs)
    if n == 0:
        return x
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [len(freqs)]
    ang = (positions.to(F64)[:, None] * freqs[None]).reshape(shape)
    c, s = torch.cos(ang) * mult, torch.sin(ang) * mult
    u, v = x[..., 0:n:2], x[..., 1:n:2]
    turned = torch.stack([u * c - v * s, v * c + u * s], -1).flatten(-2)
    return torch.cat([turned, x[..., n:]], -1)


def causal_conv(u, taps_w):
    """``y_t = sum_j w[:, j] u_(t - taps + 1 + j)``, zeros before the start.  ``u`` ``[T, C]``."""
    T, taps = u.shape[0], taps_w.shape[1]
    y = torch.zeros_like(u)
    for j in range(taps):
        shift = taps - 1 - j
        if shift < T:
            y[shift:] += taps_w[:, j] * u[: T - shift]
    return y


def causal_softmax_attention(q, k, v, scale):
    """``q`` ``[T, d]``, ``k`` ``[T, d]``, ``v`` ``[T, dv]`` of one head."""
    T = q.shape[0]
    s = (q @ k.t()) * scale
    s = s.masked_fill(torch.ones(T, T, dtype=torch.bool).triu(1), float("-inf"))
    return torch.softmax(s, -1) @ v


def differential_attention(h, w, p, m, eps):
    T = h.shape[0]
    H, G, d, dv = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = h @ w[p + "q"].t() + w[p + "q.b"]
    k = h @ w[p + "k"].t() + w[p + "k.b"]
    v = h @ w[p + "v"].t() + w[p + "v.b"]
    if m.get("conv"):
        q, k, v = causal_conv(q, w[p + "q.conv"]), causal_conv(k, w[p + "k.conv"]), causal_conv(v, w[p + "v.conv"])
    q, k, v = q.view(T, H, 2, d), k.view(T, G, 2, d), v.view(T, G, dv)
    q, k = rms_norm(q, w[p + "q.norm"], eps), rms_norm(k, w[p + "k.norm"], eps)
    rot = m.get("rot")
    if rot:
        f, mult = rotary_frequencies(rot)
        q, k = rotate_pairs(q, pos, f, mult), rotate_pairs(k, pos, f, mult)
    diff = float(m["diff"])
    lam = torch.exp((w[p + "lq1"] * w[p + "lk1"]).sum()) - torch.exp((w[p + "lq2"] * w[p + "lk2"]).sum()) + diff
    out = []
    for hq in range(H):
        g = hq // (H // G)
        a1 = causal_softmax_attention(q[:, hq, 0], k[:, g, 0], v[:, g], m["scale"])
        a2 = causal_softmax_attention(q[:, hq, 1], k[:, g, 1], v[:, g], m["scale"])
        out.append(rms_norm(a1 - lam * a2, None, eps) * (1.0 - diff))
    return torch.cat(out, -1) @ w[p + "o"].t()


def gated_linear_attention(h, w, p, m, eps):
    T = h.shape[0]
    H, d, dv, tau = m["heads"], m["dim"], m["vdim"], float(m["tau"])
    q = (h @ w[p + "q"].t() * d ** -0.5).view(T, H, d)
    k = (h @ w[p + "k"].t()).view(T, H, d)
    v = (h @ w[p + "v"].t()).view(T, H, dv)
    z = (h @ w[p + "a1"].t()) @ w[p + "a2"].t() + w[p + "a2.b"]
    alpha = torch.sigmoid(z).pow(1.0 / tau).view(T, H, d)
    S = torch.zeros(H, d, dv, dtype=F64)
    o = torch.zeros(T, H, dv, dtype=F64)
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hdv,hd->hv", S, q[t])
    o = rms_norm(o, w[p + "norm"], eps).reshape(T, H * dv)
    gate = h @ w[p + "g"].t()
    return (o * gate * torch.sigmoid(gate)) @ w[p + "o"].t()


def latent_kv(h, w, p, m, eps):
    """The latent ``c`` ``[T, kv_rank]`` and the rotated key part ``[T, rot_dim]`` of a layer that
    has a down-projection of its own."""
    r = m["kv_rank"]
    ckr = h @ w[p + "dkv"].t()
    c = rms_norm(ckr[:, :r], w[p + "dkv.norm"], eps)
    f, mult = rotary_frequencies(m["rot"])
    return c, rotate_pairs(ckr[:, r:], torch.arange(h.shape[0]), f, mult)


def latent_attention(h, w, p, m, eps, shared):
    """``shared``: ``(c, rotated key part)`` of the layer that ``kv_from`` names, else ``None``.
    Returns the mixer's output and the pair that this layer's cache holds."""
    T = h.shape[0]
    H, d, dr, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    cq = rms_norm(h @ w[p + "dq"].t(), w[p + "dq.norm"], eps)
    q = (cq @ w[p + "uq"].t()).view(T, H, d + dr)
    f, mult = rotary_frequencies(m["rot"])
    q_rot = rotate_pairs(q[..., d:], torch.arange(T), f, mult)
    c, k_rot = shared if shared is not None else latent_kv(h, w, p, m, eps)
    k_plain = (c @ w[p + "uk"].t()).view(T, H, d)
    v = (c @ w[p + "uv"].t()).view(T, H, dv)
    gate = torch.sigmoid(h @ w[p + "g"].t())
    out = []
    for hq in range(H):
        qq = torch.cat([q[:, hq, :d], q_rot[:, hq]], -1)
        kk = torch.cat([k_plain[:, hq], k_rot], -1)
        out.append(causal_softmax_attention(qq, kk, v[:, hq], m["scale"]) * gate[:, hq : hq + 1])
    return torch.cat(out, -1) @ w[p + "o"].t(), (c, k_rot)


def dense_feed_forward(h, w, p):
    g = h @ w[p + "gate"].t()
    return (g * torch.sigmoid(g) * (h @ w[p + "up"].t())) @ w[p + "down"].t()


def forward(config, w, tokens, return_layers=False):
    """Logits ``[T, vocab]`` (and the stream after every layer)."""
    eps = float(config["norm"]["eps"])
    x = w["embed"][torch.tensor(tokens)]
    kept, streams = {}, []
    for i, layer in enumerate(config["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        h = rms_norm(x, w[p + "norm1"], eps)
        if layer["type"] == "attention":
            y = differential_attention(h, w, p + "mix.", m, eps)
        elif layer["type"] == "gla":
            y = gated_linear_attention(h, w, p + "mix.", m, eps)
        elif layer["type"] == "latent_attention":
            y, kept[i] = latent_attention(h, w, p + "mix.", m, eps, kept[m["kv_from"]] if "kv_from" in m else None)
        else:
            raise ValueError(layer["type"])
        x = x + y
        if layer.get("mlp") is not None:
            x = x + dense_feed_forward(rms_norm(x, w[p + "norm2"], eps), w, p + "mlp.")
        streams.append(x)
    logits = rms_norm(x, w["final.norm"], eps) @ w["head"].t()
    return (logits, torch.stack(streams)) if return_layers else logits


def random_weights(config, seed, sharp=1.0, decay_rank=4):
    """Float32 tensors under the checkpoint's names, every vector drawn.  ``sharp`` widens the
    attention scores (the weights of the query norms and the queries' up-projection grow by it),
    so that a key which is dropped, doubled or taken from a wrong page shows in the logits."""
    g = torch.Generator().manual_seed(seed)
    D = config["width"]

    def rnd(*shape, std=1.0, mean=0.0):
        return torch.randn(*shape, generator=g) * std + mean

    w = {"embed": rnd(config["vocab"], D), "final.norm": rnd(D, std=0.1, mean=1.0), "head": rnd(config["vocab"], D, std=D ** -0.5)}
    for i, layer in enumerate(config["layers"]):
        p, m = f"l{i}.mix.", layer["mixer"]
        w[f"l{i}.norm1"] = rnd(D, std=0.1, mean=1.0)
        if layer["type"] == "attention":
            H, G, d, dv = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m["vdim"]
            for name, n in (("q", 2 * H * d), ("k", 2 * G * d), ("v", G * dv)):
                w[p + name], w[p + name + ".b"] = rnd(n, D, std=D ** -0.5), rnd(n, std=0.2)
                if m.get("conv"):
                    w[p + name + ".conv"] = rnd(n, m["conv"], std=0.6)
            w[p + "q.norm"], w[p + "k.norm"] = rnd(d, std=0.2, mean=1.0) * sharp, rnd(d, std=0.2, mean=1.0)
            for name in ("lq1", "lk1", "lq2", "lk2"):
                w[p + name] = rnd(d, std=0.15)
            w[p + "o"] = rnd(D, H * dv, std=(H * dv) ** -0.5)
        elif layer["type"] == "gla":
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            for name, n in (("q", H * d), ("k", H * d), ("v", H * dv), ("g", H * dv)):
                w[p + name] = rnd(n, D, std=D ** -0.5)
            w[p + "o"], w[p + "norm"] = rnd(D, H * dv, std=(H * dv) ** -0.5), rnd(dv, std=0.2, mean=1.0)
            w[p + "a1"], w[p + "a2"] = rnd(decay_rank, D, std=D ** -0.5), rnd(H * d, decay_rank, std=1.0)
            w[p + "a2.b"] = rnd(H * d, std=1.0, mean=1.5)
        else:
            H, d, dr, dv, Q, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["q_rank"], m["kv_rank"]
            w[p + "dq"], w[p + "dq.norm"] = rnd(Q, D, std=D ** -0.5), rnd(Q, std=0.2, mean=1.0)
            w[p + "uq"] = rnd(H * (d + dr), Q, std=Q ** -0.5) * sharp
            if "kv_from" not in m:
                w[p + "dkv"], w[p + "dkv.norm"] = rnd(R + dr, D, std=D ** -0.5), rnd(R, std=0.2, mean=1.0)
            w[p + "uk"], w[p + "uv"] = rnd(H * d, R, std=R ** -0.5), rnd(H * dv, R, std=R ** -0.5)
            w[p + "g"], w[p + "o"] = rnd(H, D, std=D ** -0.5), rnd(D, H * dv, std=(H * dv) ** -0.5)
        if layer.get("mlp") is not None:
            F = layer["mlp"]["ff"]
            w[f"l{i}.norm2"] = rnd(D, std=0.1, mean=1.0)
            w[f"l{i}.mlp.gate"], w[f"l{i}.mlp.up"] = rnd(F, D, std=D ** -0.5), rnd(F, D, std=D ** -0.5)
            w[f"l{i}.mlp.down"] = rnd(D, F, std=F ** -0.5)
    return w


def model(weights, config, tokens):
    """Logits ``[T, vocab]`` in float64 from float32 (or rounded) weights."""
    return forward(config, {k: v.double() for k, v in weights.items()}, tokens)


def greedy(weights, config, prompt, n):
    tokens, out = list(prompt), []
    for _ in range(n):
        out.append(int(model(weights, config, tokens)[-1].argmax()))
        tokens.append(out[-1])
    return out
