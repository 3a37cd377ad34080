"""Sazilorn, plainly: one function per mechanism, whole sequences, float64, no cache.

Written from the design's equations only; nothing here is shared with the engine.  ``config`` is
the config.json as a dict, ``w`` maps tensor names to float64 tensors, tokens are a list of ints.

    X_0      = embed[t_p] + pos[p]
    layer i:   h = N(x; 1 + w1);  X_(i+1) = x + mixer(h + conv(h)) + ff(h);  x <- sum_(j <= i+1) a_i[j] X_j
    N(x; g)  = x / sqrt(mean(x^2) + eps) * g
    logits   = head N(x; 1 + wf)
"""

import math

import torch

F64 = torch.float64


def rms_norm(x, weight, eps):
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z**3)))


def silu(z):
    return z * torch.sigmoid(z)


def causal_conv(u, taps_w):
    """``y_t = sum_j w[:, j] u_(t - taps + 1 + j)``, zeros before the start.  ``u`` ``[T, C]``."""
    T, taps = u.shape[0], taps_w.shape[1]
    y = torch.zeros_like(u)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += taps_w[:, j] * u[s]
    return y


def distance_bucket(n, rows, far):
    """The row of the bias table for a distance ``n >= 0``: its own row below half the table, then
    rows spaced evenly in ``ln n`` so that ``far`` would reach the end, the last row beyond."""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


def softmax_attention(q, k, v, scale, softcap=0.0, bias=None):
    """One head, causal.  ``q`` ``[T, d]``, ``k`` ``[T, d]``, ``v`` ``[T, dv]``; ``bias`` ``[T, T]`` or ``None``."""
    T = q.shape[0]
    s = (q @ k.t()) * scale
    if softcap:
        s = softcap * torch.tanh(s / softcap)
    if bias is not None:
        s = s + bias
    s = s.masked_fill(torch.ones(T, T, dtype=torch.bool).triu(1), float("-inf"))
    return torch.softmax(s, -1) @ v


def grouped_heads(h, w, p, m, normed_eps=None, softcap=0.0, rel=None, far=None):
    """Softmax attention with grouped key heads; returns the concatenated heads ``[T, H * vdim]``."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m.get("vdim", m["dim"])
    q, k, v = h @ w[p + "q"].t(), h @ w[p + "k"].t(), h @ w[p + "v"].t()
    if normed_eps is not None:
        q, k = rms_norm(q, w[p + "q.norm"], normed_eps), rms_norm(k, w[p + "k.norm"], normed_eps)
    q, k, v = q.view(T, H, d), k.view(T, G, d), v.view(T, G, dv)
    outs = []
    for head in range(H):
        g = head // (H // G)
        bias = None
        if rel is not None:
            by_distance = torch.stack([rel[distance_bucket(n, rel.shape[0], far), head] for n in range(T)])
            i = torch.arange(T)
            bias = by_distance[(i[:, None] - i[None, :]).clamp(min=0)]  # (what lies above the diagonal is masked)
        outs.append(softmax_attention(q[:, head], k[:, g], v[:, g], m["scale"], softcap, bias))
    return torch.cat(outs, -1)


def lightning_attention(h, w, p, m, eps):
    """``S_t = decay_h S_(t-1) + k_t v_t^T``, ``o_t = S_t^T q_t`` with silu on q, k and v; the heads
    normed together, gated by a sigmoid, projected."""
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m.get("vdim", m["dim"])
    q = silu(h @ w[p + "q"].t()).view(T, H, d)
    k = silu(h @ w[p + "k"].t()).view(T, H, d)
    v = silu(h @ w[p + "v"].t()).view(T, H, dv)
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for head in range(H):
        S = torch.zeros(d, dv, dtype=h.dtype)
        for t in range(T):
            S = float(m["decay"][head]) * S + torch.outer(k[t, head], v[t, head])
            out[t, head] = S.t() @ q[t, head]
    o = rms_norm(out.reshape(T, H * dv), w[p + "norm"], eps) * torch.sigmoid(h @ w[p + "g"].t())
    return o @ w[p + "o"].t()


def parallel_mixer(h, w, p, m, eps):
    left = m["left"]
    heads = grouped_heads(h, w, p + "left.", left, softcap=float(left.get("softcap", 0.0)))
    heads = heads * torch.sigmoid(h @ w[p + "left.g"].t())
    a = heads @ w[p + "left.o"].t()
    b = lightning_attention(h, w, p + "right.", m["right"], eps)
    return m["left_scale"] * a + m["right_scale"] * b


def hgrn2_mixer(h, w, p, m, eps):
    """``S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T``, ``o_t = S_t^T q_t``; ``f`` bounded below."""
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m.get("vdim", m["dim"])
    q = silu(h @ w[p + "q"].t()).view(T, H, d)
    v = (h @ w[p + "v"].t()).view(T, H, dv)
    low = w[p + "lower"]
    f = (low + (1.0 - low) * torch.sigmoid(h @ w[p + "f"].t() + w[p + "f.b"])).view(T, H, d)
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for head in range(H):
        S = torch.zeros(d, dv, dtype=h.dtype)
        for t in range(T):
            S = f[t, head][:, None] * S + torch.outer(1.0 - f[t, head], v[t, head])
            out[t, head] = S.t() @ q[t, head]
    o = rms_norm(out, w[p + "norm"], eps).reshape(T, H * dv)
    return o @ w[p + "o"].t()


def attention_mixer(h, w, p, m, eps):
    heads = grouped_heads(h, w, p, m, normed_eps=eps, rel=w[p + "rel"], far=float(m["bias_max"]))
    return heads @ w[p + "o"].t()


def gated_ff(h, w, p, act):
    return (act(h @ w[p + "gate"].t()) * (h @ w[p + "up"].t())) @ w[p + "down"].t()


def expert_choice(h, w, p, router):
    """``(chosen experts [T, top], their weights [T, top])``."""
    s = torch.softmax(h @ w[p + "router"].t(), -1)
    idx = torch.topk(s + w[p + "correction"], int(router["top"]), dim=-1).indices
    picked = torch.gather(s, 1, idx)
    weights = picked / (picked.sum(-1, keepdim=True) + 1e-20) * float(router.get("scale", 1.0))
    return idx, weights


def experts_ff(h, w, p, mlp):
    idx, weights = expert_choice(h, w, p, mlp["router"])
    out = torch.zeros(h.shape[0], w[p + "e0.down"].shape[0], dtype=h.dtype)
    for t in range(h.shape[0]):
        for e, c in zip(idx[t].tolist(), weights[t]):
            out[t] += c * gated_ff(h[t : t + 1], w, f"{p}e{e}.", silu)[0]
    if mlp.get("shared"):
        out = out + gated_ff(h, w, p + "shared.", silu)
    return out


def feed_forward(h, w, p, mlp):
    if mlp["kind"] == "dense":
        return gated_ff(h, w, p, gelu_tanh)
    return experts_ff(h, w, p, mlp)


def choice_margin(h, w, p, router):
    """How far the last chosen expert's choice score lies above the first one left out, per token
    (infinite where every expert is chosen)."""
    s = torch.softmax(h @ w[p + "router"].t(), -1) + w[p + "correction"]
    top = int(router["top"])
    if top >= s.shape[-1]:
        return torch.full((h.shape[0],), float("inf"), dtype=h.dtype)
    ranked = s.sort(-1, descending=True).values
    return ranked[:, top - 1] - ranked[:, top]


MIXERS = {"parallel": parallel_mixer, "hgrn2": hgrn2_mixer, "attention": attention_mixer}


def forward(config, w, tokens, return_layers=False, margins=None):
    """Logits ``[T, vocab]`` of a whole sequence (and the stream after every layer).  ``margins``: a
    list that gets every expert layer's ``choice_margin``."""
    eps = float(config["norm"]["eps"])
    T = len(tokens)
    x = w["embed"][torch.tensor(tokens)] + w["pos"][:T]
    history, after = [x], []
    for i, entry in enumerate(config["layers"]):
        p = f"l{i}."
        h = rms_norm(x, 1.0 + w[p + "norm1"], eps)
        hm = h + causal_conv(h, w[p + "canon1"]) if p + "canon1" in w else h
        y = x + MIXERS[entry["type"]](hm, w, p + "mix.", entry["mixer"], eps)
        if entry.get("mlp") is not None:
            y = y + feed_forward(h, w, p + "mlp.", entry["mlp"])
            if margins is not None and entry["mlp"]["kind"] == "moe":
                margins.append(choice_margin(h, w, p + "mlp.", entry["mlp"]["router"]))
        history.append(y)
        x = sum(w[p + "dwa"][j] * history[j] for j in range(i + 2)) if p + "dwa" in w else y
        after.append(x)
    logits = rms_norm(x, 1.0 + w["final.norm"], eps) @ w["head"].t()
    return (logits, torch.stack(after)) if return_layers else logits


def random_weights(config, seed, sharp=1.0):
    """Seeded float32 tensors under the checkpoint's names, every one drawn (norm weights around
    zero or one as the design stores them).  ``sharp`` multiplies the query and key projections of
    the softmax attentions, so that their maps are peaked and a key taken wrongly shows."""
    g = torch.Generator().manual_seed(int(seed))
    D, taps = config["width"], config["canon"]["taps"]

    def n(shape, std, mean=0.0):
        return torch.randn(shape, generator=g) * std + mean

    def ff(w, p, F):
        w[p + "gate"], w[p + "up"], w[p + "down"] = n((F, D), D ** -0.5), n((F, D), D ** -0.5), n((D, F), F ** -0.5)

    def heads(w, p, a):
        H, G, d, dv = a["heads"], a.get("kv_heads", a["heads"]), a["dim"], a.get("vdim", a["dim"])
        w[p + "q"], w[p + "k"] = n((H * d, D), D ** -0.5) * sharp, n((G * d, D), D ** -0.5) * sharp
        w[p + "v"], w[p + "o"] = n((G * dv, D), D ** -0.5), n((D, H * dv), (H * dv) ** -0.5)
        return H, G, d, dv

    w = {"embed": n((config["vocab"], D), 1.0), "pos": n((config["max_positions"], D), 0.5)}
    for i, entry in enumerate(config["layers"]):
        p, m = f"l{i}.", entry["mixer"]
        w[p + "norm1"], w[p + "canon1"] = n((D,), 0.1), n((D, taps), 0.4)
        w[p + "dwa"] = n((i + 2,), 0.3, 0.1)
        w[p + "dwa"][-1] += 0.7
        q = p + "mix."
        if entry["type"] == "parallel":
            H, G, d, dv = heads(w, q + "left.", m["left"])
            w[q + "left.g"] = n((H * dv, D), D ** -0.5)
            r = m["right"]
            H, d, dv = r["heads"], r["dim"], r.get("vdim", r["dim"])
            for name, rows in (("q", H * d), ("k", H * d), ("v", H * dv), ("g", H * dv)):
                w[q + "right." + name] = n((rows, D), D ** -0.5)
            w[q + "right.o"], w[q + "right.norm"] = n((D, H * dv), (H * dv) ** -0.5), n((H * dv,), 0.1, 1.0)
        elif entry["type"] == "hgrn2":
            H, d, dv = m["heads"], m["dim"], m.get("vdim", m["dim"])
            w[q + "q"], w[q + "f"], w[q + "v"] = n((H * d, D), D ** -0.5), n((H * d, D), 2.0 * D ** -0.5), n((H * dv, D), D ** -0.5)
            w[q + "f.b"], w[q + "lower"] = n((H * d,), 1.0, 1.0), torch.rand((H * d,), generator=g) * 0.95
            w[q + "norm"], w[q + "o"] = n((dv,), 0.1, 1.0), n((D, H * dv), (H * dv) ** -0.5)
        else:
            H, G, d, dv = heads(w, q, m)
            w[q + "q.norm"], w[q + "k.norm"] = n((H * d,), 0.1, 1.0), n((G * d,), 0.1, 1.0)
            w[q + "rel"] = n((m["bias_rows"], H), 1.0)
        mlp = entry.get("mlp")
        if mlp is None:
            continue
        if mlp["kind"] == "dense":
            ff(w, p + "mlp.", mlp["ff"])
        else:
            E = mlp["router"]["experts"]
            for e in range(E):
                ff(w, f"{p}mlp.e{e}.", mlp["expert"]["ff"])
            w[p + "mlp.router"], w[p + "mlp.correction"] = n((E, D), 2.0 * D ** -0.5), n((E,), 0.05)
            if mlp.get("shared"):
                ff(w, p + "mlp.shared.", mlp["shared"]["ff"])
    w["final.norm"], w["head"] = n((D,), 0.1), n((config["vocab"], D), D ** -0.5)
    return w


def model(w, config, tokens, margins=None):
    """Float64 logits ``[T, vocab]`` from float32 (or rounded) weights."""
    return forward(config, {k: v.double() for k, v in w.items()}, list(tokens), margins=margins)


def greedy(w, config, prompt, n):
    tokens, out = list(prompt), []
    for _ in range(n):
        out.append(int(model(w, config, tokens)[-1].argmax()))
        tokens.append(out[-1])
    return out
