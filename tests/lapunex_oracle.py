"""Plain float64 implementation of the Lapunex design: whole sequences, no cache, one function
per mechanism. It reads a configuration dict (the layout of the design's ``config.json``) and a
dict of checkpoint-named float64 arrays, and shares no code with the package.

    x_s = E[tok] * scale                      (s = 1 .. streams, or one x without streams)
    per sublayer q:  u = sum_s a_s x_s;  y = sublayer(norm(u));  x_t <- sum_s M[s, t] x_s + b_t y
    output:          logits = W_head norm(sum_s x_s)
"""
import math

import numpy as np


def rms(x, eps):
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps)


def norm1p(x, w, eps):
    """RMS norm whose stored weight is an offset from one."""
    return rms(x, eps) * (1.0 + w)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def logsigmoid(z):
    return -np.logaddexp(0.0, -z)


# ----------------------------------------------------------------------------- rotation
def yarn_frequencies(rot):
    """(frequency per pair, factor on cos and sin) of a rotation {base, dims, scaling}."""
    dims, base = int(rot["dims"]), float(rot["base"])
    i = np.arange(dims // 2, dtype=np.float64)
    f = base ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, orig = float(sc["factor"]), float(sc["original"])

    def dim_of(turns):
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(dim_of(float(sc["fast"]))), 0)
    hi = min(math.ceil(dim_of(float(sc["slow"]))), dims - 1)
    ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_half(x, positions, rot):
    """x [T, heads, n]: dimension i < dims/2 of every head turns with dimension i + dims/2."""
    dims = int(rot["dims"])
    f, m = yarn_frequencies(rot)
    ang = np.asarray(positions, np.float64)[:, None] * f[None, :]
    c, s = (np.cos(ang) * m)[:, None, :], (np.sin(ang) * m)[:, None, :]
    h = dims // 2
    out = x.copy()
    u, v = x[..., :h], x[..., h:dims]
    out[..., :h] = u * c - v * s
    out[..., h:dims] = v * c + u * s
    return out


# ----------------------------------------------------------------------------- mixers
def sink_attention(h, w, p, mx, eps):
    """Causal softmax attention with grouped keys, whole-projection q / k norm, partial
    rotation, one sink logit per head in the denominator and one sigmoid gate per head."""
    T = h.shape[0]
    H, G, d, dv = int(mx["heads"]), int(mx["kv_heads"]), int(mx["dim"]), int(mx["vdim"])
    q = rms(h @ w[p + "q"].T, eps) * w[p + "q.norm"]
    k = rms(h @ w[p + "k"].T, eps) * w[p + "k.norm"]
    v = (h @ w[p + "v"].T).reshape(T, G, dv)
    q, k = q.reshape(T, H, d), k.reshape(T, G, d)
    pos = np.arange(T)
    if mx.get("rot"):
        q, k = rotate_half(q, pos, mx["rot"]), rotate_half(k, pos, mx["rot"])
    gate = sigmoid(h @ w[p + "g"].T)                      # [T, H]
    out = np.zeros((T, H, dv))
    for hh in range(H):
        g = hh // (H // G)
        sc = (q[:, hh] @ k[:, g].T) * float(mx["scale"])
        sc = np.where(pos[None, :] <= pos[:, None], sc, -np.inf)
        sink = w[p + "sink"][hh]
        m = np.maximum(sc.max(-1), sink)
        e = np.exp(sc - m[:, None])
        den = e.sum(-1) + np.exp(sink - m)
        out[:, hh] = (e @ v[:, g]) / den[:, None] * gate[:, hh:hh + 1]
    return out.reshape(T, H * dv) @ w[p + "o"].T


def mlstm(h, w, p, mx, eps):
    """Matrix memory with exponential gating and a running maximum that starts at zero."""
    T = h.shape[0]
    H, d, dv, cap = int(mx["heads"]), int(mx["dim"]), int(mx["vdim"]), float(mx["gate_cap"])
    q = (h @ w[p + "q"].T).reshape(T, H, d) * d ** -0.5
    k = (h @ w[p + "k"].T).reshape(T, H, d)
    v = (h @ w[p + "v"].T).reshape(T, H, dv)
    ig = cap * np.tanh((h @ w[p + "i"].T + w[p + "i.b"]) / cap)
    fg = logsigmoid(cap * np.tanh((h @ w[p + "f"].T + w[p + "f.b"]) / cap))
    o = np.zeros((T, H, dv))
    for hh in range(H):
        S, n, m = np.zeros((d, dv)), np.zeros(d), 0.0
        for t in range(T):
            m1 = max(fg[t, hh] + m, ig[t, hh])
            a, b = math.exp(fg[t, hh] + m - m1), math.exp(ig[t, hh] - m1)
            S = a * S + b * np.outer(k[t, hh], v[t, hh])
            n = a * n + b * k[t, hh]
            m = m1
            o[t, hh] = (S.T @ q[t, hh]) / (max(abs(n @ q[t, hh]), math.exp(-m)) + 1e-6)
    o = rms(o, eps).reshape(T, H * dv) * w[p + "norm"] * sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


def parallel_mixer(h, w, p, mx, eps):
    return (float(mx["left_scale"]) * sink_attention(h, w, p + "left.", mx["left"], eps)
            + float(mx["right_scale"]) * mlstm(h, w, p + "right.", mx["right"], eps))


def lightning(h, w, p, mx, eps):
    """Linear attention with one fixed decay per head; the heads are normed together."""
    T = h.shape[0]
    H, d, dv = int(mx["heads"]), int(mx["dim"]), int(mx["vdim"])
    q = silu(h @ w[p + "q"].T).reshape(T, H, d)
    k = silu(h @ w[p + "k"].T).reshape(T, H, d)
    v = silu(h @ w[p + "v"].T).reshape(T, H, dv)
    o = np.zeros((T, H, dv))
    for hh in range(H):
        S = np.zeros((d, dv))
        for t in range(T):
            S = float(mx["decay"][hh]) * S + np.outer(k[t, hh], v[t, hh])
            o[t, hh] = S.T @ q[t, hh]
    o = rms(o.reshape(T, H * dv), eps) * w[p + "norm"] * sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


MIXERS = {"parallel": parallel_mixer, "lightning": lightning}


# ----------------------------------------------------------------------------- feed-forwards
def dense_ff(h, w, p):
    return (silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def route(h, w, p, r):
    """(chosen expert ids [T, top], their weights, the margin of the closest decision)."""
    E, top = int(r["experts"]), int(r["top"])
    z = h @ w[p + "router"].T
    s = np.exp(z - z.max(-1, keepdims=True))
    s = s / s.sum(-1, keepdims=True)
    gr = r.get("groups") or {"count": 1, "keep": 1}
    cnt, keep = int(gr["count"]), int(gr["keep"])
    gs = s.reshape(-1, cnt, E // cnt).max(-1)
    order = np.argsort(-gs, axis=-1, kind="stable")
    allowed = np.zeros_like(gs, dtype=bool)
    np.put_along_axis(allowed, order[:, :keep], True, axis=-1)
    margin = np.full(h.shape[0], np.inf)
    if keep < cnt:
        sg = np.take_along_axis(gs, order, -1)
        margin = sg[:, keep - 1] - sg[:, keep]
    ok = np.repeat(allowed, E // cnt, axis=-1)
    masked = np.where(ok, s, -1.0)
    ids = np.argsort(-masked, axis=-1, kind="stable")[:, :top]
    sm = np.take_along_axis(masked, np.argsort(-masked, axis=-1, kind="stable"), -1)
    if top < E:
        margin = np.minimum(margin, sm[:, top - 1] - np.maximum(sm[:, top], 0.0))
    return ids, np.take_along_axis(s, ids, -1) * float(r["scale"]), margin


def expert(h, w, p, limit):
    g = np.minimum(h @ w[p + "gate"].T, limit)
    u = np.clip(h @ w[p + "up"].T, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ w[p + "down"].T


def moe_ff(h, w, p, mlp):
    ids, wt, _ = route(h, w, p, mlp["router"])
    out = np.zeros((h.shape[0], w[p + "e0.down"].shape[0]))
    for t in range(h.shape[0]):
        for e, a in zip(ids[t], wt[t]):
            out[t] += a * expert(h[t:t + 1], w, f"{p}e{e}.", float(mlp["expert"]["limit"]))[0]
    return out


def feed_forward(h, w, p, mlp):
    return dense_ff(h, w, p) if mlp.get("kind", "dense") == "dense" else moe_ff(h, w, p, mlp)


# ----------------------------------------------------------------------------- the model
def layer_runs(c):
    n = len(c["layers"])
    lp = c.get("loop")
    if not lp:
        return list(range(n))
    a, b, times = int(lp["start"]), int(lp["stop"]), int(lp["times"])
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def forward(c, w, tokens, trace=None, upto=None):
    """Logits [T, vocab] of one sequence; ``trace`` (a list) receives the stream (the sum of
    the streams) after every layer run."""
    eps = float(c["norm"]["eps"])
    x = w["embed"][np.asarray(tokens)] * float(c["embedding"]["scale"])
    ns = int(c.get("streams") or 0)
    xs = np.stack([x] * ns) if ns else None
    for i in layer_runs(c)[:upto]:
        L, a = c["layers"][i], f"l{i}."
        subs = [(1, lambda h: MIXERS[L["type"]](h, w, a + "mix.", L["mixer"], eps))]
        if L.get("mlp"):
            subs.append((2, lambda h: feed_forward(h, w, a + "mlp.", L["mlp"])))
        for q, fn in subs:
            if ns:
                u = np.einsum("s,std->td", w[f"{a}hc{q}.in"], xs)
                y = fn(norm1p(u, w[f"{a}norm{q}"], eps))
                xs = (np.einsum("sr,std->rtd", w[f"{a}hc{q}.mix"], xs)
                      + w[f"{a}hc{q}.out"][:, None, None] * y[None])
            else:
                x = x + fn(norm1p(x, w[f"{a}norm{q}"], eps))
        if trace is not None:
            trace.append(xs.sum(0) if ns else x.copy())
    if ns:
        x = xs.sum(0)
    return norm1p(x, w["final.norm"], eps) @ w["head"].T


def route_margins(c, w, tokens):
    """Per position, the smallest margin of any routing decision in the model (inf without
    routed layers): positions where rounding could pick another expert."""
    eps = float(c["norm"]["eps"])
    T = len(tokens)
    best = np.full(T, np.inf)
    x = w["embed"][np.asarray(tokens)] * float(c["embedding"]["scale"])
    ns = int(c.get("streams") or 0)
    xs = np.stack([x] * ns) if ns else None
    for i in layer_runs(c):
        L, a = c["layers"][i], f"l{i}."
        for q in (1, 2):
            if q == 2 and not L.get("mlp"):
                continue
            u = np.einsum("s,std->td", w[f"{a}hc{q}.in"], xs) if ns else x
            h = norm1p(u, w[f"{a}norm{q}"], eps)
            if q == 1:
                y = MIXERS[L["type"]](h, w, a + "mix.", L["mixer"], eps)
            else:
                if L["mlp"].get("kind") == "moe":
                    best = np.minimum(best, route(h, w, a + "mlp.", L["mlp"]["router"])[2])
                y = feed_forward(h, w, a + "mlp.", L["mlp"])
            if ns:
                xs = (np.einsum("sr,std->rtd", w[f"{a}hc{q}.mix"], xs)
                      + w[f"{a}hc{q}.out"][:, None, None] * y[None])
            else:
                x = x + y
    return best


# ----------------------------------------------------------------------------- test weights
def bf16_exact(a):
    """Round to values bfloat16 holds exactly (so that every precision sees the same weights)."""
    import torch
    return torch.as_tensor(np.asarray(a, np.float64)).to(torch.bfloat16).double().numpy()


def random_weights(c, seed=0):
    """Checkpoint-named float64 arrays (bfloat16-exact) for configuration ``c``."""
    rng = np.random.default_rng(seed)
    D, V = int(c["width"]), int(c["vocab"])
    ns = int(c.get("streams") or 0)
    w = {}

    def lin(name, o, i, gain=1.0):
        w[name] = rng.standard_normal((o, i)) * gain / math.sqrt(i)

    w["embed"] = rng.standard_normal((V, D)) * 0.5
    lin("head", V, D)
    w["final.norm"] = rng.standard_normal(D) * 0.2
    for i, L in enumerate(c["layers"]):
        a, mx = f"l{i}.", L["mixer"]
        for q in (1, 2):
            if q == 2 and not L.get("mlp"):
                continue
            w[f"{a}norm{q}"] = rng.standard_normal(D) * 0.2
            if ns:
                # read weights that do not cancel: a sum of streams much smaller than the
                # streams would magnify every rounding in front of the norm
                w[f"{a}hc{q}.in"] = (1.0 + 0.3 * rng.standard_normal(ns)) / ns
                w[f"{a}hc{q}.out"] = 1.0 + 0.3 * rng.standard_normal(ns)
                w[f"{a}hc{q}.mix"] = np.eye(ns) + 0.15 * rng.standard_normal((ns, ns))
        m = a + "mix."
        if L["type"] == "lightning":
            H, d, dv = int(mx["heads"]), int(mx["dim"]), int(mx["vdim"])
            lin(m + "q", H * d, D, 2.0), lin(m + "k", H * d, D, 2.0)
            lin(m + "v", H * dv, D, 2.0), lin(m + "g", H * dv, D), lin(m + "o", D, H * dv)
            w[m + "norm"] = 1.0 + 0.2 * rng.standard_normal(H * dv)
        else:
            l, r = mx["left"], mx["right"]
            H, G, d, dv = int(l["heads"]), int(l["kv_heads"]), int(l["dim"]), int(l["vdim"])
            p = m + "left."
            lin(p + "q", H * d, D), lin(p + "k", G * d, D), lin(p + "v", G * dv, D)
            lin(p + "g", H, D), lin(p + "o", D, H * dv)
            w[p + "q.norm"] = 1.0 + 0.2 * rng.standard_normal(H * d)
            w[p + "k.norm"] = 1.0 + 0.2 * rng.standard_normal(G * d)
            w[p + "sink"] = 1.0 + rng.standard_normal(H)
            H, d, dv = int(r["heads"]), int(r["dim"]), int(r["vdim"])
            p = m + "right."
            lin(p + "q", H * d, D), lin(p + "k", H * d, D), lin(p + "v", H * dv, D)
            lin(p + "g", H * dv, D), lin(p + "o", D, H * dv)
            lin(p + "i", H, D, 2.0), lin(p + "f", H, D, 2.0)
            w[p + "i.b"] = rng.standard_normal(H) - 0.5
            w[p + "f.b"] = rng.standard_normal(H) + 2.0
            w[p + "norm"] = 1.0 + 0.2 * rng.standard_normal(H * dv)
        mlp = L.get("mlp")
        if not mlp:
            continue
        f = a + "mlp."
        if mlp.get("kind", "dense") == "dense":
            F = int(mlp["ff"])
            lin(f + "gate", F, D), lin(f + "up", F, D), lin(f + "down", D, F)
        else:
            F, E = int(mlp["expert"]["ff"]), int(mlp["router"]["experts"])
            lin(f + "router", E, D, 2.0)
            for e in range(E):
                lin(f"{f}e{e}.gate", F, D, 1.5), lin(f"{f}e{e}.up", F, D, 1.5)
                lin(f"{f}e{e}.down", D, F)
    return {k: bf16_exact(v) for k, v in w.items()}
