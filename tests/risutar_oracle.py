"""A plain, slow Risutar in float64, one function per mechanism, written from the design's
equations and sharing no code with the package. Tests compare the framework with it.

A model is (cfg, sd): ``cfg`` the checkpoint's config dict, ``sd`` its tensors by checkpoint
name (any float dtype; everything is computed in float64). Every function handles ONE sequence
given whole: ``tokens`` is its full list of ids.
"""
import math

import torch

F64 = torch.float64


def f64(t):
    return t.to(F64)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def gelu_erf(z):
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def silu(z):
    return z * torch.sigmoid(z)


def rms_div(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * f64(w) + f64(b)


# ----------------------------------------------------------------------------- embedding
def bigram_rows(cfg, tokens):
    bg = (cfg.get("embedding") or {}).get("bigram")
    rows = []
    for t, tok in enumerate(tokens):
        if t == 0:
            rows.append(bg["buckets"])
        else:
            rows.append((tokens[t - 1] * bg["mul_prev"] + tok * bg["mul_cur"]) % bg["buckets"])
    return rows


def embed(cfg, sd, tokens):
    x = f64(sd["embed"])[tokens]
    if (cfg.get("embedding") or {}).get("bigram"):
        x = x + f64(sd["bigram"])[bigram_rows(cfg, tokens)]
    return x


# ----------------------------------------------------------------------------- mixers
def rotate_half(v, pos, dims, base):
    """v [T, ..., n]: the first ``dims`` of the last axis rotate, i paired with i + dims/2."""
    half = dims // 2
    i = torch.arange(half, dtype=F64)
    freq = base ** (-2.0 * i / dims)
    ang = pos.to(F64)[:, None] * freq[None, :]
    while ang.dim() < v.dim():
        ang = ang.unsqueeze(1)
    c, s = torch.cos(ang), torch.sin(ang)
    u, w = v[..., :half], v[..., half:dims]
    out = v.clone()
    out[..., :half] = u * c - w * s
    out[..., half:dims] = w * c + u * s
    return out


def latent_kv(m, sd, pre, h, eps):
    """(latent c [T, r], rotated shared key [T, dr]) of the layer that owns the projection."""
    r, dr = m["kv_rank"], m["rot_dim"]
    T = h.shape[0]
    dkv = h @ f64(sd[pre + "dkv"]).T
    c = rms_div(dkv[:, :r], eps) * f64(sd[pre + "dkv.norm"])
    pos = torch.arange(T)
    kr = rotate_half(dkv[:, r:r + dr], pos, m["rot"]["dims"], m["rot"]["base"])
    return c, kr


def latent_attention(m, sd, pre, h, eps, kv):
    """``kv`` = (c, kr) of this layer or of the layer it borrows from."""
    H, d, dr, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    T = h.shape[0]
    c, kr = kv
    cq = rms_div(h @ f64(sd[pre + "dq"]).T, eps) * f64(sd[pre + "dq.norm"])
    q = (cq @ f64(sd[pre + "uq"]).T).reshape(T, H, d + dr)
    pos = torch.arange(T)
    qn = q[:, :, :d]
    qr = rotate_half(q[:, :, d:], pos, m["rot"]["dims"], m["rot"]["base"])
    kn = (c @ f64(sd[pre + "uk"]).T).reshape(T, H, d)
    v = (c @ f64(sd[pre + "uv"]).T).reshape(T, H, dv)
    sc = (torch.einsum("thd,jhd->htj", qn, kn) + torch.einsum("thd,jd->htj", qr, kr)) * m["scale"]
    vis = pos[:, None] >= pos[None, :]
    sc = sc.masked_fill(~vis[None], float("-inf"))
    w = torch.softmax(sc, -1)
    o = torch.einsum("htj,jhd->thd", w, v)
    gate = torch.sigmoid(h @ f64(sd[pre + "g"]).T)              # [T, H]
    o = o * gate[:, :, None]
    return o.reshape(T, H * dv) @ f64(sd[pre + "o"]).T


def gla(m, sd, pre, h, eps):
    H, d, dv, tau = m["heads"], m["dim"], m["vdim"], m["tau"]
    T = h.shape[0]
    q = (h @ f64(sd[pre + "q"]).T).reshape(T, H, d) * d ** -0.5
    k = (h @ f64(sd[pre + "k"]).T).reshape(T, H, d)
    v = (h @ f64(sd[pre + "v"]).T).reshape(T, H, dv)
    z = (h @ f64(sd[pre + "a1"]).T) @ f64(sd[pre + "a2"]).T + f64(sd[pre + "a2.b"])
    alpha = (torch.sigmoid(z) ** (1.0 / tau)).reshape(T, H, d)
    S = torch.zeros(H, d, dv, dtype=F64)
    o = torch.zeros(T, H, dv, dtype=F64)
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hdv,hd->hv", S, q[t])
    o = rms_div(o, eps) * f64(sd[pre + "norm"])
    o = o.reshape(T, H * dv) * silu(h @ f64(sd[pre + "g"]).T)
    return o @ f64(sd[pre + "o"]).T


# ----------------------------------------------------------------------------- feed-forwards
def dense_ff(sd, pre, h):
    return (silu(h @ f64(sd[pre + "gate"]).T) * (h @ f64(sd[pre + "up"]).T)) @ f64(sd[pre + "down"]).T


def expert(sd, pre, h):
    return gelu_erf(h @ f64(sd[pre + "up"]).T) @ f64(sd[pre + "down"]).T


def route(mlp, sd, pre, h):
    """(ids [T, top], weights [T, top]): top-k by logit, weights renormalised among the k."""
    z = h @ f64(sd[pre + "router"]).T + f64(sd[pre + "router.b"])
    top = mlp["router"]["top"]
    val, ids = torch.topk(z, top, dim=-1)
    return ids, torch.softmax(val, -1)


def moe_ff(mlp, sd, pre, h):
    ids, w = route(mlp, sd, pre, h)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(ids.shape[1]):
            out[t] += w[t, j] * expert(sd, f"{pre}e{int(ids[t, j])}.", h[t:t + 1])[0]
    if mlp.get("shared"):
        out = out + expert(sd, pre + "shared.", h)
    return out


def side_input(cfg, sd, i, x, tokens, eps):
    dim = cfg["token_side"]["dim"]
    pre = f"l{i}.side."
    e = f64(sd["side.embed"])[tokens][:, i * dim:(i + 1) * dim]
    g = gelu_tanh(x @ f64(sd[pre + "gate"]).T) * e
    y = g @ f64(sd[pre + "proj"]).T
    return x + rms_div(y, eps) * f64(sd[pre + "norm"])


# ----------------------------------------------------------------------------- the model
def forward(cfg, sd, tokens, trace=None):
    """Logits [T, vocab] (float64) of one sequence; ``trace`` (a list) receives the residual
    stream after every layer."""
    eps, alpha = cfg["norm"]["eps"], cfg["postln_alpha"]
    x = embed(cfg, sd, tokens)
    kvs = {}
    for i, L in enumerate(cfg["layers"]):
        pre, m = f"l{i}.", L["mixer"]
        if L["type"] == "latent_attention":
            src = m.get("kv_from")
            if src is None:
                kvs[i] = latent_kv(m, sd, pre + "mix.", x, eps)
                src = i
            y = latent_attention(m, sd, pre + "mix.", x, eps, kvs[src])
        elif L["type"] == "gla":
            y = gla(m, sd, pre + "mix.", x, eps)
        else:
            raise ValueError(L["type"])
        x = layer_norm(alpha * x + y, sd[pre + "norm1"], sd[pre + "norm1.b"], eps)
        mlp = L.get("mlp")
        if mlp:
            y = dense_ff(sd, pre + "mlp.", x) if mlp["kind"] == "dense" else moe_ff(mlp, sd, pre + "mlp.", x)
            x = layer_norm(alpha * x + y, sd[pre + "norm2"], sd[pre + "norm2.b"], eps)
        if cfg.get("token_side"):
            x = side_input(cfg, sd, i, x, tokens, eps)
        if trace is not None:
            trace.append(x.clone())
    x = layer_norm(x, sd["final.norm"], sd["final.norm.b"], eps)
    return x @ f64(sd["head"]).T


# ----------------------------------------------------------------------------- test models
def tensor_shapes(cfg, decay_rank=6):
    """Checkpoint tensor names and shapes of a configuration."""
    D, V = cfg["width"], cfg["vocab"]
    out = {"embed": (V, D), "final.norm": (D,), "final.norm.b": (D,), "head": (V, D)}
    bg = (cfg.get("embedding") or {}).get("bigram")
    if bg:
        out["bigram"] = (bg["buckets"] + 1, D)
    side = (cfg.get("token_side") or {}).get("dim", 0)
    if side:
        out["side.embed"] = (V, side * len(cfg["layers"]))
    for i, L in enumerate(cfg["layers"]):
        a, m = f"l{i}.", L["mixer"]
        for n in ("norm1", "norm2") if L.get("mlp") else ("norm1",):
            out[a + n] = (D,)
            out[a + n + ".b"] = (D,)
        H = m["heads"]
        if L["type"] == "gla":
            d, dv = m["dim"], m["vdim"]
            out.update({a + "mix.q": (H * d, D), a + "mix.k": (H * d, D), a + "mix.v": (H * dv, D),
                        a + "mix.g": (H * dv, D), a + "mix.o": (D, H * dv), a + "mix.norm": (dv,),
                        a + "mix.a1": (decay_rank, D), a + "mix.a2": (H * d, decay_rank),
                        a + "mix.a2.b": (H * d,)})
        else:
            d, dr, dv, r, rq = m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            out.update({a + "mix.dq": (rq, D), a + "mix.dq.norm": (rq,),
                        a + "mix.uq": (H * (d + dr), rq), a + "mix.uk": (H * d, r),
                        a + "mix.uv": (H * dv, r), a + "mix.g": (H, D), a + "mix.o": (D, H * dv)})
            if m.get("kv_from") is None:
                out.update({a + "mix.dkv": (r + dr, D), a + "mix.dkv.norm": (r,)})
        mlp = L.get("mlp")
        if mlp and mlp["kind"] == "dense":
            F = mlp["ff"]
            out.update({a + "mlp.gate": (F, D), a + "mlp.up": (F, D), a + "mlp.down": (D, F)})
        elif mlp:
            F = mlp["expert"]["ff"]
            E = mlp["router"]["experts"]
            out.update({a + "mlp.router": (E, D), a + "mlp.router.b": (E,)})
            for e in range(E):
                out.update({f"{a}mlp.e{e}.up": (F, D), f"{a}mlp.e{e}.down": (D, F)})
            if mlp.get("shared"):
                Fs = mlp["shared"]["ff"]
                out.update({a + "mlp.shared.up": (Fs, D), a + "mlp.shared.down": (D, Fs)})
        if side:
            out.update({a + "side.gate": (side, D), a + "side.proj": (D, side),
                        a + "side.norm": (D,)})
    return out


def bf16_exact(t):
    """Round to values bfloat16 holds exactly (so that a bf16 and an fp32 copy agree)."""
    return t.to(torch.float32).to(torch.bfloat16).to(F64)


def random_weights(cfg, seed=0, decay_rank=6):
    """Random float64 weights that bfloat16 holds exactly, sized so that every mechanism
    matters: norm weights and biases away from 1 and 0, router biases, decays spread between
    fast and slow, side inputs and bigram rows as large as the embedding."""
    g = torch.Generator().manual_seed(seed)
    w = {}
    for name, shape in tensor_shapes(cfg, decay_rank).items():
        rn = torch.randn(shape, generator=g, dtype=F64)
        if name.endswith((".norm1", ".norm2", "final.norm", ".dq.norm", ".dkv.norm", "mix.norm",
                          "side.norm")):
            v = 0.7 + 0.6 * torch.rand(shape, generator=g, dtype=F64)
        elif name.endswith("a2.b"):
            v = 1.5 + 2.0 * rn
        elif name.endswith(".b"):
            v = 0.3 * rn
        elif name in ("embed", "bigram", "side.embed"):
            v = rn
        elif name.endswith("mlp.router"):
            v = 2.0 * rn / math.sqrt(shape[-1])
        elif name.endswith("mix.a2"):
            v = 2.0 * rn / math.sqrt(shape[-1])
        else:
            v = rn / math.sqrt(shape[-1])
        w[name] = bf16_exact(v)
    return w


def route_margins(cfg, sd, tokens):
    """Per position, the smallest gap between the last chosen and the first rejected router
    logit over all routed layers (a small gap: a close call that rounding may turn)."""
    eps, alpha = cfg["norm"]["eps"], cfg["postln_alpha"]
    T = len(tokens)
    gaps = torch.full((T,), float("inf"), dtype=F64)
    trace = []
    forward(cfg, sd, tokens, trace)
    # replay the layers to reach each feed-forward's input
    x = embed(cfg, sd, tokens)
    kvs = {}
    for i, L in enumerate(cfg["layers"]):
        pre, m = f"l{i}.", L["mixer"]
        if L["type"] == "latent_attention":
            src = m.get("kv_from")
            if src is None:
                kvs[i] = latent_kv(m, sd, pre + "mix.", x, eps)
                src = i
            y = latent_attention(m, sd, pre + "mix.", x, eps, kvs[src])
        else:
            y = gla(m, sd, pre + "mix.", x, eps)
        x = layer_norm(alpha * x + y, sd[pre + "norm1"], sd[pre + "norm1.b"], eps)
        mlp = L.get("mlp")
        if mlp and mlp["kind"] == "moe" and mlp["router"]["top"] < mlp["router"]["experts"]:
            z = x @ f64(sd[pre + "mlp.router"]).T + f64(sd[pre + "mlp.router.b"])
            s = torch.sort(z, dim=-1, descending=True).values
            top = mlp["router"]["top"]
            gaps = torch.minimum(gaps, s[:, top - 1] - s[:, top])
        x = trace[i]
    return gaps.numpy()
