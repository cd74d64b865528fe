"""Pure-PyTorch reference implementations of every hot op (fp32 math).

These are (a) the CPU execution path (config 1: gpt2 on a CPU worker, and every
CPU test), and (b) the golden each HIP kernel is tested against
(SURVEY.md §4 tier T3). They define the tensor layouts the HIP kernels share:

* hidden states: ``[T, D]`` (tokens of all sequences flattened, bf16)
* fused QKV activations: ``[T, (Hq + 2*Hkv) * hd]``
* paged KV cache, per layer:
    ``k_cache [num_blocks, Hkv, block_size, hd]``
    ``v_cache [num_blocks, Hkv, block_size, hd]``  (token-major like K: a decode step's
    K/V write is one contiguous 2*hd-byte row per head; the decode kernel transposes V
    tiles through LDS with ds_read_b64_tr_b16 for its P·V MFMA)
* ``slot_mapping[t] = block * block_size + offset`` (int32)
* gate/up weights interleaved in 16-row groups: rows ``[32i, 32i+16)`` are gate
  features ``[16i, 16i+16)`` and rows ``[32i+16, 32i+32)`` the matching up
  features, so a GEMM tile owns both halves of every SiLU·mul pair.

The implicit HF ops these replace are listed in SURVEY.md §2.4 (K1-K16).
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch
import torch.nn.functional as F

GU_GROUP = 16  # gate/up interleave granularity (rows)


# ----------------------------------------------------------------------------- norms (K2, K3)
def rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    xf = x.float()
    var = xf.pow(2).mean(-1, keepdim=True)
    return (xf * torch.rsqrt(var + eps) * w.float()).to(x.dtype)


def fused_add_rmsnorm(x: torch.Tensor, residual: Optional[torch.Tensor], w: torch.Tensor,
                      eps: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """residual' = residual + x (or x when residual is None); out = rmsnorm(residual')."""
    r = x.float() if residual is None else residual.float() + x.float()
    r_out = r.to(x.dtype)
    r = r_out.float()  # the residual stream is bf16 (HF semantics): normalise what is stored
    var = r.pow(2).mean(-1, keepdim=True)
    out = (r * torch.rsqrt(var + eps) * w.float()).to(x.dtype)
    return out, r_out


def layernorm(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float) -> torch.Tensor:
    return F.layer_norm(x.float(), (x.shape[-1],), w.float(), b.float(), eps).to(x.dtype)


def fused_add_layernorm(x, residual, w, b, eps):
    r = x.float() if residual is None else residual.float() + x.float()
    r_out = r.to(x.dtype)
    out = F.layer_norm(r_out.float(), (x.shape[-1],), w.float(), b.float(), eps).to(x.dtype)
    return out, r_out


# ----------------------------------------------------------------------------- embedding (K1)
def embedding(ids: torch.Tensor, table: torch.Tensor,
              pos_table: Optional[torch.Tensor] = None,
              positions: Optional[torch.Tensor] = None) -> torch.Tensor:
    x = table[ids.long()]
    if pos_table is not None:
        x = (x.float() + pos_table[positions.long()].float()).to(table.dtype)
    return x


# ----------------------------------------------------------------------------- GEMMs (K4, K9-K12)
def linear(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None,
           out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """y = x @ w.T (+ bias); w is [N, K] like torch.nn.Linear."""
    y = x.float() @ w.float().t()
    if bias is not None:
        y = y + bias.float()
    return y.to(out_dtype or x.dtype)


def interleave_gate_up(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """[F, K] x2 -> [2F, K] in the 16-row interleaved layout (see module doc)."""
    f, k = gate.shape
    assert f % GU_GROUP == 0, "intermediate size must be a multiple of 16"
    g = gate.reshape(f // GU_GROUP, 1, GU_GROUP, k)
    u = up.reshape(f // GU_GROUP, 1, GU_GROUP, k)
    return torch.cat([g, u], dim=1).reshape(2 * f, k)


def split_gate_up(gu: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Inverse of the interleave on the last dim of activations [T, 2F]."""
    t, f2 = gu.shape
    v = gu.reshape(t, f2 // (2 * GU_GROUP), 2, GU_GROUP)
    return v[:, :, 0, :].reshape(t, f2 // 2), v[:, :, 1, :].reshape(t, f2 // 2)


def silu_mul(gu: torch.Tensor) -> torch.Tensor:
    g, u = split_gate_up(gu)
    return (F.silu(g.float()) * u.float()).to(gu.dtype)


def gelu_tanh(x: torch.Tensor) -> torch.Tensor:
    return F.gelu(x.float(), approximate="tanh").to(x.dtype)


def linear_silu_mul(x, w_gu):
    return silu_mul(linear(x, w_gu))


# ----------------------------------------------------------------------------- RoPE + KV write (K5, K6)
def rope_cos_sin(max_pos: int, head_dim: int, theta: float, device=None,
                 scaling=()) -> torch.Tensor:
    """[max_pos, head_dim] fp32 table: cols [0, hd/2) = cos, [hd/2, hd) = sin. ``scaling``:
    the HF ``rope_scaling`` of the checkpoint as (key, value) pairs (ModelConfig)."""
    half = head_dim // 2
    inv = 1.0 / (theta ** (torch.arange(0, half, dtype=torch.float64) * 2.0 / head_dim))
    inv = rope_scaled_inv_freq(inv, dict(scaling))
    ang = torch.arange(max_pos, dtype=torch.float64)[:, None] * inv[None, :]
    return torch.cat([ang.cos(), ang.sin()], dim=1).float().to(device)


def rope_scaled_inv_freq(inv: torch.Tensor, sc: dict) -> torch.Tensor:
    """HF ``rope_scaling`` applied to the inverse frequencies (the table absorbs it, so the
    kernels are unchanged). ``llama3``: wavelengths longer than original_max / low_freq_factor
    are divided by ``factor``, shorter than original_max / high_freq_factor kept, the band
    between interpolated (transformers ``_compute_llama3_parameters``); ``linear``: every
    frequency divided by ``factor`` (= positions / factor). Other types are refused."""
    kind = sc.get("rope_type", sc.get("type", "default")) if sc else "default"
    if kind in ("default", None):
        return inv
    factor = float(sc["factor"])
    if kind == "linear":
        return inv / factor
    if kind == "llama3":
        lo, hi = float(sc.get("low_freq_factor", 1.0)), float(sc.get("high_freq_factor", 4.0))
        old = float(sc.get("original_max_position_embeddings", 8192))
        lo_wl, hi_wl = old / lo, old / hi
        wl = 2 * math.pi / inv
        out = torch.where(wl > lo_wl, inv / factor, inv)
        smooth = (old / wl - lo) / (hi - lo)
        smoothed = (1 - smooth) * out / factor + smooth * out
        medium = (wl >= hi_wl) & (wl <= lo_wl)
        return torch.where(medium, smoothed, out)
    raise ValueError(f"unsupported rope_scaling type {kind!r} (supported: llama3, linear)")


def apply_rope(x: torch.Tensor, positions: torch.Tensor, cos_sin: torch.Tensor) -> torch.Tensor:
    """x [T, H, hd] rotate-half RoPE (HF Llama convention), fp32 math."""
    hd = x.shape[-1]
    half = hd // 2
    cs = cos_sin[positions.long()]              # [T, hd]
    cos, sin = cs[:, None, :half], cs[:, None, half:]
    xf = x.float()
    x1, x2 = xf[..., :half], xf[..., half:]
    return torch.cat([x1 * cos - x2 * sin, x2 * cos + x1 * sin], dim=-1).to(x.dtype)


def split_qkv(qkv: torch.Tensor, hq: int, hkv: int, hd: int):
    t = qkv.shape[0]
    q = qkv[:, : hq * hd].reshape(t, hq, hd)
    k = qkv[:, hq * hd: (hq + hkv) * hd].reshape(t, hkv, hd)
    v = qkv[:, (hq + hkv) * hd:].reshape(t, hkv, hd)
    return q, k, v


def write_kv(k: torch.Tensor, v: torch.Tensor, slot_mapping: torch.Tensor,
             k_cache: torch.Tensor, v_cache: torch.Tensor) -> None:
    bs = k_cache.shape[2]
    slots = slot_mapping.long()
    valid = slots >= 0
    slots, kk, vv = slots[valid], k[valid], v[valid]
    blk, off = slots // bs, slots % bs
    k_cache[blk, :, off, :] = kk.to(k_cache.dtype)
    v_cache[blk, :, off, :] = vv.to(v_cache.dtype)


def rope_and_cache(qkv, positions, slot_mapping, cos_sin, k_cache, v_cache,
                   hq: int, hkv: int, hd: int, use_rope: bool = True):
    """Rotates q and k IN PLACE inside ``qkv`` and writes k/v to the paged cache.
    Returns strided views (q [T,Hq,hd], k [T,Hkv,hd], v [T,Hkv,hd]) into ``qkv``."""
    q, k, v = split_qkv(qkv, hq, hkv, hd)
    if use_rope:
        q.copy_(apply_rope(q, positions, cos_sin))
        k.copy_(apply_rope(k, positions, cos_sin))
    if k_cache is not None:
        write_kv(k, v, slot_mapping, k_cache, v_cache)
    return q, k, v


# ----------------------------------------------------------------------------- attention (K7, K8)
def prefill_attention(q, k, v, cu_seqlens: torch.Tensor, scale: float) -> torch.Tensor:
    """Causal varlen GQA attention. q [T,Hq,hd], k/v [T,Hkv,hd] -> [T,Hq,hd]."""
    out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    hq, hkv = q.shape[1], k.shape[1]
    rep = hq // hkv
    cu = cu_seqlens.tolist()
    for i in range(len(cu) - 1):
        s, e = cu[i], cu[i + 1]
        if e <= s:
            continue
        qs = q[s:e].float().transpose(0, 1)                   # [Hq, L, hd]
        ks = k[s:e].float().transpose(0, 1).repeat_interleave(rep, 0)
        vs = v[s:e].float().transpose(0, 1).repeat_interleave(rep, 0)
        sc = (qs @ ks.transpose(1, 2)) * scale
        L = e - s
        mask = torch.ones(L, L, dtype=torch.bool, device=q.device).triu(1)
        sc = sc.masked_fill(mask, float("-inf"))
        o = sc.softmax(-1) @ vs
        out[s:e] = o.transpose(0, 1).to(q.dtype)
    return out


def gather_kv(k_cache, v_cache, block_table: torch.Tensor, ctx_len: int):
    """Contiguous [ctx, Hkv, hd] K and V for one sequence from the paged cache."""
    bs = k_cache.shape[2]
    nblk = (ctx_len + bs - 1) // bs
    blocks = block_table[:nblk].long()
    kk = k_cache[blocks].permute(0, 2, 1, 3).reshape(nblk * bs, k_cache.shape[1], -1)[:ctx_len]
    vv = v_cache[blocks].permute(0, 2, 1, 3).reshape(nblk * bs, v_cache.shape[1], -1)[:ctx_len]
    return kk, vv


def prefill_attention_paged(q, k_cache, v_cache, cu_seqlens, context_lens, block_tables,
                            scale: float) -> torch.Tensor:
    """Chunked prefill: the queries q[cu[i]:cu[i+1]] sit at positions [ctx-L, ctx) of
    sequence i and attend causally over its ctx = context_lens[i] cached keys."""
    out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    hq, hkv = q.shape[1], k_cache.shape[1]
    rep = hq // hkv
    cu, lens = cu_seqlens.tolist(), context_lens.tolist()
    for i in range(len(cu) - 1):
        s, e = cu[i], cu[i + 1]
        if e <= s:
            continue
        L, ctx = e - s, lens[i]
        kk, vv = gather_kv(k_cache, v_cache, block_tables[i], ctx)
        kk = kk.float().transpose(0, 1).repeat_interleave(rep, 0)   # [Hq, ctx, hd]
        vv = vv.float().transpose(0, 1).repeat_interleave(rep, 0)
        qs = q[s:e].float().transpose(0, 1)                          # [Hq, L, hd]
        sc = (qs @ kk.transpose(1, 2)) * scale                       # [Hq, L, ctx]
        qpos = torch.arange(ctx - L, ctx, device=q.device).unsqueeze(1)
        mask = torch.arange(ctx, device=q.device).unsqueeze(0) > qpos
        sc = sc.masked_fill(mask, float("-inf"))
        out[s:e] = (sc.softmax(-1) @ vv).transpose(0, 1).to(q.dtype)
    return out


def decode_attention(q, k_cache, v_cache, block_tables, context_lens, scale) -> torch.Tensor:
    """q [B,Hq,hd] single query per sequence against its paged cache."""
    out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    hq, hkv = q.shape[1], k_cache.shape[1]
    rep = hq // hkv
    lens = context_lens.tolist()
    for b, L in enumerate(lens):
        if L <= 0:
            out[b] = 0
            continue
        kk, vv = gather_kv(k_cache, v_cache, block_tables[b], L)
        kk = kk.float().transpose(0, 1).repeat_interleave(rep, 0)   # [Hq, L, hd]
        vv = vv.float().transpose(0, 1).repeat_interleave(rep, 0)
        sc = (kk @ q[b].float().unsqueeze(-1)).squeeze(-1) * scale  # [Hq, L]
        out[b] = (sc.softmax(-1).unsqueeze(1) @ vv).squeeze(1).to(q.dtype)
    return out


# ----------------------------------------------------------------------------- sampling (K13)
def topk_topp_filter(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor,
                     top_p: torch.Tensor) -> torch.Tensor:
    """HF warper order: Temperature -> TopK (ties kept) -> TopP (min_tokens_to_keep=1).
    Returns filtered fp32 logits (-inf outside the support)."""
    x = logits.float() / temperature.float().clamp_min(1e-6)[:, None]
    out = torch.full_like(x, float("-inf"))
    for i in range(x.shape[0]):
        row = x[i]
        k = int(top_k[i])
        if 0 < k < row.numel():
            kth = torch.topk(row, k).values[-1]
            row = row.masked_fill(row < kth, float("-inf"))
        p = float(top_p[i])
        if p < 1.0:
            srt, idx = torch.sort(row, descending=False)
            cum = srt.softmax(-1).cumsum(-1)
            remove = cum <= (1 - p)
            remove[-1] = False
            row = row.clone()
            row[idx[remove]] = float("-inf")
        out[i] = row
    return out


def _draw(probs: torch.Tensor, ids: torch.Tensor, g: torch.Generator) -> int:
    """Inverse-CDF draw over the support ordered by (probability desc, token id asc): the
    token drawn depends only on (token id, probability) pairs, not on where they sit in the
    row, so sampling from a candidate list (vocab-parallel LM head) equals sampling from the
    full vocabulary (same contract as the HIP sampler's sorted inverse-CDF draw)."""
    nz = (probs > 0).nonzero().squeeze(-1)
    pv, iv = probs[nz].double(), ids[nz]
    o1 = torch.argsort(iv)
    pv, iv = pv[o1], iv[o1]
    o2 = torch.sort(-pv, stable=True).indices
    pv, iv = pv[o2], iv[o2]
    u = torch.rand((), generator=g, dtype=torch.float64) * pv.sum()
    j = int(torch.searchsorted(pv.cumsum(0), u, right=True).clamp_max(pv.numel() - 1))
    return int(iv[j])


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor,
           top_p: torch.Tensor, generator: Optional[torch.Generator] = None,
           seeds: Optional[torch.Tensor] = None,
           ids: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Returns int32 token ids [B]. temperature<=0 (or top_k == 1) -> greedy argmax (lowest
    token id on ties). ``ids`` [B, C]: the row holds candidates (vocab-parallel LM head)
    whose token ids are ``ids``; default ids = column index. With per-row ``seeds`` each row
    draws from its own generator, so a request's tokens do not depend on its batch
    neighbours (same contract as the HIP sampler)."""
    B, V = logits.shape
    if ids is None:
        ids = torch.arange(V, device=logits.device, dtype=torch.int64).expand(B, V)
    ids = ids.long()
    greedy = (temperature <= 0) | (top_k == 1)
    out = torch.empty(B, dtype=torch.int32, device=logits.device)
    x = logits.float()
    for r in greedy.nonzero().squeeze(-1).tolist():
        m = x[r] == x[r].max()
        out[r] = int(ids[r][m].min())
    ng = ~greedy
    if ng.any():
        rows = ng.nonzero().squeeze(-1).tolist()
        filt = topk_topp_filter(x[ng], temperature[ng], top_k[ng], top_p[ng])
        probs = filt.softmax(-1)
        sd = seeds.tolist() if seeds is not None else None
        for j, r in enumerate(rows):
            if sd is None:
                g = generator
                if g is None:
                    g = torch.Generator(device=probs.device)
                    g.seed()
            else:
                g = torch.Generator(device=probs.device)
                g.manual_seed(int(sd[r]) & 0x7FFF_FFFF_FFFF_FFFF)
            out[r] = _draw(probs[j], ids[r], g)
    return out


def head_candidates(h: torch.Tensor, w_slice: torch.Tensor, offset: int, c: int):
    """Vocab-parallel LM head slice: fp32 logits of rows ``[offset, offset + V_r)`` and
    their top-``c`` (values desc, token ids) -> (fp32 [S, c], int32 [S, c])."""
    lg = linear(h, w_slice, out_dtype=torch.float32)
    v, i = torch.topk(lg, min(c, lg.shape[1]), dim=-1)
    return v, (i + offset).to(torch.int32)


# ----------------------------------------------------------------------------- MoE (K15, K16)
def router_topk(router_logits: torch.Tensor, k: int):
    """Mixtral routing: softmax -> topk -> renormalise. Returns (weights fp32 [T,k], ids int32)."""
    p = router_logits.float().softmax(-1)
    w, ids = torch.topk(p, k, dim=-1)
    w = w / w.sum(-1, keepdim=True)
    return w, ids.to(torch.int32)


def moe_mlp(x: torch.Tensor, w_gu: torch.Tensor, w_down: torch.Tensor,
            topk_w: torch.Tensor, topk_ids: torch.Tensor,
            expert_offset: int = 0) -> torch.Tensor:
    """x [T,D]; w_gu [E_local, 2F, D] (interleaved); w_down [E_local, D, F].
    Only experts in [expert_offset, expert_offset+E_local) contribute (EP shard)."""
    t = x.shape[0]
    e_local = w_gu.shape[0]
    out = torch.zeros(t, x.shape[1], dtype=torch.float32, device=x.device)
    for le in range(e_local):
        e = le + expert_offset
        rows, slot = (topk_ids == e).nonzero(as_tuple=True)
        if rows.numel() == 0:
            continue
        h = silu_mul(linear(x[rows], w_gu[le]))
        y = linear(h, w_down[le]).float()
        out.index_add_(0, rows, y * topk_w[rows, slot][:, None])
    return out.to(x.dtype)


# ----------------------------------------------------------------------------- hybrid family
# Mixed attention / recurrent designs (models/hybrid.py): fp32 residual stream and norms, GEMM
# operands in the storage dtype. Layouts shared with the HIP kernels:
# * token-major paged caches: row ``slot`` of ``[num_slots, width]`` (slot = block * block_size
#   + offset), kv head g at columns ``[g*d, (g+1)*d)``
# * recurrent state ``[state_slots, H, d, dv]`` fp32, one slot per live sequence
def group_rmsnorm(x: torch.Tensor, w: torch.Tensor, groups: int, eps: float,
                  out_dtype: torch.dtype, w_offset: float = 0.0) -> torch.Tensor:
    """x fp32 [T, D] cut into ``groups`` equal parts, each divided by its own
    sqrt(mean(part^2) + eps); the whole times w."""
    T, D = x.shape
    xg = x.float().reshape(T, groups, D // groups)
    n = xg * torch.rsqrt(xg.pow(2).mean(-1, keepdim=True) + eps)
    return (n.reshape(T, D) * (w.float() + w_offset)).to(out_dtype)


def act_mul(gu: torch.Tensor, F_: int, out_dtype: torch.dtype, kind: str,
            limit: float = 0.0) -> torch.Tensor:
    """The feed-forward's middle, fp32 in: ``gelu_mul`` / ``silu_mul`` = act(gu[:, :F]) *
    gu[:, F:2F]; ``gelu`` = gelu_tanh(gu[:, :F]); ``gelu_erf`` = the exact GELU of gu[:, :F];
    ``copy`` = gu[:, :F] itself."""
    if kind == "clamp_swish":
        return clamp_swish_mul(gu, F_, limit, out_dtype)
    g = gu[:, :F_].float()
    if kind == "gelu":
        return F.gelu(g, approximate="tanh").to(out_dtype)
    if kind == "gelu_erf":
        return F.gelu(g).to(out_dtype)
    if kind == "copy":
        return g.to(out_dtype)
    u = gu[:, F_:2 * F_].float()
    a = F.gelu(g, approximate="tanh") if kind == "gelu_mul" else F.silu(g)
    return (a * u).to(out_dtype)


def gelu_mul(gu: torch.Tensor, F_: int, out_dtype: torch.dtype) -> torch.Tensor:
    """gelu_tanh(gu[:, :F]) * gu[:, F:2F] (plain concatenation, fp32 in)."""
    g, u = gu[:, :F_].float(), gu[:, F_:2 * F_].float()
    return (F.gelu(g, approximate="tanh") * u).to(out_dtype)


def attn_prepare(proj, qw, kw, eps, H, G, d, kcache, vcache, slots, out_dtype):
    """proj fp32 [T, >= (H+G)*d] = [q | k | ...]: per-head RMS norm (shared weights) of q and k;
    normed k -> kcache rows, raw k -> vcache rows; returns normed q [T, H*d]."""
    T = proj.shape[0]
    q = proj[:, :H * d].float().reshape(T, H, d)
    k = proj[:, H * d:(H + G) * d].float().reshape(T, G, d)
    qn = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + eps) * qw.float()
    kn = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + eps) * kw.float()
    ok = slots >= 0
    idx = slots[ok].long()
    kcache[idx] = kn.reshape(T, G * d)[ok].to(kcache.dtype)
    vcache[idx] = k.reshape(T, G * d)[ok].to(vcache.dtype)
    return qn.reshape(T, H * d).to(out_dtype)


def rotate_interleaved(x: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor,
                       rot_dims: int) -> torch.Tensor:
    """Pairs (2i, 2i+1), i < rot_dims/2, of the last dim rotate by positions * inv_freq[i]
    (fp32 angles); the rest passes unchanged. x [..., T, n] with T = len(positions) on dim -2
    or x [T, n]."""
    ang = positions.float()[:, None] * inv_freq.float()[None, :]
    c, s = ang.cos(), ang.sin()
    out = x.clone()
    a, b = x[..., 0:rot_dims:2], x[..., 1:rot_dims:2]
    if x.dim() == 3:          # [T, H, n]
        c, s = c[:, None, :], s[:, None, :]
    out[..., 0:rot_dims:2] = a * c - b * s
    out[..., 1:rot_dims:2] = b * c + a * s
    return out


def mla_prepare(proj, cw, eps, H, d, dr, r, rot_dims, inv_freq, positions, slots, cache,
                out_dtype):
    """proj fp32 [T, H*(d+dr) + r + dr] = [q heads | compressed kv | shared rotated key].
    Cache row = [normed latent | rotated key]. Returns (q_nope [T, H, d], q_rot [T, H, dr])."""
    T = proj.shape[0]
    q = proj[:, :H * (d + dr)].float().reshape(T, H, d + dr)
    dkv = proj[:, H * (d + dr):H * (d + dr) + r + dr].float()
    c = dkv[:, :r]
    c = c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps) * cw.float()
    kr = rotate_interleaved(dkv[:, r:], positions, inv_freq, rot_dims)
    ok = slots >= 0
    cache[slots[ok].long()] = torch.cat([c, kr], 1)[ok].to(cache.dtype)
    qr = rotate_interleaved(q[:, :, d:], positions, inv_freq, rot_dims)
    return q[:, :, :d].to(out_dtype).contiguous(), qr.to(out_dtype)


def window_attention(q, k_cache, v_cache, dq, dv, H, G, cu_seqlens, positions, block_tables,
                     block_size, window, scale, slopes=None, talk=None, gate=None,
                     out_dtype=None, chunk=0, k_groups=None, sink=None, head_gate=False,
                     out_scale=1.0):
    """q [T, H*dq]; k_cache rows [slots, G*dq]; v_cache rows [slots, >= G*dv] (may be k_cache:
    values = the first dv columns of each kv head's... row when G == 1). Every query at position
    p attends cached positions [max(0, p-window+1), p] of its sequence. fp32 softmax; ``talk``
    [H, H] mixes the heads' normalised weights; ``slopes`` [H] subtract slope*(p-j); ``gate``
    fp32 [T, H*dv] multiplies the output by its sigmoid. ``chunk`` > 0: only keys of the
    query's own block of ``chunk`` positions are visible. ``k_groups``: key heads per cache row
    when it differs from the value heads G (1: every query head scores the whole key row).
    ``sink`` fp32 [H]: exp(sink_h) is added to head h's softmax denominator (a key without a
    value). ``head_gate``: gate is fp32 [T, H], one number per head. ``out_scale`` multiplies
    the output."""
    T = q.shape[0]
    Gk = G if k_groups is None else k_groups
    out = torch.zeros(T, H * dv, dtype=torch.float32, device=q.device)
    cu = cu_seqlens.tolist()
    for s in range(len(cu) - 1):
        t0, t1 = cu[s], cu[s + 1]
        if t1 <= t0:
            continue
        pos = positions[t0:t1].long()
        ctx = int(pos.max()) + 1
        j = torch.arange(ctx, device=q.device)
        sl = (block_tables[s].long()[j // block_size] * block_size + j % block_size)
        kk = k_cache[sl][:, :Gk * dq].float().reshape(ctx, Gk, dq)
        vv = v_cache[sl].float()
        vv = torch.stack([vv[:, g * dv:(g + 1) * dv] for g in range(G)], 1)   # [ctx, G, dv]
        qq = q[t0:t1].float().reshape(t1 - t0, H, dq)
        rep = H // G
        ke = kk.repeat_interleave(H // Gk, dim=1)                               # [ctx, H, dq]
        sc = torch.einsum("thd,jhd->htj", qq, ke) * scale
        dist = (pos[:, None] - j[None, :]).float()                              # [n, ctx]
        if slopes is not None:
            sc = sc - slopes.float()[:, None, None] * dist[None]
        vis = (dist >= 0) & (dist < window)
        if chunk:
            vis = vis & ((pos[:, None] // chunk) == (j[None, :] // chunk))
        sc = sc.masked_fill(~vis[None], float("-inf"))
        if sink is not None:
            n = sc.shape[1]
            sc = torch.cat([sc, sink.float()[:, None, None].expand(H, n, 1)], -1)
            w = torch.softmax(sc, dim=-1)[..., :-1]
        else:
            w = torch.softmax(sc, dim=-1)
        if talk is not None:
            w = torch.einsum("hg,gtj->htj", talk.float(), w)
        ve = vv.repeat_interleave(rep, dim=1)                                   # [ctx, H, dv]
        o = torch.einsum("htj,jhd->thd", w, ve)
        out[t0:t1] = o.reshape(t1 - t0, H * dv)
    if gate is not None and head_gate:
        out = (out.reshape(T, H, dv) * torch.sigmoid(gate.float())[:, :, None]).reshape(T, H * dv)
    elif gate is not None:
        out = out * torch.sigmoid(gate.float())
    if out_scale != 1.0:
        out = out * out_scale
    return out.to(out_dtype or q.dtype)


def hgrn2(proj, f_bias, lower, norm_w, eps, state, slots, cu_seqlens, positions, H, d, dv,
          out_dtype):
    """proj fp32 [T, 2*H*d + H*dv] = [qz | fz | v]; state fp32 [slots, H, d, dv] updated in
    place; a portion whose first position is 0 starts from zero. See csrc/kernels/recurrent.hip."""
    T = proj.shape[0]
    out = torch.zeros(T, H * dv, dtype=torch.float32, device=proj.device)
    cu = cu_seqlens.tolist()
    sl = slots.tolist()
    low = lower.float().reshape(H, d)
    fb = f_bias.float().reshape(H, d)
    nw = norm_w.float()
    for s in range(len(cu) - 1):
        t0, t1 = cu[s], cu[s + 1]
        if t1 <= t0 or sl[s] < 0:
            continue
        S = state[sl[s]].clone()
        if int(positions[t0]) == 0:
            S.zero_()
        p = proj[t0:t1].float()
        qv = F.silu(p[:, :H * d]).reshape(-1, H, d)
        fv = low + (1.0 - low) * torch.sigmoid(p[:, H * d:2 * H * d].reshape(-1, H, d) + fb)
        vv = p[:, 2 * H * d:2 * H * d + H * dv].reshape(-1, H, dv)
        for t in range(t1 - t0):
            S = fv[t][:, :, None] * S + (1.0 - fv[t])[:, :, None] * vv[t][:, None, :]
            o = torch.einsum("hdv,hd->hv", S, qv[t])
            o = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps) * nw
            out[t0 + t] = o.reshape(H * dv)
        state[sl[s]] = S
    return out.to(out_dtype)


def token_shift(h, mu, state, slots, cu_seqlens, positions, out_dtype):
    """h fp32 [T, D] (normed rows): row t becomes h_t + (h_{t-1} - h_t) * mu, with h_{t-1} the
    sequence's previous row as it came in — the row before it in this step, the row kept in
    ``state`` [slots, D] fp32 for a portion's first row, zeros at position 0. The last row of
    every sequence is kept in ``state``."""
    out = torch.empty_like(h, dtype=torch.float32)
    cu, sl = cu_seqlens.tolist(), slots.tolist()
    m = mu.float()
    for s in range(len(cu) - 1):
        t0, t1 = cu[s], cu[s + 1]
        if t1 <= t0 or sl[s] < 0:
            continue
        hh = h[t0:t1].float()
        first = (torch.zeros_like(hh[:1]) if int(positions[t0]) == 0
                 else state[sl[s]].float()[None])
        prev = torch.cat([first, hh[:-1]], 0)
        out[t0:t1] = hh + (prev - hh) * m
        state[sl[s]] = hh[-1]
    return out.to(out_dtype)


def talk_prepare(proj, bias, talk, eps, H, G, d, dv, kcache, vcache, slots, own_kv, out_dtype):
    """proj fp32 [T, H*d (+ G*d + G*dv)] = [q | k | v] and its bias. q and k heads are divided
    by their RMS; with ``own_kv`` normed k and v go to the cache rows ``slots``. Returns the
    queries with the pre-softmax head mixing folded in: since
        sum_g talk[h, g] (q_g . k_{c(g)}) = sum_c (sum_{g in c} talk[h, g] q_g) . k_c,
    head h scores the whole cached key row with q'_h [G*d], part c = sum_{g in c} talk[h, g] q_g."""
    T = proj.shape[0]
    p = proj.float() + bias.float()
    q = p[:, :H * d].reshape(T, H, d)
    qn = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + eps)
    if own_kv:
        k = p[:, H * d:(H + G) * d].reshape(T, G, d)
        kn = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + eps)
        v = p[:, (H + G) * d:(H + G) * d + G * dv]
        ok = slots >= 0
        idx = slots[ok].long()
        kcache[idx] = kn.reshape(T, G * d)[ok].to(kcache.dtype)
        vcache[idx] = v[ok].to(vcache.dtype)
    rep = H // G
    tk = talk.float().reshape(H, G, rep)                       # [h, c, g in c]
    qm = torch.einsum("hcr,tcrd->thcd", tk, qn.reshape(T, G, rep, d))
    return qm.reshape(T, H * G * d).to(out_dtype)


def score_router(h, w_router, correction, top, n_gate=0):
    """Router of a mixture with un-renormalised softmax weights: logits = h @ w_router[:n].T in
    fp32, s = softmax over all n experts, the ``top`` largest of s + correction are chosen
    (lowest index on ties), their weights are s. The last ``n_gate`` rows of ``w_router`` are
    extra gates: sigmoid(h . row). Returns (weights fp32 [T, top], ids int32, gates [T, n_gate])."""
    n = w_router.shape[0] - n_gate
    z = h.float() @ w_router.float().t()
    sc = torch.softmax(z[:, :n], -1)
    choice = sc + correction.float()
    ids = torch.sort(choice, dim=-1, descending=True, stable=True).indices[:, :top]
    return sc.gather(1, ids), ids.to(torch.int32), torch.sigmoid(z[:, n:])


def moe_experts_f32(x, w_gu, w_down, topk_w, topk_ids, shared=None, act="silu_mul", limit=0.0):
    """Weighted sum of each token's chosen experts, fp32 out. Expert e < E (w_gu [E, 2F, D] =
    gate | up, w_down [E, D, F]) is down(silu(gate) * up); ids >= E are identity experts (the
    input itself). ``shared`` = (ws_gu, ws_down, gate [T]) adds an always-on expert times its
    per-token gate."""
    T, D = x.shape
    E, F2, _ = w_gu.shape
    out = torch.zeros(T, D, dtype=torch.float32, device=x.device)
    for e in range(E):
        rows, slot = (topk_ids == e).nonzero(as_tuple=True)
        if rows.numel() == 0:
            continue
        a = act_mul(linear(x[rows], w_gu[e], out_dtype=torch.float32), F2 // 2, x.dtype, act, limit)
        y = linear(a, w_down[e], out_dtype=torch.float32)
        out.index_add_(0, rows, y * topk_w[rows, slot][:, None])
    wi = (topk_w * (topk_ids >= E)).sum(-1, keepdim=True)
    out += wi * x.float()
    if shared is not None:
        ws_gu, ws_down, gate = shared
        a = act_mul(linear(x, ws_gu, out_dtype=torch.float32), ws_gu.shape[0] // 2, x.dtype,
                    "silu_mul")
        out += gate.float().reshape(T, 1) * linear(a, ws_down, out_dtype=torch.float32)
    return out


# ----------------------------------------------------------------------------- post-norm designs
def prev_tokens(ids, state, slots, cu_seqlens, positions):
    """The token before each row of a step: the row above inside a portion, the sequence's slot
    of ``state`` (int32 [slots]) for a portion's first row, -1 at position 0. The slot then
    receives the portion's last token."""
    prev = torch.full_like(ids, -1)
    cu, sl = cu_seqlens.tolist(), slots.tolist()
    for s in range(len(cu) - 1):
        t0, t1 = cu[s], cu[s + 1]
        if t1 <= t0 or sl[s] < 0:
            continue
        prev[t0 + 1:t1] = ids[t0:t1 - 1]
        if int(positions[t0]) != 0:
            prev[t0] = state[sl[s]]
        state[sl[s]] = ids[t1 - 1]
    return prev


def embedding_bigram(ids, prev, table, bigram, buckets, mul_prev, mul_cur, out_dtype):
    """fp32 rows table[id] + bigram[(prev * mul_prev + id * mul_cur) mod buckets] (row
    ``buckets`` where prev < 0; ``bigram`` None: the first table alone), and their rounding to
    ``out_dtype``."""
    x = table[ids.long()].float()
    if bigram is not None:
        row = (prev.long() * mul_prev + ids.long() * mul_cur) % buckets
        row = torch.where(prev < 0, torch.full_like(row, buckets), row)
        x = x + bigram[row].float()
    return x, x.to(out_dtype)


def postnorm(x, y, w, b, eps, keep, out_dtype, rows_idx=None):
    """Layer norm with weight and bias of keep * x + y (y optional) over the fp32 stream x, in
    place; returns the new rows rounded to ``out_dtype``. With ``rows_idx`` only those rows are
    normed and returned, and x stays as it is."""
    src = x if rows_idx is None else x.index_select(0, rows_idx)
    v = src.float() * keep
    if y is not None:
        v = v + y.float()
    mu = v.mean(-1, keepdim=True)
    var = (v - mu).pow(2).mean(-1, keepdim=True)
    n = (v - mu) * torch.rsqrt(var + eps) * w.float() + b.float()
    if rows_idx is None:
        x.copy_(n)
    return n.to(out_dtype)


def add_rmsnormed(x, y, w, eps, out_dtype):
    """x += y / sqrt(mean(y^2) + eps) * w on the fp32 stream, in place; returns the new x
    rounded to ``out_dtype``."""
    yy = y.float()
    x.add_(yy * torch.rsqrt(yy.pow(2).mean(-1, keepdim=True) + eps) * w.float())
    return x.to(out_dtype)


def side_gate(gate, ids, table, col0, out_dtype):
    """gelu_tanh(gate) * table[id, col0 : col0 + n] for an fp32 projection gate [T, n]."""
    n = gate.shape[1]
    e = table[ids.long()][:, col0:col0 + n].float()
    return (F.gelu(gate.float(), approximate="tanh") * e).to(out_dtype)


def rmsnorm_cols(src, w, eps, out_dtype, gate=None):
    """Rows of the fp32 (column-sliced) matrix ``src`` divided by their RMS, times w (and times
    sigmoid(gate), an fp32 matrix of the same shape, when given)."""
    v = src.float()
    o = v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps) * w.float()
    if gate is not None:
        o = o * torch.sigmoid(gate.float())
    return o.to(out_dtype)


def rotate_pairs(x, positions, inv_freq, rot_dims, half):
    """``half``: dimension i < rot_dims/2 pairs with i + rot_dims/2; else pairs (2i, 2i+1)."""
    if not half:
        return rotate_interleaved(x, positions, inv_freq, rot_dims)
    h = rot_dims // 2
    ang = positions.to(inv_freq.dtype)[:, None] * inv_freq[None, :]
    c, s = ang.cos().float(), ang.sin().float()
    if x.dim() == 3:
        c, s = c[:, None, :], s[:, None, :]
    out = x.clone()
    u, v = x[..., :h], x[..., h:rot_dims]
    out[..., :h] = u * c - v * s
    out[..., h:rot_dims] = v * c + u * s
    return out


def latent_prepare(qproj, kvproj, cw, eps, H, d, dr, r, rot_dims, inv_freq, positions, slots,
                   cache, out_dtype, half):
    """qproj fp32 [T, H*(d+dr)] (heads laid out [d unrotated | dr rotated]); kvproj fp32
    [T, r + dr] = [latent | shared key to rotate] or None (the layer reads another layer's
    cache and writes nothing). Cache row = [normed latent | rotated key]. Returns
    (q_nope [T, H, d], q_rot [T, H, dr])."""
    T = qproj.shape[0]
    q = qproj.float().reshape(T, H, d + dr)
    if kvproj is not None:
        c = kvproj[:, :r].float()
        c = c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps) * cw.float()
        kr = rotate_pairs(kvproj[:, r:r + dr].float(), positions, inv_freq, rot_dims, half)
        ok = slots >= 0
        cache[slots[ok].long()] = torch.cat([c, kr], 1)[ok].to(cache.dtype)
    qr = rotate_pairs(q[:, :, d:], positions, inv_freq, rot_dims, half)
    return q[:, :, :d].to(out_dtype).contiguous(), qr.to(out_dtype)


def head_gate(o, g, out_dtype):
    """o fp32 [T, H, n] times sigmoid(g [T, H]) per head -> [T, H*n]."""
    T, H, n = o.shape
    return (o.float() * torch.sigmoid(g.float())[:, :, None]).reshape(T, H * n).to(out_dtype)


def gla(proj, z, a_bias, tau, norm_w, eps, state, slots, cu_seqlens, positions, H, d, dv,
        out_dtype):
    """Gated linear attention. proj fp32 [T, 2*H*d + 2*H*dv (+ ...)] = [q | k | v | gate];
    z fp32 [T, H*d] the decay's pre-activation (its bias ``a_bias`` is added here). Per head
    S = diag(alpha) S + k v^T with alpha = sigmoid(z + b)^(1/tau), o = S^T (q / sqrt(d)); o is
    RMS-normed over dv times norm_w, then times silu(gate). state fp32 [slots, H, d, dv] is
    updated in place; a portion whose first position is 0 starts from zero."""
    T = proj.shape[0]
    out = torch.zeros(T, H * dv, dtype=torch.float32, device=proj.device)
    cu, sl = cu_seqlens.tolist(), slots.tolist()
    nw = norm_w.float()
    for s in range(len(cu) - 1):
        t0, t1 = cu[s], cu[s + 1]
        if t1 <= t0 or sl[s] < 0:
            continue
        S = state[sl[s]].clone()
        if int(positions[t0]) == 0:
            S.zero_()
        p = proj[t0:t1].float()
        qv = p[:, :H * d].reshape(-1, H, d) * (d ** -0.5)
        kv = p[:, H * d:2 * H * d].reshape(-1, H, d)
        vv = p[:, 2 * H * d:2 * H * d + H * dv].reshape(-1, H, dv)
        gv = p[:, 2 * H * d + H * dv:2 * H * d + 2 * H * dv]
        la = -F.softplus(-(z[t0:t1].float() + a_bias.float())) / tau      # log of the decay
        av = torch.exp(la).reshape(-1, H, d)
        for t in range(t1 - t0):
            S = av[t][:, :, None] * S + kv[t][:, :, None] * vv[t][:, None, :]
            o = torch.einsum("hdv,hd->hv", S, qv[t])
            o = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps) * nw
            out[t0 + t] = o.reshape(H * dv) * F.silu(gv[t])
        state[sl[s]] = S
    return out.to(out_dtype)


def logit_router(h, w_router, bias, top):
    """Router logits h @ w_router^T + bias in fp32; the ``top`` largest are chosen (lowest
    index on ties) and weighted by a softmax renormalised over those ``top`` logits. Returns (weights
    fp32 [T, top], ids int32 [T, top])."""
    z = h.float() @ w_router.float().t() + bias.float()
    order = torch.sort(z, dim=-1, descending=True, stable=True)
    return torch.softmax(order.values[:, :top], -1), order.indices[:, :top].to(torch.int32)


def moe_gelu_experts_f32(x, w_up, w_down, topk_w, topk_ids, shared=None):
    """Weighted sum of each token's chosen ungated experts down(gelu_erf(up x)), fp32 out;
    ``shared`` = (ws_up, ws_down) adds an always-on expert of the same form."""
    T, D = x.shape
    out = torch.zeros(T, D, dtype=torch.float32, device=x.device)
    for e in range(w_up.shape[0]):
        rows, slot = (topk_ids == e).nonzero(as_tuple=True)
        if rows.numel() == 0:
            continue
        a = F.gelu(linear(x[rows], w_up[e], out_dtype=torch.float32)).to(x.dtype)
        out.index_add_(0, rows, linear(a, w_down[e], out_dtype=torch.float32)
                       * topk_w[rows, slot][:, None])
    if shared is not None:
        a = F.gelu(linear(x, shared[0], out_dtype=torch.float32)).to(x.dtype)
        out += linear(a, shared[1], out_dtype=torch.float32)
    return out


# ----------------------------------------------------------------------------- hyper-connected designs
def hyper_mix(xs, y, prev, read, w, eps, w_offset, out_dtype):
    """Hyper-connections over xs fp32 [T, S, D] (in place). ``prev`` / ``read`` are fp32
    vectors [S + S + S*S] = read weights | write weights | stream mix [from, to] of the
    sublayer that produced y and of the one that runs next. With y: every stream becomes
    xs[:, t] = sum_s mix[s, t] xs[:, s] + write[t] * y. With ``read``: u = sum_s read[s] xs[:, s]
    is returned, RMS-normed times (w + w_offset) in ``out_dtype`` when w is given, else as
    fp32."""
    T, S, D = xs.shape
    if y is not None:
        mix = prev[2 * S:].reshape(S, S).float()
        new = torch.einsum("sr,tsd->trd", mix, xs) + prev[S:2 * S].float()[None, :, None] * y.float()[:, None, :]
        xs.copy_(new)
    if read is None:
        return None
    u = torch.einsum("s,tsd->td", read[:S].float(), xs)
    if w is None:
        return u
    h = u * torch.rsqrt(u.pow(2).mean(-1, keepdim=True) + eps) * (w.float() + w_offset)
    return h.to(out_dtype)


def sink_prepare(proj, qw, kw, eps, H, G, d, dv, rot_dims, freq, mscale, positions, kcache,
                 vcache, slots, out_dtype):
    """proj fp32 [T, >= H*d + G*d + G*dv] = [q | k | v | ...]: q and k are RMS-normed over their
    whole rows (all heads at once) times qw / kw, then the first rot_dims dims of every head
    rotate (dimension i with i + rot_dims/2) by positions * freq (float64) with cos and sin
    times mscale; k and v go to the cache rows; returns q [T, H*d]."""
    T = proj.shape[0]
    q = proj[:, :H * d].float()
    k = proj[:, H * d:(H + G) * d].float()
    v = proj[:, (H + G) * d:(H + G) * d + G * dv].float()
    q = (q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + eps) * qw.float()).reshape(T, H, d)
    k = (k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + eps) * kw.float()).reshape(T, G, d)
    if rot_dims:
        hh = rot_dims // 2
        ang = positions.double()[:, None] * freq.double()[None, :]
        c = (ang.cos() * mscale).float()[:, None, :]
        s = (ang.sin() * mscale).float()[:, None, :]

        def rot(x):
            o = x.clone()
            a, b = x[..., :hh], x[..., hh:rot_dims]
            o[..., :hh] = a * c - b * s
            o[..., hh:rot_dims] = b * c + a * s
            return o
        q, k = rot(q), rot(k)
    ok = slots >= 0
    idx = slots[ok].long()
    kcache[idx] = k.reshape(T, G * d)[ok].to(kcache.dtype)
    vcache[idx] = v[ok].to(vcache.dtype)
    return q.reshape(T, H * d).to(out_dtype)


def lightning(proj, decays, state, slots, cu_seqlens, positions, H, d, dv):
    """Linear attention with a fixed decay per head. proj fp32 [T, 2*H*d + H*dv (+ ...)] = [q |
    k | v | ...] before their SiLU; per head S = decay_h S + k v^T, o = S^T q; returns the raw
    read-outs fp32 [T, H*dv]. state fp32 [slots, H, d, dv] in place; a portion whose first
    position is 0 starts from zero."""
    T = proj.shape[0]
    out = torch.zeros(T, H * dv, dtype=torch.float32, device=proj.device)
    cu, sl = cu_seqlens.tolist(), slots.tolist()
    a = decays.float().reshape(H, 1, 1)
    for s in range(len(cu) - 1):
        t0, t1 = cu[s], cu[s + 1]
        if t1 <= t0 or sl[s] < 0:
            continue
        S = state[sl[s]].clone()
        if int(positions[t0]) == 0:
            S.zero_()
        p = F.silu(proj[t0:t1, :2 * H * d + H * dv].float())
        qv = p[:, :H * d].reshape(-1, H, d)
        kv = p[:, H * d:2 * H * d].reshape(-1, H, d)
        vv = p[:, 2 * H * d:].reshape(-1, H, dv)
        for t in range(t1 - t0):
            S = a * S + kv[t][:, :, None] * vv[t][:, None, :]
            out[t0 + t] = torch.einsum("hdv,hd->hv", S, qv[t]).reshape(H * dv)
        state[sl[s]] = S
    return out


def mlstm(proj, if_b, cap, norm_w, eps, state, mstate, slots, cu_seqlens, positions, H, d, dv,
          out, out_scale):
    """Matrix memory with exponential gating. proj fp32 [T, 2*H*d + 2*H*dv + 2*H] = [q | k | v |
    output gate | input gates | forget gates]. Per head, with i = cap tanh((z_i + b_i) / cap),
    f = logsigmoid(cap tanh((z_f + b_f) / cap)) and a running maximum m (0 at the start):
        m' = max(f + m, i);  S = e^(f + m - m') S + e^(i - m') k v^T;  n likewise with k alone;
        o = S^T q d^(-1/2) / (max(|n . q d^(-1/2)|, e^(-m')) + 1e-6)
    o is RMS-normed per head, times norm_w [H*dv], sigmoid(gate) and out_scale, and written to
    ``out`` [T, H*dv]. state fp32 [slots, H, d, dv] holds S; mstate fp32 [slots, H, d + 1] holds
    n and, last, m."""
    T = proj.shape[0]
    cu, sl = cu_seqlens.tolist(), slots.tolist()
    nw = norm_w.float().reshape(H, dv)
    o0 = 2 * H * d
    for s in range(len(cu) - 1):
        t0, t1 = cu[s], cu[s + 1]
        if t1 <= t0:
            continue
        if sl[s] < 0:
            out[t0:t1] = 0
            continue
        S = torch.cat([state[sl[s]], mstate[sl[s]][:, :d, None]], 2)      # [H, d, dv + 1]
        m = mstate[sl[s]][:, d].clone()
        if int(positions[t0]) == 0:
            S.zero_()
            m.zero_()
        p = proj[t0:t1].float()
        qv = p[:, :H * d].reshape(-1, H, d) * (d ** -0.5)
        kv = p[:, H * d:o0].reshape(-1, H, d)
        vv = p[:, o0:o0 + H * dv].reshape(-1, H, dv)
        gv = p[:, o0 + H * dv:o0 + 2 * H * dv].reshape(-1, H, dv)
        b = if_b.float()
        ig = cap * torch.tanh((p[:, o0 + 2 * H * dv:o0 + 2 * H * dv + H] + b[:H]) / cap)
        fg = F.logsigmoid(cap * torch.tanh((p[:, o0 + 2 * H * dv + H:o0 + 2 * H * dv + 2 * H]
                                            + b[H:]) / cap))
        ones = torch.ones(H, 1, dtype=torch.float32, device=proj.device)
        for t in range(t1 - t0):
            m1 = torch.maximum(fg[t] + m, ig[t])
            a, bb = torch.exp(fg[t] + m - m1), torch.exp(ig[t] - m1)
            v1 = torch.cat([vv[t], ones], 1)
            S = a[:, None, None] * S + bb[:, None, None] * kv[t][:, :, None] * v1[:, None, :]
            m = m1
            r = torch.einsum("hdv,hd->hv", S, qv[t])
            o = r[:, :dv] / (torch.maximum(r[:, dv:].abs(), torch.exp(-m)[:, None]) + 1e-6)
            o = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps) * nw
            out[t0 + t] = (o * torch.sigmoid(gv[t]) * out_scale).reshape(H * dv).to(out.dtype)
        state[sl[s]] = S[:, :, :dv]
        mstate[sl[s]] = torch.cat([S[:, :, dv], m[:, None]], 1)
    return out


def group_router(h, w_router, top, groups, keep, wscale):
    """Router over groups of neighbouring experts: s = softmax of the fp32 logits h @ w^T over
    all experts; a group scores its best expert; only experts of the ``keep`` best of
    ``groups`` equal groups can be chosen; the ``top`` largest s among them are chosen (lowest
    index on ties) with weights s * wscale (not renormalised). Returns (weights fp32 [T, top],
    ids int32 [T, top])."""
    z = h.float() @ w_router.float().t()
    s = torch.softmax(z, -1)
    T, E = s.shape
    gs = s.reshape(T, groups, E // groups).max(-1).values
    order = torch.sort(gs, dim=-1, descending=True, stable=True).indices[:, :keep]
    allowed = torch.zeros(T, groups, dtype=torch.bool, device=h.device)
    allowed.scatter_(1, order, True)
    masked = torch.where(allowed.repeat_interleave(E // groups, dim=1), s, torch.full_like(s, -1.0))
    ids = torch.sort(masked, dim=-1, descending=True, stable=True).indices[:, :top]
    return s.gather(1, ids) * wscale, ids.to(torch.int32)


def clamp_swish_mul(gu, F_, limit, out_dtype):
    """g = min(gu[:, :F], limit), u = clamp(gu[:, F:2F], -limit, limit): g sigmoid(1.702 g) (u + 1)."""
    g = gu[:, :F_].float().clamp(max=limit)
    u = gu[:, F_:2 * F_].float().clamp(-limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)).to(out_dtype)
