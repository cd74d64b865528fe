"""Sequence mixers of the hybrid (layer-list) model family, one function per kind.

Every mixer maps the normed layer input ``h`` [T, D] (storage dtype) to the layer's update
[T, D] in fp32, reading and writing its run's cache or state. They share one calling form so a
design lists its layers by kind (``MIXERS``):

    y = MIXERS[spec.kind](spec, lp, h, step, cache, eps)

``lp``: the layer's tensors (``models/weights.hybrid_layer_shapes``) plus the constants
derived at load time (``derive_constants``); ``step``: the per-step metadata (``StepView``);
``cache``: this run's entry of ``engine.kv_cache.HybridCache``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

from ..ops import hybrid as H
from .configs import LayerSpec


@dataclass
class StepView:
    """What the mixers need of a step: packed tokens of S sequences, each a run of consecutive
    rows [cu[s], cu[s+1]) at consecutive positions, attending through its block table."""
    cu_seqlens: torch.Tensor        # [S+1] int32
    max_seqlen: int
    positions: torch.Tensor         # [T] int32
    slot_mapping: torch.Tensor      # [T] int32, cache row of each token (-1: not stored)
    block_tables: torch.Tensor      # [S, W] int32
    block_size: int
    state_slots: Optional[torch.Tensor]   # [S] int32 recurrent-state slot (-1: padding row)
    max_context: int = 1 << 30      # no position of this step is at or beyond this


def derive_constants(spec: LayerSpec, lp: dict, device) -> None:
    """Constants a design fixes by formula, computed once (float64 on the host, stored fp32)."""
    if spec.kind == "attention":
        # per-head slope of the linear distance bias: 2^(-8 (h+1) / H)
        h = torch.arange(1, spec.heads + 1, dtype=torch.float64)
        lp["slopes"] = torch.pow(2.0, -8.0 * h / spec.heads).float().to(device)
        lp["talk"] = lp["talk"].float().contiguous()
    elif spec.kind == "latent_attention":
        # float64: the angle position * frequency is formed in double and rounded once
        i = torch.arange(spec.rot_dims // 2, dtype=torch.float64)
        lp["inv_freq"] = torch.pow(spec.rot_base, -2.0 * i / max(1, spec.rot_dims)).to(device)
    elif spec.kind == "talk_attention":
        lp["talk"] = lp["talk"].float().contiguous()
    elif spec.kind == "lightning":
        lp["decays"] = torch.tensor(spec.decays, dtype=torch.float64).float().to(device)
    elif spec.kind == "parallel":
        freq, mscale = yarn_frequencies(spec.left.rot_dims, spec.left.rot_base,
                                        spec.left.rot_scaling)
        lp["rot_freq"], lp["rot_mscale"] = freq.to(device), mscale
        lp["sink"] = lp["sink"].float().contiguous()
        lp["if_b"] = lp["if_b"].float().contiguous()
    if spec.ff_kind == "moe" and spec.ff and spec.router == "score" and "correction" in lp:
        lp["correction"] = lp["correction"].float().contiguous()
    if spec.ff_kind == "moe" and spec.ff and spec.router == "logit_topk":
        lp["router_b"] = lp["router_b"].float().contiguous()


def yarn_frequencies(dims: int, base: float, scaling: tuple = ()):
    """(float64 frequency of every rotated pair, factor on cos and sin). Pair i turns by
    position * base^(-2i/dims). With YaRN scaling (factor, original length, fast turns, slow
    turns) a pair that makes more than ``fast`` turns over the original length keeps its
    frequency, one that makes fewer than ``slow`` is slowed by ``factor``, with a linear ramp
    over the pair index between the two, and cos / sin grow by 0.1 ln(factor) + 1."""
    import math
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = torch.pow(torch.tensor(base, dtype=torch.float64), -2.0 * i / max(1, dims))
    if not scaling or not dims:
        return f, 1.0
    factor, orig, fast, slow = scaling

    def pair_at(turns):          # the (fractional) pair index that makes this many turns
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(pair_at(fast)), 0)
    hi = min(math.ceil(pair_at(slow)), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def attention_mixer(spec: LayerSpec, lp: dict, h, step: StepView, cache, eps: float):
    """Windowed softmax attention: per-head RMS-normed q / k, values = the un-normed keys,
    linear distance bias, the heads' softmax weights mixed by ``talk``, sigmoid output gate."""
    Hh, G, d = spec.heads, spec.kv_heads, spec.dim
    kc, vc = cache
    proj = H.linear_any(h, lp["w_in"])                       # fp32 [T, q | k | gate]
    q = H.attn_prepare(proj, lp["q_norm"], lp["k_norm"], eps, Hh, G, d, kc, vc,
                       step.slot_mapping)
    gate = proj[:, (Hh + G) * d:]
    o = H.window_attention(q, kc, vc, d, d, Hh, G, step.cu_seqlens, step.max_seqlen,
                           step.positions, step.block_tables, step.block_size, spec.window,
                           spec.scale, slopes=lp["slopes"], talk=lp["talk"], gate=gate)
    return H.linear_any(o, lp["wo"])


def hgrn2_mixer(spec: LayerSpec, lp: dict, h, step: StepView, cache, eps: float):
    """Gated linear recurrence: the forget gate (bounded below by ``lower``) also sets what is
    written; per-head RMS norm of the read-out."""
    (state,) = cache
    proj = H.linear_any(h, lp["w_in"])                       # fp32 [T, q | f | v]
    o = H.hgrn2(proj, lp["f_b"], lp["lower"], lp["o_norm"], eps, state, step.state_slots,
                step.cu_seqlens, step.max_seqlen, step.positions, spec.heads, spec.dim,
                spec.vdim)
    return H.linear_any(o, lp["wo"])


def latent_attention_mixer(spec: LayerSpec, lp: dict, h, step: StepView, cache, eps: float):
    """Latent attention in the absorbed form. Only the normed latent c and the shared rotated
    key are cached. With k_h = W_uk,h c and v_h = W_uv,h c,
        q_h . k_h = (W_uk,h^T q_h) . c      and      sum_j w_j v_h,j = W_uv,h (sum_j w_j c_j),
    so every head attends the same cached row [c | k_rot] with the query [W_uk,h^T q_h | q_rot]
    and its output is expanded afterwards: one multi-query attention over the latent, for
    prompts and decoding alike, and no per-step expansion of the window's keys."""
    Hh, d, dr, dv, r = spec.heads, spec.dim, spec.rot_dim, spec.vdim, spec.kv_rank
    (c,) = cache
    T = h.shape[0]
    proj = H.linear_any(h, lp["w_in"])
    gates = None
    if spec.q_rank or spec.head_gate or spec.kv_from >= 0 or spec.rot_half:
        # fp32 [T, query latent (or q heads) | ckv | k_rot (own cache only) | head gates]
        nq = spec.q_rank or Hh * (d + dr)
        qproj = proj[:, :nq]
        if spec.q_rank:                     # queries through an RMS-normed latent
            qproj = H.linear_any(H.rmsnorm_cols(qproj, lp["q_norm"], eps), lp["w_uq"])
        own = spec.kv_from < 0
        kvproj = proj[:, nq:nq + r + dr] if own else None
        if spec.head_gate:
            g0 = nq + (r + dr if own else 0)
            gates = proj[:, g0:g0 + Hh]
        q_nope, q_full = H.latent_prepare(qproj, kvproj, lp.get("c_norm"), eps, Hh, d, dr, r,
                                          spec.rot_dims, lp["inv_freq"], step.positions,
                                          step.slot_mapping, c, h.dtype, spec.rot_half)
    else:                                   # fp32 [T, q heads | ckv | k_rot]
        q_nope, q_full = H.mla_prepare(proj, lp["c_norm"], eps, Hh, d, dr, r, spec.rot_dims,
                                       lp["inv_freq"], step.positions, step.slot_mapping, c)
    H.head_linear(q_nope, lp["w_ukT"], q_full)               # q_full[:, h, :r] = W_uk,h^T q_h
    # a window no shorter than the step's longest context masks nothing: the tight bound lets
    # the kernel size its slot table and key splits for the keys that exist
    win = min(spec.window, max(1, step.max_context))
    ol = H.window_attention(q_full.view(T, Hh * (r + dr)), c, c, r + dr, r, Hh, 1,
                            step.cu_seqlens, step.max_seqlen, step.positions,
                            step.block_tables, step.block_size, win, spec.scale)
    if gates is not None:                   # one sigmoid gate per head, on the fp32 expansion
        o32 = torch.empty(T, Hh, dv, dtype=torch.float32, device=h.device)
        H.head_linear(ol.view(T, Hh, r), lp["w_uv"], o32)
        return H.linear_any(H.head_gate(o32, gates, h.dtype), lp["wo"])
    o = torch.empty(T, Hh, dv, dtype=h.dtype, device=h.device)
    H.head_linear(ol.view(T, Hh, r), lp["w_uv"], o)
    return H.linear_any(o.view(T, Hh * dv), lp["wo"])


def gla_mixer(spec: LayerSpec, lp: dict, h, step: StepView, cache, eps: float):
    """Gated linear attention: independent keys, a per-channel decay sigmoid(z)^(1/tau) with z
    from a two-step low-rank projection, per-head RMS norm of the read-out, SiLU output gate.
    The projections run in the storage dtype; the decay, the state and the norm in fp32."""
    (state,) = cache
    Hh, d, dv = spec.heads, spec.dim, spec.vdim
    proj = H.linear_any(h, lp["w_in"])          # fp32 [T, q | k | v | gate | decay-in]
    a0 = 2 * Hh * (d + dv)
    a1 = H.act_mul(proj[:, a0:], spec.decay_rank, h.dtype, "copy")
    z = H.linear_any(a1, lp["w_a2"])
    o = H.gla(proj, z, lp["a_b"], spec.tau, lp["o_norm"], eps, state, step.state_slots,
              step.cu_seqlens, step.max_seqlen, step.positions, Hh, d, dv)
    return H.linear_any(o, lp["wo"])


def talk_attention_mixer(spec: LayerSpec, lp: dict, h, step: StepView, cache, eps: float):
    """Softmax attention inside blocks of ``spec.chunk`` positions: biased q / k / v, unit-RMS
    q and k, the heads' scores mixed by ``talk`` before the softmax. The mixing is folded into
    the queries (``ops.hybrid.talk_prepare``), so the attention itself is the plain kernel with
    one key head spanning the cached row and G value heads. ``cache`` may be another layer's
    (``spec.kv_from``): then only queries are projected."""
    Hh, G, d, dv = spec.heads, spec.kv_heads, spec.dim, spec.vdim
    kc, vc = cache
    proj = H.linear_any(h, lp["w_in"])                       # fp32 [T, q (| k | v)]
    q = H.talk_prepare(proj, lp["b_in"], lp["talk"], eps, Hh, G, d, dv, kc, vc,
                       step.slot_mapping, own_kv=spec.kv_from < 0)
    o = H.window_attention(q, kc, vc, G * d, dv, Hh, G, step.cu_seqlens, step.max_seqlen,
                           step.positions, step.block_tables, step.block_size,
                           spec.window or (1 << 30), spec.scale, chunk=spec.chunk, k_groups=1)
    return H.linear_any(o, lp["wo"])


def lightning_mixer(spec: LayerSpec, lp: dict, h, step: StepView, cache, eps: float):
    """Linear attention with one fixed decay per head: SiLU on q / k / v, the state and its
    read-out in fp32, all heads RMS-normed together, sigmoid output gate."""
    (state,) = cache
    Hh, d, dv = spec.heads, spec.dim, spec.vdim
    proj = H.linear_any(h, lp["w_in"])                       # fp32 [T, q | k | v | gate]
    o = H.lightning(proj, lp["decays"], state, step.state_slots, step.cu_seqlens,
                    step.max_seqlen, step.positions, Hh, d, dv)
    g0 = 2 * Hh * d + Hh * dv
    return H.linear_any(H.rmsnorm_cols(o, lp["o_norm"], eps, gate=proj[:, g0:g0 + Hh * dv]),
                        lp["wo"])


def parallel_mixer(spec: LayerSpec, lp: dict, h, step: StepView, cache, eps: float):
    """Two mixers on the same input, summed with fixed scales: causal grouped-query attention
    (whole-row q / k norm, partial rotation, a sink logit per head, a sigmoid gate per head)
    and a matrix memory with exponential gating. One fused input projection; both sides write
    their gated, scaled outputs side by side, so one output GEMM over [left | right] sums them."""
    l, r = spec.left, spec.right
    kc, vc, state, mstate = cache
    T = h.shape[0]
    proj = H.linear_any(h, lp["w_in"])
    nl = l.heads * l.dim + l.kv_heads * (l.dim + l.vdim)
    q = H.sink_prepare(proj, lp["q_norm"], lp["k_norm"], eps, l.heads, l.kv_heads, l.dim,
                       l.vdim, l.rot_dims, lp["rot_freq"], lp["rot_mscale"], step.positions,
                       kc, vc, step.slot_mapping)
    wl, wr = l.heads * l.vdim, r.heads * r.vdim
    o = torch.empty(T, wl + wr, dtype=h.dtype, device=h.device)
    # causal, unwindowed: a window as long as the step's longest context masks nothing
    win = min(l.window or (1 << 30), max(1, step.max_context))
    H.window_attention(q, kc, vc, l.dim, l.vdim, l.heads, l.kv_heads, step.cu_seqlens,
                       step.max_seqlen, step.positions, step.block_tables, step.block_size,
                       win, l.scale, gate=proj[:, nl:nl + l.heads], sink=lp["sink"],
                       head_gate=True, out_scale=spec.left_scale, out=o[:, :wl])
    H.mlstm(proj[:, nl + l.heads:], lp["if_b"], r.gate_cap, lp["o_norm"], eps, state, mstate,
            step.state_slots, step.cu_seqlens, step.max_seqlen, step.positions, r.heads, r.dim,
            r.vdim, o[:, wl:], spec.right_scale)
    return H.linear_any(o, lp["wo"])


MIXERS = {"attention": attention_mixer, "hgrn2": hgrn2_mixer,
          "latent_attention": latent_attention_mixer, "talk_attention": talk_attention_mixer,
          "gla": gla_mixer, "lightning": lightning_mixer, "parallel": parallel_mixer}


# ----------------------------------------------------------------------------- feed-forwards
# Two layouts of a feed-forward's weights. The plain one ([gate | up] stacked) runs the
# shape-agnostic GEMM with fp32 outputs and separate activation kernels: any sizes, bf16 or
# fp32. The tuned one (``prepare_feed_forward``: bf16, sizes the tile family takes) fuses the
# activation into the first GEMM's epilogue — SiLU * up over the 16-row interleaved gate/up
# weight, bias + GELU for the ungated form — and runs the experts as the grouped GEMMs of the
# framework's other mixture model.
def prepare_feed_forward(spec: LayerSpec, params: dict, pre: str) -> None:
    """Re-lay the feed-forward weights of layer ``pre`` for the tuned GEMMs when they fit
    (in ``params``, in place; marked by ``<pre>ff_tuned`` so that it happens once). Ungated
    experts (``expert_act`` = ``gelu_erf``) need no re-layout: their activation is an epilogue
    of the plain weight."""
    from ..ops.reference import interleave_gate_up
    w = params.get(pre + "w_down")
    if (not spec.ff or w is None or pre + "ff_tuned" in params or w.dtype != torch.bfloat16
            or not w.is_cuda or spec.ff_kind not in ("gelu", "moe", "gated_silu")
            or w.shape[-2] % 64 or spec.ff % 64 or spec.shared_ff % 64):
        return
    if spec.ff_kind == "gelu":
        params[pre + "b_up"] = torch.zeros(spec.ff, dtype=w.dtype, device=w.device)
    elif spec.ff_kind == "gated_silu":
        gu = params[pre + "w_gu"]
        params[pre + "w_gu"] = interleave_gate_up(gu[:spec.ff], gu[spec.ff:]).contiguous()
    elif spec.ff_kind == "moe" and spec.expert_act == "clamp_swish":
        pass                                         # the plain [gate | up] weight serves
    elif spec.expert_act == "silu_mul":
        gu = params[pre + "w_gu"]
        for e in range(gu.shape[0]):                 # expert by expert: no second full copy
            gu[e] = interleave_gate_up(gu[e, :spec.ff].clone(), gu[e, spec.ff:].clone())
        if spec.shared_ff:
            s = params[pre + "ws_gu"]
            params[pre + "ws_gu"] = interleave_gate_up(s[:spec.shared_ff], s[spec.shared_ff:]).contiguous()
    params[pre + "ff_tuned"] = torch.ones(1, dtype=torch.int8, device=w.device)


def gated_gelu_ff(spec: LayerSpec, lp: dict, h):
    act = H.act_mul(H.linear_any(h, lp["w_gu"]), spec.ff, h.dtype, "gelu_mul")
    return H.linear_any(act, lp["w_down"])


def gelu_ff(spec: LayerSpec, lp: dict, h):
    if "ff_tuned" in lp:
        from .. import ops
        act = ops.linear(h, lp["w_up"], lp["b_up"], epi="bias_gelu")
    else:
        act = H.act_mul(H.linear_any(h, lp["w_up"]), spec.ff, h.dtype, "gelu")
    return H.linear_any(act, lp["w_down"])


def gated_silu_ff(spec: LayerSpec, lp: dict, h):
    if "ff_tuned" in lp:
        from .. import ops
        act = ops.linear(h, lp["w_gu"], epi="silu_mul")
    else:
        act = H.act_mul(H.linear_any(h, lp["w_gu"]), spec.ff, h.dtype, "silu_mul")
    return H.linear_any(act, lp["w_down"])


def moe_ff(spec: LayerSpec, lp: dict, h):
    """Routed gated-SiLU experts + identity experts + a gated shared expert, summed in fp32;
    with ``router`` = ``logit_topk``: biased logits, softmax over the chosen, ungated exact-GELU
    experts and an always-on shared expert; with ``router`` = ``group_score``: group-limited
    choice, scaled scores, clamped-swish experts."""
    if spec.router == "group_score":
        tw, ti, _ = H.score_router(h, lp["router"], None, spec.top, 0, spec.router_groups,
                                   spec.router_keep, spec.router_scale)
        if "ff_tuned" not in lp:
            return H.moe_experts_f32(h, lp["w_gu"], lp["w_down"], tw, ti, None,
                                     act="clamp_swish", limit=spec.act_limit)
        from .. import ops
        routed = ops.moe_mlp(h, lp["w_gu"], lp["w_down"], tw, ti, 0, act="clamp_swish",
                             limit=spec.act_limit)
        return H.moe_finish(routed, tw, ti, h, lp["w_gu"].shape[0])
    if spec.router == "logit_topk":
        tw, ti = H.logit_router(h, lp["router"], lp["router_b"], spec.top)
        if "ff_tuned" not in lp:
            shared = (lp["ws_up"], lp["ws_down"]) if spec.shared_ff else None
            return H.moe_gelu_experts_f32(h, lp["w_up"], lp["w_down"], tw, ti, shared)
        from .. import ops
        routed = ops.moe_mlp(h, lp["w_up"], lp["w_down"], tw, ti, 0, act="gelu_erf")
        ys = None
        if spec.shared_ff:
            ys = H.linear_any(ops.linear(h, lp["ws_up"], epi="gelu_erf"), lp["ws_down"])
        return H.moe_finish(routed, tw, ti, h, lp["w_up"].shape[0], ys, None)
    ng = 1 if spec.shared_ff else 0
    tw, ti, gates = H.score_router(h, lp["router"], lp["correction"], spec.top, ng)
    if "ff_tuned" not in lp:
        shared = (lp["ws_gu"], lp["ws_down"], gates) if ng else None
        return H.moe_experts_f32(h, lp["w_gu"], lp["w_down"], tw, ti, shared)
    from .. import ops
    # ids from E on (identity experts) match no local expert and add nothing here
    routed = ops.moe_mlp(h, lp["w_gu"], lp["w_down"], tw, ti, 0)
    ys = None
    if ng:
        ys = H.linear_any(ops.linear(h, lp["ws_gu"], epi="silu_mul"), lp["ws_down"])
    return H.moe_finish(routed, tw, ti, h, lp["w_gu"].shape[0], ys, gates if ng else None)


FEED_FORWARDS = {"gated_gelu": gated_gelu_ff, "gelu": gelu_ff, "moe": moe_ff,
                 "gated_silu": gated_silu_ff}
