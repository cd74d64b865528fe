"""Ops of the hybrid model family (models/hybrid.py): fp32 residual stream and norms, grouped
RMS norm, windowed attention with distance bias / head mixing / output gate over token-major
paged caches, latent (compressed-kv) attention in the absorbed form, a gated linear recurrence
with per-sequence state slots, and a shape-agnostic GEMM.

Dispatch is the package's: CUDA (HIP) tensors run the gfx950 kernels (``csrc/kernels``:
hybrid_elementwise.hip, window_attention.hip, recurrent.hip, gemm_any.hip), CPU tensors the
PyTorch reference (``ops/reference.py``). The storage dtype (bf16 when serving, fp32 in the
exact mode) is the dtype of the weights; kernels take it as ``dt``.
"""
from __future__ import annotations

import os
from typing import Optional

import torch

from . import _native as N
from . import gemm as _gemm
from . import reference as R

_call = N.call
_p = N.ptr
_NOT_SUPPORTED = 801            # hipErrorNotSupported: a launcher declining a shape
# DLI_WINATTN_SCALAR=1 keeps bf16 windowed attention on the scalar kernel (A/B, debugging)
MFMA_ATTENTION = os.environ.get("DLI_WINATTN_SCALAR", "0") != "1"


def _dt(dtype: torch.dtype) -> int:
    if dtype == torch.bfloat16:
        return 0
    if dtype == torch.float32:
        return 1
    raise ValueError(f"hybrid ops: storage dtype {dtype} (bfloat16 or float32)")


def _st():
    return N.stream_ptr()


# ----------------------------------------------------------------------------- GEMM
def linear_any(x: torch.Tensor, w: torch.Tensor, out_f32: bool = True,
               out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x [M, K] @ w [N, K]^T with fp32 accumulation -> fp32 (or the storage dtype). bf16 shapes
    the tuned tile family accepts (K a multiple of its K-tile, 16-byte rows) run there; every
    other shape, and fp32 operands, run the shape-agnostic kernel."""
    if not x.is_cuda:
        y = R.linear(x, w, out_dtype=torch.float32 if out_f32 else x.dtype)
        if out is not None:
            out.copy_(y)
            return out
        return y
    M, K = x.shape
    Nn = w.shape[0]
    if x.dtype != w.dtype or w.shape[1] != K or x.stride(1) != 1 or w.stride(1) != 1:
        raise ValueError("linear_any: operand dtypes / inner dims do not match")
    f32 = out_f32 or x.dtype == torch.float32
    if out is None:
        out = torch.empty(M, Nn, dtype=torch.float32 if f32 else x.dtype, device=x.device)
    if (x.dtype == torch.bfloat16 and K % 64 == 0 and x.stride(0) % 8 == 0
            and w.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0
            and out.stride(1) == 1):
        from . import _gemm_native
        return _gemm_native(x, w, "f32" if f32 else "none", out=out)
    _call("dli_gemm_any", _p(x), x.stride(0), _p(w), w.stride(0), _p(out), out.stride(0), M, Nn,
          K, _dt(x.dtype), int(f32), 1, 0, 0, 0, _st())
    return out


def head_linear(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """Per-head projection: out[:, h, :n] = x[:, h, :] @ w[h]^T for x [T, H, k], w [H, n, k],
    out [T, H, >= n] (the result lands in the first n columns of each head's row; x and out may
    be column slices of wider rows). One batched launch."""
    T, H, k = x.shape
    n = w.shape[1]
    if not x.is_cuda:
        y = torch.einsum("thk,hnk->thn", x.float(), w.float())
        out[:, :, :n] = y.to(out.dtype)
        return out
    if x.stride(2) != 1 or w.stride(2) != 1 or out.stride(2) != 1 or x.dtype != w.dtype:
        raise ValueError("head_linear: inner dims must be contiguous")
    _call("dli_gemm_any", _p(x), x.stride(0), _p(w), w.stride(1), _p(out), out.stride(0), T, n, k,
          _dt(x.dtype), int(out.dtype == torch.float32), H, x.stride(1), w.stride(0),
          out.stride(1), _st())
    return out


# ----------------------------------------------------------------------------- rows
def embedding_f32(ids: torch.Tensor, table: torch.Tensor, copy: bool = False,
                  scale: float = 1.0, pos_table: Optional[torch.Tensor] = None,
                  positions: Optional[torch.Tensor] = None):
    """fp32 rows of ``table`` times ``scale``, plus the row ``positions[t]`` of ``pos_table``
    when given (and a second copy when asked: the loop input)."""
    if not table.is_cuda:
        x = table[ids.long()].float() * scale
        if pos_table is not None:
            x = x + pos_table[positions.long()].float()
        return (x, x.clone()) if copy else (x, None)
    T, D = ids.shape[0], table.shape[1]
    x = torch.empty(T, D, dtype=torch.float32, device=table.device)
    x0 = torch.empty_like(x) if copy else None
    _call("dli_embedding_f32", _p(x), _p(x0), _p(ids), _p(table), T, D, table.shape[0],
          float(scale), _p(pos_table), _p(positions),
          pos_table.shape[0] if pos_table is not None else 0, _dt(table.dtype), _st())
    return x, x0


def resadd_groupnorm(x: torch.Tensor, y: Optional[torch.Tensor], w: Optional[torch.Tensor],
                     groups: int, eps: float, mult: float = 1.0, keep: float = 1.0,
                     bias: Optional[torch.Tensor] = None, dtype=None, gain: float = 1.0,
                     out_f32: bool = False, w_offset: float = 0.0) -> Optional[torch.Tensor]:
    """In place on the fp32 stream: x = keep * x + mult * y + bias (y, bias optional); returns
    the grouped RMS norm of the new x times ``w`` times ``gain`` in the storage dtype (None when
    w is None), or unrounded in fp32 with ``out_f32`` (what a token shift reads). ``w_offset``
    is added to the weight in fp32 (weights stored as offsets from one)."""
    dtype = dtype or (w.dtype if w is not None else torch.bfloat16)
    if not x.is_cuda:
        if keep != 1.0:
            x.mul_(keep) if keep != 0.0 else x.zero_()
        if y is not None:
            x.add_(y.float(), alpha=mult)
        if bias is not None:
            x.add_(bias.float())
        if w is None:
            return None
        h = R.group_rmsnorm(x, w, groups, eps, torch.float32, w_offset)
        if gain != 1.0:
            h = h * gain
        return h if out_f32 else h.to(dtype)
    rows, dim = x.shape
    h = (torch.empty(rows, dim, dtype=torch.float32 if out_f32 else dtype, device=x.device)
         if w is not None else None)
    _call("dli_resadd_groupnorm", _p(x), _p(y), y.stride(0) if y is not None else 0, _p(bias),
          float(keep), float(mult), _p(w), _p(h), dim, rows, dim, groups, float(eps), None,
          float(gain), int(out_f32), float(w_offset), _dt(dtype), _st())
    return h


def groupnorm_rows(x: torch.Tensor, rows_idx: torch.Tensor, w: torch.Tensor, groups: int,
                   eps: float, gain: float = 1.0, w_offset: float = 0.0) -> torch.Tensor:
    """Grouped RMS norm (times ``gain``) of the rows ``rows_idx`` (int64) of the fp32 stream."""
    if not x.is_cuda:
        h = R.group_rmsnorm(x.index_select(0, rows_idx), w, groups, eps, torch.float32, w_offset)
        return (h * gain if gain != 1.0 else h).to(w.dtype)
    n, dim = rows_idx.shape[0], x.shape[1]
    h = torch.empty(n, dim, dtype=w.dtype, device=x.device)
    _call("dli_resadd_groupnorm", _p(x), None, 0, None, 1.0, 1.0, _p(w), _p(h), dim, n, dim,
          groups, float(eps), _p(rows_idx), float(gain), 0, float(w_offset), _dt(w.dtype), _st())
    return h


def token_shift(h: torch.Tensor, mu: torch.Tensor, state: torch.Tensor, slots: torch.Tensor,
                cu_seqlens: torch.Tensor, max_seqlen: int, positions: torch.Tensor) -> torch.Tensor:
    """Token shift of the normed rows h (fp32 [T, D]): u_t = h_t + (h_{t-1} - h_t) * mu, in the
    storage dtype of ``mu``. h_{t-1} of a portion's first row comes from the sequence's slot
    of ``state`` (fp32 [slots, D]; zeros at position 0), which then receives the portion's
    last row."""
    if not h.is_cuda:
        return R.token_shift(h, mu, state, slots, cu_seqlens, positions, mu.dtype)
    T, D = h.shape
    S = cu_seqlens.shape[0] - 1
    out = torch.empty(T, D, dtype=mu.dtype, device=h.device)
    _call("dli_token_shift", _p(h), _p(mu), _p(state), _p(slots), _p(cu_seqlens), _p(positions),
          _p(out), S, int(max_seqlen), D, _dt(mu.dtype), _st())
    return out


def concat_cast(a: torch.Tensor, b: torch.Tensor, dtype) -> torch.Tensor:
    """[a ; b] (fp32 [T, D] each) as [T, 2D] in the storage dtype."""
    if not a.is_cuda:
        return torch.cat([a, b], 1).to(dtype)
    T, D = a.shape
    out = torch.empty(T, 2 * D, dtype=dtype, device=a.device)
    _call("dli_concat_cast", _p(out), _p(a), _p(b), T, D, _dt(dtype), _st())
    return out


_ACT_KINDS = {"gelu_mul": 0, "silu_mul": 1, "gelu": 2, "gelu_erf": 3, "copy": 4,
              "clamp_swish": 5}


def act_mul(gu: torch.Tensor, F_: int, dtype, kind: str = "gelu_mul",
            rows: Optional[torch.Tensor] = None, limit: float = 0.0) -> torch.Tensor:
    """The feed-forward's middle for an fp32 projection: ``gelu_mul`` / ``silu_mul`` =
    act(gu[:, :F]) * gu[:, F:2F]; ``gelu`` = gelu_tanh(gu[:, :F]); ``gelu_erf`` = the exact GELU
    of gu[:, :F]; ``copy`` = gu[:, :F] rounded to the storage dtype; ``clamp_swish`` = g
    sigmoid(1.702 g) (u + 1) with g = min(gu[:, :F], limit), u = clamp(gu[:, F:2F], +-limit).
    ``gu`` may also be a bf16 projection (a tuned GEMM's output) when ``dtype`` is bf16.
    ``rows`` (device int32
    scalar): only that many leading rows hold data (routed rows of a mixture)."""
    if not gu.is_cuda:
        return R.act_mul(gu, F_, dtype, kind, limit)
    T = gu.shape[0]
    out = torch.empty(T, F_, dtype=dtype, device=gu.device)
    _call("dli_act_mul", _p(out), F_, _p(gu), gu.stride(0), T, F_, _ACT_KINDS[kind], _p(rows),
          float(limit), _dt(gu.dtype), _dt(dtype), _st())
    return out


def gelu_mul(gu: torch.Tensor, F_: int, dtype) -> torch.Tensor:
    """gelu_tanh(gu[:, :F]) * gu[:, F:2F] for an fp32 [T, 2F] projection."""
    return act_mul(gu, F_, dtype, "gelu_mul")


# ----------------------------------------------------------------------------- mixers
def attn_prepare(proj, qw, kw, eps, H, G, d, kcache, vcache, slots):
    dtype = qw.dtype
    if not proj.is_cuda:
        return R.attn_prepare(proj, qw, kw, eps, H, G, d, kcache, vcache, slots, dtype)
    T = proj.shape[0]
    q = torch.empty(T, H * d, dtype=dtype, device=proj.device)
    _call("dli_attn_prepare", _p(proj), proj.stride(0), _p(qw), _p(kw), float(eps), T, H, G, d,
          _p(q), _p(kcache), _p(vcache), _p(slots), _dt(dtype), _st())
    return q


def talk_prepare(proj, bias, talk, eps, H, G, d, dv, kcache, vcache, slots, own_kv: bool):
    """q / k / v of an attention whose scores are mixed across heads before the softmax (see
    ``reference.talk_prepare``): adds the projection bias, divides q and k heads by their RMS,
    writes k and v to the cache rows (``own_kv``), and returns the mixed queries
    [T, H * G*d] in the storage dtype: head h scores whole key rows."""
    dtype = bias.dtype
    if not proj.is_cuda:
        return R.talk_prepare(proj, bias, talk, eps, H, G, d, dv, kcache, vcache, slots, own_kv,
                              dtype)
    T = proj.shape[0]
    q = torch.empty(T, H * G * d, dtype=dtype, device=proj.device)
    _call("dli_talk_prepare", _p(proj), proj.stride(0), _p(bias), _p(talk), float(eps), T, H, G,
          d, dv, _p(q), _p(kcache) if own_kv else None, _p(vcache) if own_kv else None,
          _p(slots), _dt(dtype), _st())
    return q


def mla_prepare(proj, cw, eps, H, d, dr, r, rot_dims, inv_freq, positions, slots, cache):
    """Returns (q_nope [T, H, d], q_full [T, H, r + dr]) with q_full's rotated tail written;
    its first r columns are for the absorb projection (``head_linear``)."""
    dtype = cw.dtype
    T = proj.shape[0]
    if not proj.is_cuda:
        qn, qr = R.mla_prepare(proj, cw, eps, H, d, dr, r, rot_dims, inv_freq, positions, slots,
                               cache, dtype)
        qf = torch.zeros(T, H, r + dr, dtype=dtype)
        qf[:, :, r:] = qr
        return qn, qf
    qn = torch.empty(T, H, d, dtype=dtype, device=proj.device)
    qf = torch.empty(T, H, r + dr, dtype=dtype, device=proj.device)
    _call("dli_mla_prepare", _p(proj), proj.stride(0), _p(cw), float(eps), T, H, d, dr, r,
          rot_dims, _p(inv_freq), _p(positions), _p(slots), _p(qn), _p(qf), _p(cache),
          _dt(dtype), _st())
    return qn, qf


def window_attention(q, k_cache, v_cache, dq, dv, H, G, cu_seqlens, max_seqlen, positions,
                     block_tables, block_size, window, scale, slopes=None, talk=None, gate=None,
                     chunk: int = 0, k_groups: Optional[int] = None, sink=None,
                     head_gate: bool = False, out_scale: float = 1.0, out=None):
    """See ``reference.window_attention`` / window_attention.hip. q [T, H*dq] (storage dtype);
    caches are token-major rows; returns [T, H*dv] in the storage dtype. ``chunk`` > 0 limits
    a query to the keys of its own block of that many positions; ``k_groups`` is the number of
    key heads per cache row when it is not the number of value heads G. ``sink`` fp32 [H]
    adds exp(sink_h) to head h's softmax denominator; ``head_gate``: the gate is fp32 [T, H],
    one number per head; ``out_scale`` multiplies the output; ``out`` (rows of a wider buffer)
    receives it."""
    Gk = G if k_groups is None else int(k_groups)
    chunk = int(chunk)
    if not q.is_cuda:
        o = R.window_attention(q, k_cache, v_cache, dq, dv, H, G, cu_seqlens, positions,
                               block_tables, block_size, window, scale, slopes, talk, gate,
                               out_dtype=q.dtype, chunk=chunk, k_groups=Gk, sink=sink,
                               head_gate=head_gate, out_scale=out_scale)
        if out is not None:
            out.copy_(o)
            return out
        return o
    T = q.shape[0]
    S = cu_seqlens.shape[0] - 1
    if out is None:
        out = torch.empty(T, H * dv, dtype=q.dtype, device=q.device)
    hg = int(bool(head_gate))
    if q.dtype == torch.bfloat16 and MFMA_ATTENTION:
        # the MFMA form; shapes it does not take (odd head sizes, > 32 heads) fall through
        lib = N.require_native()
        # decode steps of heads that share one cached row per position (latent attention):
        # the heads become the query rows of a one-head problem
        rowhead = int(Gk == 1 and H > 1 and int(max_seqlen) == 1 and talk is None and gate is None
                      and slopes is None and sink is None and q.stride(0) == H * dq)
        nb = lib.dli_window_attention_mfma_workspace_bytes(S, int(max_seqlen), T, H, dv,
                                                           int(min(window, chunk) if chunk else window),
                                                           int(talk is not None), rowhead)
        ws = _gemm.workspace(q.device, nb) if nb else None       # key-split form (decode steps)
        rc = lib.dli_window_attention_mfma(
            _p(q), q.stride(0), _p(k_cache), k_cache.stride(0), _p(v_cache), v_cache.stride(0),
            _p(out), out.stride(0), _p(gate), gate.stride(0) if gate is not None else 0,
            _p(slopes), _p(talk), _p(cu_seqlens), _p(positions), _p(block_tables),
            block_tables.stride(0), block_size, S, int(max_seqlen), H, G, dq, dv, int(window),
            float(scale), T, _p(ws), rowhead, Gk, chunk, _p(sink), hg, float(out_scale), _st())
        if rc == 0:
            return out
        if rc != _NOT_SUPPORTED:
            raise RuntimeError(f"dli_window_attention_mfma failed with hipError {rc}")
    _call("dli_window_attention", _p(q), q.stride(0), _p(k_cache), k_cache.stride(0),
          _p(v_cache), v_cache.stride(0), _p(out), out.stride(0), _p(gate),
          gate.stride(0) if gate is not None else 0, _p(slopes), _p(talk), _p(cu_seqlens),
          _p(positions), _p(block_tables), block_tables.stride(0), block_size, S,
          int(max_seqlen), H, G, dq, dv, int(window), float(scale), Gk, chunk, _p(sink), hg,
          float(out_scale), _dt(q.dtype), _st())
    return out


def hgrn2(proj, f_bias, lower, norm_w, eps, state, slots, cu_seqlens, max_seqlen, positions,
          H, d, dv):
    dtype = norm_w.dtype
    if not proj.is_cuda:
        return R.hgrn2(proj, f_bias, lower, norm_w, eps, state, slots, cu_seqlens, positions,
                       H, d, dv, dtype)
    T = proj.shape[0]
    S = cu_seqlens.shape[0] - 1
    out = torch.empty(T, H * dv, dtype=dtype, device=proj.device)
    _call("dli_hgrn2", _p(proj), proj.stride(0), _p(f_bias), _p(lower), _p(norm_w), float(eps),
          _p(state), _p(slots), _p(cu_seqlens), _p(positions), _p(out), out.stride(0), S,
          int(max_seqlen), H, d, dv, _dt(dtype), _st())
    return out


# ----------------------------------------------------------------------------- mixture of experts
def score_router(h, w_router, correction, top: int, n_gate: int = 0, groups: int = 1,
                 keep: int = 1, wscale: float = 1.0):
    """Router with un-renormalised softmax weights and a choice correction (see
    ``reference.score_router``): (weights fp32 [T, top], ids int32 [T, top], gates fp32
    [T, n_gate]) from one pass over each token's row, logits in fp32. With ``groups`` > 1 only
    the experts of the ``keep`` best groups of neighbours can be chosen (a group scores its
    best expert; ``reference.group_router``); ``wscale`` multiplies the weights."""
    if not h.is_cuda:
        if groups > 1 or wscale != 1.0 or correction is None:
            tw, ti = R.group_router(h, w_router, top, groups, keep, wscale)
            return tw, ti, None
        return R.score_router(h, w_router, correction, top, n_gate)
    T, D = h.shape
    n = w_router.shape[0] - n_gate
    w = torch.empty(T, top, dtype=torch.float32, device=h.device)
    ids = torch.empty(T, top, dtype=torch.int32, device=h.device)
    gates = torch.empty(T, max(n_gate, 1), dtype=torch.float32, device=h.device)
    _call("dli_score_router", _p(w), _p(ids), _p(gates), _p(h), h.stride(0), _p(w_router),
          _p(correction), T, D, n, n_gate, top, int(groups), int(keep), float(wscale),
          _dt(h.dtype), _st())
    return w, ids, gates[:, :n_gate]


def grouped_linear_any(x, w, offsets, src, n: int) -> torch.Tensor:
    """Per-expert projections of routed rows: out[p] = x[src[p]] @ w[e]^T for the permuted rows
    p in [offsets[e], offsets[e+1]) (``src`` None: x is already permuted). x [*, K], w
    [E, N, K], out fp32 [n, N]; rows past offsets[E] are not written."""
    E, Nn, K = w.shape
    out = torch.empty(max(n, 1), Nn, dtype=torch.float32, device=x.device)
    if n > 0:
        _call("dli_gemm_any_grouped", _p(x), x.stride(0), _p(w), w.stride(1), w.stride(0),
              _p(out), out.stride(0), n, Nn, K, _dt(x.dtype), E, _p(offsets), _p(src), _st())
    return out


def moe_experts_f32(x, w_gu, w_down, topk_w, topk_ids, shared=None, act: str = "silu_mul",
                    limit: float = 0.0) -> torch.Tensor:
    """Weighted sum of every token's chosen experts in fp32 (``reference.moe_experts_f32``):
    ids below E run the gated-SiLU experts as grouped GEMMs over the rows sorted by expert, ids
    from E on are identity experts; ``shared`` = (ws_gu, ws_down, gate [T]) adds the always-on
    expert times its gate. No host synchronisation: a captured graph replays it."""
    if not x.is_cuda:
        return R.moe_experts_f32(x, w_gu, w_down, topk_w, topk_ids, shared, act, limit)
    T, D = x.shape
    k = topk_ids.shape[1]
    E, F2, _ = w_gu.shape
    n = T * k
    dev = x.device
    offsets = torch.empty(E + 1, dtype=torch.int32, device=dev)
    pos = torch.empty(n, dtype=torch.int32, device=dev)
    src = torch.empty(max(n, 1), dtype=torch.int32, device=dev)
    _call("dli_moe_align", _p(offsets), _p(pos), _p(src), _p(topk_ids), n, k, 0, E, _st())
    gu = grouped_linear_any(x, w_gu, offsets, src, n)
    act = act_mul(gu, F2 // 2, x.dtype, act, rows=offsets[E:], limit=limit)
    y = grouped_linear_any(act, w_down, offsets, None, n)
    ys = gate = None
    if shared is not None:
        ws_gu, ws_down, gate = shared
        a = act_mul(linear_any(x, ws_gu), ws_gu.shape[0] // 2, x.dtype, "silu_mul")
        ys = linear_any(a, ws_down)
    out = torch.empty(T, D, dtype=torch.float32, device=dev)
    _call("dli_moe_combine_f32", _p(out), _p(y), None, _p(topk_w), _p(pos), _p(topk_ids), _p(x),
          x.stride(0), _p(ys), _p(gate), gate.stride(0) if gate is not None else 0, T, k, D, E,
          _dt(x.dtype), _st())
    return out


def moe_finish(routed, topk_w, topk_ids, x, n_real: int, ys=None, gate=None) -> torch.Tensor:
    """fp32 [T, D]: ``routed`` (the weighted sum of the real experts, storage dtype) + the
    identity experts' share (weights of ids >= n_real) * x + gate * ys (the shared expert)."""
    T, D = x.shape
    if not x.is_cuda:
        out = routed.float() + (topk_w * (topk_ids >= n_real)).sum(-1, keepdim=True) * x.float()
        if ys is not None:
            out = out + gate.float().reshape(T, 1) * ys.float()
        return out
    out = torch.empty(T, D, dtype=torch.float32, device=x.device)
    _call("dli_moe_combine_f32", _p(out), None, _p(routed), _p(topk_w), None, _p(topk_ids),
          _p(x), x.stride(0), _p(ys), _p(gate), gate.stride(0) if gate is not None else 0, T,
          topk_ids.shape[1], D, n_real, _dt(x.dtype), _st())
    return out


# ----------------------------------------------------------------------------- post-norm designs
def prev_tokens(ids, state, slots, cu_seqlens, max_seqlen, positions) -> torch.Tensor:
    """int32 [T]: the token before each row (-1 at position 0). A portion's first row takes it
    from the sequence's slot of ``state`` (int32 [slots]), which then receives the portion's
    last token: the previous token is part of a sequence's state."""
    if not ids.is_cuda:
        return R.prev_tokens(ids, state, slots, cu_seqlens, positions)
    T = ids.shape[0]
    S = cu_seqlens.shape[0] - 1
    prev = torch.empty(T, dtype=torch.int32, device=ids.device)
    _call("dli_prev_tokens", _p(prev), _p(ids), _p(state), _p(slots), _p(cu_seqlens),
          _p(positions), S, int(max_seqlen), _st())
    return prev


def embedding_bigram(ids, prev, table, bigram, buckets: int, mul_prev: int, mul_cur: int):
    """(x fp32 [T, D], x rounded to the storage dtype): table[id] plus the hashed bigram row
    (``reference.embedding_bigram``); ``bigram`` None leaves the first table alone."""
    if not table.is_cuda:
        return R.embedding_bigram(ids, prev, table, bigram, buckets, mul_prev, mul_cur,
                                  table.dtype)
    T, D = ids.shape[0], table.shape[1]
    x = torch.empty(T, D, dtype=torch.float32, device=table.device)
    xb = torch.empty(T, D, dtype=table.dtype, device=table.device)
    if bigram is not None and bigram.shape[0] != buckets + 1:
        raise ValueError("bigram table: buckets + 1 rows")
    _call("dli_embedding_bigram", _p(x), _p(xb), _p(ids), _p(prev), _p(table), _p(bigram), T, D,
          table.shape[0], int(buckets), int(mul_prev), int(mul_cur), _dt(table.dtype), _st())
    return x, xb


def postnorm(x, y, w, b, eps: float, keep: float = 1.0,
             rows_idx: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x = LayerNorm(keep * x + y) * w + b on the fp32 stream, in place (y optional, fp32);
    returns the new rows in the storage dtype (w's). With ``rows_idx`` (int64) only those rows
    are normed and returned and x is left alone."""
    if not x.is_cuda:
        return R.postnorm(x, y, w, b, eps, keep, w.dtype, rows_idx)
    dim = x.shape[1]
    rows = x.shape[0] if rows_idx is None else rows_idx.shape[0]
    h = torch.empty(rows, dim, dtype=w.dtype, device=x.device)
    _call("dli_postnorm", _p(x), _p(y), y.stride(0) if y is not None else 0, float(keep), _p(w),
          _p(b), _p(h), rows, dim, float(eps), _p(rows_idx), _dt(w.dtype), _st())
    return h


def add_rmsnormed(x, y, w, eps: float) -> torch.Tensor:
    """x += y / sqrt(mean(y^2) + eps) * w on the fp32 stream (y fp32); returns the new x in
    the storage dtype."""
    if not x.is_cuda:
        return R.add_rmsnormed(x, y, w, eps, w.dtype)
    rows, dim = x.shape
    h = torch.empty(rows, dim, dtype=w.dtype, device=x.device)
    _call("dli_add_rmsnormed", _p(x), _p(y), y.stride(0), _p(w), _p(h), rows, dim, float(eps),
          _dt(w.dtype), _st())
    return h


def side_gate(gate, ids, table, col0: int) -> torch.Tensor:
    """gelu_tanh(gate) * table[id, col0 : col0 + n] for the fp32 projection gate [T, n], in the
    storage dtype (the table's)."""
    if not gate.is_cuda:
        return R.side_gate(gate, ids, table, col0, table.dtype)
    T, n = gate.shape
    out = torch.empty(T, n, dtype=table.dtype, device=gate.device)
    _call("dli_side_gate", _p(out), _p(gate), gate.stride(0), _p(ids), _p(table),
          table.stride(0), int(col0), T, n, table.shape[0], _dt(table.dtype), _st())
    return out


def rmsnorm_cols(src, w, eps: float, gate=None, groups: int = 1, out=None,
                 out_scale: float = 1.0) -> torch.Tensor:
    """RMS norm times w of the rows of an fp32 matrix that may be a column slice of a wider
    one, times sigmoid(gate) (fp32, same shape, may be a column slice) when given, times
    ``out_scale``; storage dtype out. With ``groups`` > 1 each row is that many equal parts,
    each normed by itself (heads). ``out`` may be a column slice of a wider buffer."""
    if not src.is_cuda:
        T, n = src.shape
        o = R.rmsnorm_cols(src.reshape(T * groups, n // groups),
                           w.reshape(groups, n // groups).repeat(T, 1), eps, torch.float32,
                           gate.reshape(T * groups, n // groups) if gate is not None else None)
        o = (o.reshape(T, n) * out_scale).to(w.dtype)
        if out is not None:
            out.copy_(o)
            return out
        return o
    T, n = src.shape
    if out is None:
        out = torch.empty(T, n, dtype=w.dtype, device=src.device)
    _call("dli_rmsnorm_cols", _p(out), _p(src), src.stride(0), _p(w), T, n // groups,
          float(eps), _p(gate), gate.stride(0) if gate is not None else 0, int(groups),
          out.stride(0), float(out_scale), _dt(w.dtype), _st())
    return out


def latent_prepare(qproj, kvproj, cw, eps, H, d, dr, r, rot_dims, inv_freq, positions, slots,
                   cache, dtype, half: bool):
    """Query / cache preparation of latent attention with the queries and the compressed kv in
    separate fp32 projections (``reference.latent_prepare``); ``kvproj`` None: the cache is
    another layer's and nothing is written. Returns (q_nope [T, H, d], q_full [T, H, r + dr])
    with q_full's rotated tail written."""
    T = qproj.shape[0]
    if not qproj.is_cuda:
        qn, qr = R.latent_prepare(qproj, kvproj, cw, eps, H, d, dr, r, rot_dims, inv_freq,
                                  positions, slots, cache, dtype, half)
        qf = torch.zeros(T, H, r + dr, dtype=dtype)
        qf[:, :, r:] = qr
        return qn, qf
    qn = torch.empty(T, H, d, dtype=dtype, device=qproj.device)
    qf = torch.empty(T, H, r + dr, dtype=dtype, device=qproj.device)
    own = kvproj is not None
    _call("dli_latent_prepare", _p(qproj), qproj.stride(0), _p(kvproj),
          kvproj.stride(0) if own else 0, _p(cw) if own else None, float(eps), T, H, d, dr, r,
          rot_dims, _p(inv_freq), _p(positions), _p(slots), _p(qn), _p(qf),
          _p(cache) if own else None, int(half), _dt(dtype), _st())
    return qn, qf


def head_gate(o, g, dtype) -> torch.Tensor:
    """o fp32 [T, H, n] times sigmoid(g[t, h]) (g an fp32 column slice [T, H]) -> storage
    dtype [T, H*n]."""
    if not o.is_cuda:
        return R.head_gate(o, g, dtype)
    T, H, n = o.shape
    out = torch.empty(T, H * n, dtype=dtype, device=o.device)
    _call("dli_head_gate", _p(out), _p(o), _p(g), g.stride(0), T, H, n, _dt(dtype), _st())
    return out


def gla(proj, z, a_bias, tau: float, norm_w, eps, state, slots, cu_seqlens, max_seqlen,
        positions, H, d, dv):
    """Gated linear attention over per-sequence state slots (``reference.gla``): proj fp32
    [T, q | k | v | gate | ...], z fp32 [T, H*d]; returns the normed, gated read-out
    [T, H*dv] in the storage dtype."""
    dtype = norm_w.dtype
    if not proj.is_cuda:
        return R.gla(proj, z, a_bias, tau, norm_w, eps, state, slots, cu_seqlens, positions,
                     H, d, dv, dtype)
    T = proj.shape[0]
    S = cu_seqlens.shape[0] - 1
    out = torch.empty(T, H * dv, dtype=dtype, device=proj.device)
    _call("dli_gla", _p(proj), proj.stride(0), _p(z), z.stride(0), _p(a_bias), float(1.0 / tau),
          float(d ** -0.5), _p(norm_w), float(eps), _p(state), _p(slots), _p(cu_seqlens),
          _p(positions), _p(out), out.stride(0), S, int(max_seqlen), H, d, dv, _dt(dtype), _st())
    return out


def logit_router(h, w_router, bias, top: int):
    """(weights fp32 [T, top], ids int32 [T, top]): fp32 logits h . w + bias, the ``top``
    largest chosen (lowest index on ties), softmax over the chosen ones."""
    if not h.is_cuda:
        return R.logit_router(h, w_router, bias, top)
    T, D = h.shape
    n = w_router.shape[0]
    w = torch.empty(T, top, dtype=torch.float32, device=h.device)
    ids = torch.empty(T, top, dtype=torch.int32, device=h.device)
    _call("dli_logit_router", _p(w), _p(ids), _p(h), h.stride(0), _p(w_router), _p(bias), T, D,
          n, top, _dt(h.dtype), _st())
    return w, ids


def moe_gelu_experts_f32(x, w_up, w_down, topk_w, topk_ids, shared=None) -> torch.Tensor:
    """Weighted sum of every token's chosen ungated experts down(gelu_erf(up x)) in fp32, as
    grouped GEMMs over the rows sorted by expert; ``shared`` = (ws_up, ws_down) adds the
    always-on expert. No host synchronisation."""
    if not x.is_cuda:
        return R.moe_gelu_experts_f32(x, w_up, w_down, topk_w, topk_ids, shared)
    T, D = x.shape
    k = topk_ids.shape[1]
    E, F_, _ = w_up.shape
    n = T * k
    dev = x.device
    offsets = torch.empty(E + 1, dtype=torch.int32, device=dev)
    pos = torch.empty(n, dtype=torch.int32, device=dev)
    src = torch.empty(max(n, 1), dtype=torch.int32, device=dev)
    _call("dli_moe_align", _p(offsets), _p(pos), _p(src), _p(topk_ids), n, k, 0, E, _st())
    up = grouped_linear_any(x, w_up, offsets, src, n)
    act = act_mul(up, F_, x.dtype, "gelu_erf", rows=offsets[E:])
    y = grouped_linear_any(act, w_down, offsets, None, n)
    ys = None
    if shared is not None:
        a = act_mul(linear_any(x, shared[0]), shared[0].shape[0], x.dtype, "gelu_erf")
        ys = linear_any(a, shared[1])
    out = torch.empty(T, D, dtype=torch.float32, device=dev)
    _call("dli_moe_combine_f32", _p(out), _p(y), None, _p(topk_w), _p(pos), _p(topk_ids), _p(x),
          x.stride(0), _p(ys), None, 0, T, k, D, E, _dt(x.dtype), _st())
    return out


# ----------------------------------------------------------------------------- hyper-connected designs
def hyper_mix(xs, y, prev, read, w, eps: float = 0.0, w_offset: float = 0.0, dtype=None):
    """One step of hyper-connections on the fp32 streams xs [T, S, D], in place
    (``reference.hyper_mix``): with y (a sublayer's fp32 output) and ``prev`` (that sublayer's
    fp32 vector read | write | mix) the streams are mixed and receive y; with ``read`` (the next
    sublayer's vector, or ones for the plain sum) the weighted sum of the new streams is
    returned — RMS-normed times (w + w_offset) in the storage dtype when w is given, else fp32."""
    if not xs.is_cuda:
        return R.hyper_mix(xs, y, prev, read, w, eps, w_offset, dtype or (w.dtype if w is not None else None))
    T, S, D = xs.shape
    h = None
    if read is not None:
        h = torch.empty(T, D, dtype=torch.float32 if w is None else w.dtype, device=xs.device)
    _call("dli_hyper_mix", _p(xs), _p(y), y.stride(0) if y is not None else 0, _p(prev),
          _p(read), _p(w), _p(h), T, S, D, float(eps), float(w_offset),
          _dt(w.dtype) if w is not None else 1, _st())
    return h


def sink_prepare(proj, qw, kw, eps, H, G, d, dv, rot_dims, freq, mscale, positions, kcache,
                 vcache, slots):
    """Query / cache preparation of an attention whose q and k are RMS-normed over the whole
    projection and partly rotated (``reference.sink_prepare``): k and v go to the cache rows,
    the queries [T, H*d] come back in the storage dtype."""
    dtype = qw.dtype
    if not proj.is_cuda:
        return R.sink_prepare(proj, qw, kw, eps, H, G, d, dv, rot_dims, freq, mscale, positions,
                              kcache, vcache, slots, dtype)
    T = proj.shape[0]
    q = torch.empty(T, H * d, dtype=dtype, device=proj.device)
    _call("dli_sink_prepare", _p(proj), proj.stride(0), _p(qw), _p(kw), float(eps), T, H, G, d,
          dv, int(rot_dims), _p(freq), float(mscale), _p(positions), _p(q), _p(kcache),
          _p(vcache), _p(slots), _dt(dtype), _st())
    return q


def lightning(proj, decays, state, slots, cu_seqlens, max_seqlen, positions, H, d, dv):
    """Linear attention with one fixed decay per head over per-sequence state slots
    (``reference.lightning``): the raw read-outs fp32 [T, H*dv]."""
    if not proj.is_cuda:
        return R.lightning(proj, decays, state, slots, cu_seqlens, positions, H, d, dv)
    T = proj.shape[0]
    S = cu_seqlens.shape[0] - 1
    out = torch.empty(T, H * dv, dtype=torch.float32, device=proj.device)
    _call("dli_scalar_recurrence", _p(proj), proj.stride(0), 0, _p(decays), None, 0.0, None, 0.0,
          _p(state), None, _p(slots), _p(cu_seqlens), _p(positions), _p(out), out.stride(0), 1.0,
          S, int(max_seqlen), H, d, dv, _column_block(S, H, d, dv, max_seqlen), None, 1, _st())
    return out


def _column_block(S: int, H: int, d: int, dv: int, max_seqlen: int) -> int:
    """State columns per workgroup of a recurrence over a step's portions: few (head,
    sequence) pairs with long portions leave most of the chip idle, so the columns are dealt
    to several workgroups (0: one workgroup holds all of them). States too wide for one
    workgroup's registers (d in 16 / 32 / 64 / 128) or LDS (any other d) are always dealt."""
    if S * H < 256 and max_seqlen >= 64 and dv >= 128:
        return 64
    if d in (16, 32, 64, 128):
        return 256 if dv > 256 else 0
    return 64 if dv > 64 and d * ((dv + 63) // 64 * 64) * 4 > 96 * 1024 else 0


def mlstm(proj, if_b, cap: float, norm_w, eps: float, state, mstate, slots, cu_seqlens,
          max_seqlen, positions, H, d, dv, out, out_scale: float = 1.0):
    """Matrix memory with exponential gating over per-sequence state slots
    (``reference.mlstm``); the normed, gated, scaled read-out is written to ``out`` [T, H*dv]
    (storage dtype; may be a column slice of a wider buffer). ``state`` fp32 [slots, H, d, dv];
    ``mstate`` fp32 [slots, H, d + 1] holds the normaliser vector and the running maximum."""
    if not proj.is_cuda:
        return R.mlstm(proj, if_b, cap, norm_w, eps, state, mstate, slots, cu_seqlens, positions,
                       H, d, dv, out, out_scale)
    S = cu_seqlens.shape[0] - 1
    cw = _column_block(S, H, d, dv, max_seqlen)
    # with column blocks no workgroup sees a whole head: the read-outs leave in fp32 and the
    # per-head norm, gate and scale run as a row kernel
    raw = torch.empty(proj.shape[0], H * dv, dtype=torch.float32, device=proj.device) if cw else None
    _call("dli_scalar_recurrence", _p(proj), proj.stride(0), 1, None, _p(if_b), float(cap),
          _p(norm_w), float(eps), _p(state), _p(mstate), _p(slots), _p(cu_seqlens),
          _p(positions), _p(out), out.stride(0), float(out_scale), S, int(max_seqlen), H, d, dv,
          cw, _p(raw), _dt(norm_w.dtype), _st())
    if cw:
        g0 = 2 * H * d + H * dv
        rmsnorm_cols(raw, norm_w, eps, gate=proj[:, g0:g0 + H * dv], groups=H, out=out,
                     out_scale=out_scale)
    return out
