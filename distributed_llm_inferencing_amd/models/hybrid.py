"""Hybrid decoder (archs ``buborax``, ``pulunex``, ``risutar``, ``lapunex``): a layer list that
mixes windowed attention, latent attention, gated linear recurrences (HGRN2, gated linear
attention, fixed-decay linear attention, a matrix memory beside a sink attention) and block
attention with head-mixed scores; dense, gated and routed feed-forwards; a shared-weight loop,
grouped RMS norms, token shift and an fp32 residual stream (or several hyper-connected
streams) — served by the same engine, scheduler, block manager and runner as the transformer
families.

    embed (fp32) -> per layer run: x += m * mixer(gnorm(x)); x += m * ff(gnorm(x))
                 -> gnorm -> LM head (fp32 logits) -> sampler

Post-norm designs (``cfg.post_norm``; ``risutar``) run

    embed + hashed bigram (fp32) -> per layer: x = LN(a x + mixer(x)); x = LN(a x + ff(x));
                 x += rmsnorm(side_proj(gelu(side_gate x) * side_embed[token]))
                 -> LN -> LM head

with layer norms that carry weight and bias, the sublayers reading x itself (its rounding to
the storage dtype feeds the GEMMs; the stream, the norms and the sums stay fp32).

Hyper-connected designs (``cfg.streams``; ``lapunex``) keep S copies x_1 .. x_S of the stream,
all equal to the embedding output at first. A sublayer with read weights a, write weights b
and stream mix M runs

    u = sum_s a_s x_s;   y = sublayer(norm(u));   x_t <- sum_s M[s, t] x_s + b_t y   (all t at once)

and the final norm reads the sum of the streams (``ops.hybrid.hyper_mix`` fuses a sublayer's
write-back with the next sublayer's read and norm).

* Layers [start, stop) of the loop run ``times`` times with the same weights; a pass starts
  with x = W_in [x ; x0] + step[pass] (x0 = the embedding output). Every run owns its cache or
  state (``engine.kv_cache.HybridCache``).
* The residual stream and every norm are fp32; GEMM operands use the storage dtype of the
  weights (bf16 when serving; fp32 weights give an all-fp32 model). Each residual add is fused
  with the norm that follows it (``ops.hybrid.resadd_groupnorm``).
* Every step kind — whole prompts, prompt portions, decode rows, mixed — runs the same path:
  new tokens are written to the paged caches, then attend through the block tables, so a
  position's logits do not depend on how its sequence was cut into steps.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..engine.batch import DeviceBatch
from ..ops import hybrid as H
from .configs import ModelConfig
from .mixers import (FEED_FORWARDS, MIXERS, StepView, derive_constants,
                     prepare_feed_forward)
from .model import TransformerLM


class HybridLM(TransformerLM):
    # the scheduler builds block tables for every step, not only chunked ones
    needs_block_tables = True

    def __init__(self, cfg: ModelConfig, params: Dict[str, torch.Tensor], layer_start: int = 0,
                 layer_end: Optional[int] = None, device="cpu", expert_range=None):
        if layer_start != 0 or (layer_end is not None and layer_end != cfg.num_layers):
            raise ValueError("hybrid designs run on one stage (the loop entry reads the "
                             "embedding output)")
        for i, spec in enumerate(cfg.layer_specs):
            prepare_feed_forward(spec, params, f"layers.{i}.")
        super().__init__(cfg, params, 0, None, device)
        self.dtype = params["embed"].dtype
        self.runs = cfg.layer_runs()
        for spec, lp in zip(cfg.layer_specs, self.layers):
            derive_constants(spec, lp, self.device)
        self._cu: Dict[int, torch.Tensor] = {}
        self._rows: Dict[int, torch.Tensor] = {}
        # read weights of the plain sum of the streams (made here, not inside a captured step)
        self._sum_streams = (torch.ones(cfg.streams, dtype=torch.float32, device=self.device)
                             if cfg.streams else None)
        # debugging aid: when a list, forward_layers appends the residual after every run
        self.layer_trace: Optional[List[torch.Tensor]] = None

    def to(self, device):
        super().to(device)
        for i, spec in enumerate(self.cfg.layer_specs):
            prepare_feed_forward(spec, self.params, f"layers.{i}.")
        self.layers = [self._layer_params(i) for i in range(len(self.cfg.layer_specs))]
        for spec, lp in zip(self.cfg.layer_specs, self.layers):
            derive_constants(spec, lp, self.device)
        self._cu.clear()
        self._rows.clear()
        if self.cfg.streams:
            self._sum_streams = torch.ones(self.cfg.streams, dtype=torch.float32,
                                           device=self.device)
        return self

    # ------------------------------------------------------------------ step metadata
    def _step_view(self, b: DeviceBatch, block_size: int) -> StepView:
        if b.is_prefill:
            cu, mx = b.cu_seqlens, b.max_seqlen
        else:                                   # decode: one row per sequence
            n = b.num_tokens
            cu = self._cu.get(n)
            if cu is None:
                cu = self._cu[n] = torch.arange(n + 1, dtype=torch.int32, device=self.device)
            mx = 1
        if b.block_tables is None:
            raise ValueError("hybrid models attend through the paged cache: the step carries "
                             "no block tables")
        return StepView(cu, mx, b.positions, b.slot_mapping, b.block_tables, block_size,
                        b.state_slots, b.max_context if b.max_context > 0 else 1 << 30)

    def _all_rows(self, n: int) -> torch.Tensor:
        r = self._rows.get(n)
        if r is None:
            r = self._rows[n] = torch.arange(n, dtype=torch.int64, device=self.device)
        return r

    # ------------------------------------------------------------------ forward
    def embed(self, b: DeviceBatch, kv_caches=None) -> torch.Tensor:
        cfg, p = self.cfg, self.params
        if cfg.post_norm:
            # (fp32 stream, its storage-dtype rounding): the first layer's sublayers read both
            prev, bg = None, cfg.bigram or (0, 0, 0)
            if cfg.bigram:
                step = self._step_view(b, kv_caches.block_size)
                prev = H.prev_tokens(b.input_ids, kv_caches.prev_token, step.state_slots,
                                     step.cu_seqlens, step.max_seqlen, step.positions)
            return H.embedding_bigram(b.input_ids, prev, p["embed"], p.get("bigram"), *bg)
        return H.embedding_f32(b.input_ids, p["embed"], scale=cfg.embed_scale,
                               pos_table=p.get("pos_embed") if cfg.learned_pos else None,
                               positions=b.positions)[0]

    def _postnorm_layers(self, xs, b: DeviceBatch, kv_caches) -> torch.Tensor:
        """Post-norm layers: every sublayer reads the stream itself and the norm follows the
        sum. ``xs`` = (fp32 stream, its storage-dtype copy)."""
        cfg, p = self.cfg, self.params
        eps, a = cfg.norm_eps, cfg.postln_alpha
        step = self._step_view(b, kv_caches.block_size)
        x, xb = xs
        for li, (spec, lp) in enumerate(zip(cfg.layer_specs, self.layers)):
            y = MIXERS[spec.kind](spec, lp, xb, step, kv_caches.entries[li], eps)
            xb = H.postnorm(x, y, lp["norm1"], lp["norm1_b"], eps, keep=a)
            if spec.ff:
                y = FEED_FORWARDS[spec.ff_kind](spec, lp, xb)
                xb = H.postnorm(x, y, lp["norm2"], lp["norm2_b"], eps, keep=a)
            elif "norm2" in lp:
                xb = H.postnorm(x, None, lp["norm2"], lp["norm2_b"], eps, keep=a)
            if cfg.side_dim:            # per-layer token input
                g = H.side_gate(H.linear_any(xb, lp["side_gate"]), b.input_ids, p["side_embed"],
                                li * cfg.side_dim)
                xb = H.add_rmsnormed(x, H.linear_any(g, lp["side_proj"]), lp["side_norm"], eps)
            if self.layer_trace is not None:
                self.layer_trace.append(x.clone())
        return x

    def _hyper_layers(self, x: torch.Tensor, b: DeviceBatch, kv_caches) -> torch.Tensor:
        """Pre-norm layers over hyper-connected streams; returns the sum of the streams."""
        cfg = self.cfg
        eps, off, S = cfg.norm_eps, cfg.norm_offset, cfg.streams
        step = self._step_view(b, kv_caches.block_size)
        T, D = x.shape
        xs = x.unsqueeze(1).expand(T, S, D).contiguous()
        y = prev = None                     # a sublayer's output awaiting its write-back
        for ri, (li, _, _) in enumerate(self.runs):
            spec, lp = cfg.layer_specs[li], self.layers[li]
            h = H.hyper_mix(xs, y, prev, lp["hc1"], lp["norm1"], eps, off)
            y, prev = MIXERS[spec.kind](spec, lp, h, step, kv_caches.entries[ri], eps), lp["hc1"]
            if spec.ff:
                h = H.hyper_mix(xs, y, prev, lp["hc2"], lp["norm2"], eps, off)
                y, prev = FEED_FORWARDS[spec.ff_kind](spec, lp, h), lp["hc2"]
            if self.layer_trace is not None:
                self.layer_trace.append(H.hyper_mix(xs, y, prev, self._sum_streams, None))
                y = prev = None
        return H.hyper_mix(xs, y, prev, self._sum_streams, None)

    def forward_layers(self, x: torch.Tensor, b: DeviceBatch, kv_caches) -> torch.Tensor:
        cfg, p = self.cfg, self.params
        if cfg.post_norm:
            return self._postnorm_layers(x, b, kv_caches)
        if cfg.streams:
            return self._hyper_layers(x, b, kv_caches)
        eps, groups, m, off = cfg.norm_eps, cfg.norm_groups, cfg.residual_mult, cfg.norm_offset
        step = self._step_view(b, kv_caches.block_size)
        entries = kv_caches.entries
        x0 = x.clone() if cfg.loop and cfg.loop_entry else None
        pending = None                      # a sub-block's fp32 output awaiting its add
        for ri, (li, t, first) in enumerate(self.runs):
            spec, lp = cfg.layer_specs[li], self.layers[li]
            if first:
                if pending is not None:
                    H.resadd_groupnorm(x, pending, None, groups, eps, mult=m)
                    pending = None
                y = H.linear_any(H.concat_cast(x, x0, self.dtype), p["loop_in"])
                h = H.resadd_groupnorm(x, y, lp["norm1"], groups, eps, mult=1.0, keep=0.0,
                                       bias=p["loop_step"][t], out_f32=spec.shift)
            else:
                h = H.resadd_groupnorm(x, pending, lp["norm1"], groups, eps, mult=m,
                                       out_f32=spec.shift, w_offset=off)
            if spec.shift:                  # the mixer reads the rows mixed with their predecessors
                h = H.token_shift(h, lp["shift"], kv_caches.shift_states[ri], step.state_slots,
                                  step.cu_seqlens, step.max_seqlen, step.positions)
            y = MIXERS[spec.kind](spec, lp, h, step, entries[ri], eps)
            if spec.ff:
                h = H.resadd_groupnorm(x, y, lp["norm2"], groups, eps, mult=m, w_offset=off)
                y = FEED_FORWARDS[spec.ff_kind](spec, lp, h)
            pending = y
            if self.layer_trace is not None:
                H.resadd_groupnorm(x, pending, None, groups, eps, mult=m)
                pending = None
                self.layer_trace.append(x.clone())
        if pending is not None:
            H.resadd_groupnorm(x, pending, None, groups, eps, mult=m)
        return x

    def final_hidden(self, hidden: torch.Tensor, b: DeviceBatch) -> torch.Tensor:
        cfg, p = self.cfg, self.params
        if b.logit_rows is not None:
            rows = b.logit_rows
        elif b.is_prefill:
            rows = b.last_token_idx
        else:
            rows = None
        if cfg.post_norm:
            if rows is None:
                rows = self._all_rows(hidden.shape[0])
            return H.postnorm(hidden, None, p["final_norm"], p["final_norm_b"], cfg.norm_eps,
                              rows_idx=rows)
        if rows is None:
            return H.resadd_groupnorm(hidden, None, p["final_norm"], cfg.norm_groups,
                                      cfg.norm_eps, gain=cfg.logit_scale,
                                      w_offset=cfg.norm_offset)
        # the logit scale rides on the final norm's output: the head is linear
        return H.groupnorm_rows(hidden, rows, p["final_norm"], cfg.norm_groups, cfg.norm_eps,
                                gain=cfg.logit_scale, w_offset=cfg.norm_offset)

    def head_logits(self, h: torch.Tensor) -> torch.Tensor:
        return H.linear_any(h, self.params["lm_head"], out_f32=True)

    def forward(self, b: DeviceBatch, kv_caches, hidden: Optional[torch.Tensor] = None,
                return_logits: bool = False):
        """Sampled int32 tokens [S] (and the logits when asked). With ``b.logit_rows`` the
        logits of exactly those rows are returned and nothing is sampled."""
        x = self.forward_layers(self.embed(b, kv_caches), b, kv_caches)
        lg = self.logits(x, b)
        if b.logit_rows is not None:
            return lg
        tok = self.sample(lg, b)
        return (tok, lg) if return_logits else tok

    # ------------------------------------------------------------------ planning
    def gemm_shapes(self, M: int):
        """(shapes, weights) of the projection GEMMs a step of M rows runs on the tuned tile
        family (fp32-output plans; other shapes run the shape-agnostic kernel)."""
        shapes, weights = [], {}
        if self.dtype != torch.bfloat16:
            return shapes, weights
        mats = [w for lp in self.layers for w in lp.values()
                if isinstance(w, torch.Tensor) and w.dim() == 2 and w.dtype == self.dtype]
        mats += [self.params[k] for k in ("loop_in", "lm_head") if k in self.params]
        fused = {}                     # first GEMMs of feed-forwards in the tuned layout
        for spec, lp in zip(self.cfg.layer_specs, self.layers):
            if "ff_tuned" in lp:
                if spec.ff_kind == "gelu":
                    fused[id(lp["w_up"])] = "bias_gelu"
                elif spec.ff_kind == "gated_silu":
                    fused[id(lp["w_gu"])] = "silu_mul"
                elif spec.shared_ff and spec.expert_act == "gelu_erf":
                    fused[id(lp["ws_up"])] = "gelu_erf"
                elif spec.shared_ff:
                    fused[id(lp["ws_gu"])] = "silu_mul"
        for w in mats:
            n, k = w.shape
            epi = fused.get(id(w), "f32")
            if k % 64 == 0 and (n, k, epi) not in weights and n >= 16:
                shapes.append((M, n, k, epi))
                weights[(n, k, epi)] = w
        # the autotune keys weights by (n, k)
        return shapes, {(n, k): w for (n, k, _), w in weights.items()}

    def grouped_gemm_shapes(self, M: int):
        """(rows, expert weights, epilogue) of the grouped expert GEMMs a step of M rows runs
        on the tuned tile family (uniform routing: M x top rows over the experts)."""
        out, seen = [], set()
        for spec, lp in zip(self.cfg.layer_specs, self.layers):
            if spec.ff_kind == "moe" and "ff_tuned" in lp:
                w1, epi = ((lp["w_up"], "gelu_erf") if spec.expert_act == "gelu_erf"
                           else (lp["w_gu"], "none") if spec.expert_act == "clamp_swish"
                           else (lp["w_gu"], "silu_mul"))
                key = (tuple(w1.shape), spec.top, epi)
                if key not in seen:
                    seen.add(key)
                    rows = M * spec.top
                    out += [(rows, w1, epi), (rows, lp["w_down"], "none")]
        return out
