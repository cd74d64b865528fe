"""Weight naming, random init, HF-layout conversion and per-stage selection.

Our in-memory layout (all [out, in] row-major like torch Linear, bf16):

llama / mixtral (per layer ``layers.{i}.``):
    attn_norm [D], wqkv [(Hq+2Hkv)*hd, D], wo [D, Hq*hd], mlp_norm [D],
    dense: w_gu [2F, D] (16-row gate/up interleave, see ops/reference.py), w_down [D, F]
    moe:   router [E, D], w_gu [E, 2F, D], w_down [E, D, F]
gpt2 (per layer): ln1_w, ln1_b, wqkv [3D, D], bqkv [3D], wo [D, D], bo [D], ln2_w, ln2_b,
    w_fc [F, D], b_fc [F], w_proj [D, F], b_proj [D]
globals: embed [V, D], (gpt2) pos_embed [P, D], final_norm [D], (gpt2) final_norm_b [D],
    lm_head [V, D] (absent when tied to embed)

Random init mirrors HF ``_init_weights`` (normal(0, 0.02), norms = 1, biases = 0) and is
generated directly on the target device, per stage, so a 70B stage never materialises the
full model anywhere.
"""
from __future__ import annotations

from typing import Dict, Iterable, Optional

import torch

from .configs import ModelConfig
from ..ops.reference import interleave_gate_up

INIT_STD = 0.02


def hybrid_layer_shapes(cfg: ModelConfig, i: int) -> Dict[str, tuple]:
    """In-memory tensors of hybrid layer ``i`` (``layers.{i}.``), projections that read the
    same input fused row-wise:
      attention:        w_in [(H + G + H)*d, D] = q | k | gate, q_norm [d], k_norm [d],
                        talk [H, H] fp32, wo [D, H*d]
      hgrn2:            w_in [(2*H*d + H*dv), D] = q | f | v, f_b [H*d], lower [H*d],
                        o_norm [dv], wo [D, H*dv]
      latent_attention: w_in [H*(d+dr) + r + dr, D] = q | compressed kv, c_norm [r],
                        w_ukT [H, r, d] (per head, transposed: the absorb projection),
                        w_uv [H, dv, r], wo [D, H*dv]
      talk_attention:   shift [D], w_in [(H*d + G*d + G*dv), D] = q | k | v with b_in (a layer
                        that attends another layer's cache holds the q part only),
                        talk [H, H] fp32, wo [D, H*dv]
      feed-forward:     norm2 [D], then by ``ff_kind``
        gated_gelu:     w_gu [2F, D] = gate | up, w_down [D, F]
        gelu:           w_up [F, D], w_down [D, F]
        moe:            router [E + I (+ 1), D] (the last row is the shared expert's gate),
                        correction [E + I] fp32, w_gu [E, 2F, D] = gate | up per expert,
                        w_down [E, D, F], shared expert ws_gu [2Fs, D], ws_down [D, Fs]
        gated_silu:     w_gu [2F, D] = gate | up, w_down [D, F]
        moe, router ``logit_topk`` with ``gelu_erf`` experts: router [E, D], router_b [E] fp32,
                        w_up [E, F, D], w_down [E, D, F], shared ws_up [Fs, D], ws_down [D, Fs]
      gla:              w_in [2*H*d + 2*H*dv + ra, D] = q | k | v | output gate | decay-in,
                        w_a2 [H*d, ra], a_b [H*d], o_norm [dv], wo [D, H*dv]
      latent_attention with ``q_rank`` / ``head_gate``: w_in [rq + (r + dr) + H, D] = query
                        latent | compressed kv (absent with ``kv_from``) | head gates,
                        q_norm [rq], w_uq [H*(d+dr), rq], then as above
      lightning:        w_in [2*H*d + 2*H*dv, D] = q | k | v | output gate, o_norm [H*dv],
                        wo [D, H*dv]
      parallel:         w_in = left q [Hl*d] | left k [G*d] | left v [G*dvl] | left head gates
                        [Hl] | right q [Hr*dr] | right k [Hr*dr] | right v [Hr*dvr] | right
                        output gate [Hr*dvr] | right input gates [Hr] | right forget gates [Hr],
                        q_norm [Hl*d], k_norm [G*d], sink [Hl] fp32, o_norm [Hr*dvr],
                        if_b [2*Hr] fp32 (input | forget gate biases),
                        wo [D, Hl*dvl + Hr*dvr] = left | right output projections
        moe, router ``group_score`` with ``clamp_swish`` experts: router [E, D],
                        w_gu [E, 2F, D], w_down [E, D, F]
    Post-norm designs add the norms' biases norm1_b / norm2_b [D]; with a per-layer token input
    of width s: side_gate [s, D], side_proj [D, s], side_norm [D]. With hyper-connections over
    S streams every sublayer has hc1 / hc2 fp32 [S + S + S*S] = read weights | write weights |
    stream mix [from, to]."""
    D = cfg.hidden_size
    s = cfg.layer_specs[i]
    p = f"layers.{i}."
    H, d, dv = s.heads, s.dim, s.vdim
    out = {p + "norm1": (D,)}
    if s.kind == "attention":
        out.update({p + "w_in": ((2 * H + s.kv_heads) * d, D), p + "q_norm": (d,),
                    p + "k_norm": (d,), p + "talk": (H, H), p + "wo": (D, H * d)})
    elif s.kind == "hgrn2":
        out.update({p + "w_in": (2 * H * d + H * dv, D), p + "f_b": (H * d,),
                    p + "lower": (H * d,), p + "o_norm": (dv,), p + "wo": (D, H * dv)})
    elif s.kind == "latent_attention":
        nkv = 0 if s.kv_from >= 0 else s.kv_rank + s.rot_dim
        nq = s.q_rank if s.q_rank else H * (d + s.rot_dim)
        out.update({p + "w_in": (nq + nkv + (H if s.head_gate else 0), D),
                    p + "w_ukT": (H, s.kv_rank, d),
                    p + "w_uv": (H, dv, s.kv_rank), p + "wo": (D, H * dv)})
        if nkv:
            out[p + "c_norm"] = (s.kv_rank,)
        if s.q_rank:
            out.update({p + "q_norm": (s.q_rank,), p + "w_uq": (H * (d + s.rot_dim), s.q_rank)})
    elif s.kind == "gla":
        ra = s.decay_rank
        out.update({p + "w_in": (2 * H * d + 2 * H * dv + ra, D), p + "w_a2": (H * d, ra),
                    p + "a_b": (H * d,), p + "o_norm": (dv,), p + "wo": (D, H * dv)})
    elif s.kind == "talk_attention":
        n_in = H * d + (0 if s.kv_from >= 0 else s.kv_heads * (d + dv))
        out.update({p + "shift": (D,), p + "w_in": (n_in, D), p + "b_in": (n_in,),
                    p + "talk": (H, H), p + "wo": (D, H * dv)})
    elif s.kind == "lightning":
        out.update({p + "w_in": (2 * H * (d + dv), D), p + "o_norm": (H * dv,),
                    p + "wo": (D, H * dv)})
    elif s.kind == "parallel":
        l, r = s.left, s.right
        n_in = (l.heads * l.dim + l.kv_heads * (l.dim + l.vdim) + l.heads
                + r.heads * (2 * r.dim + 2 * r.vdim + 2))
        out.update({p + "w_in": (n_in, D), p + "q_norm": (l.heads * l.dim,),
                    p + "k_norm": (l.kv_heads * l.dim,), p + "sink": (l.heads,),
                    p + "o_norm": (r.heads * r.vdim,), p + "if_b": (2 * r.heads,),
                    p + "wo": (D, l.heads * l.vdim + r.heads * r.vdim)})
    else:
        raise ValueError(f"unknown mixer kind '{s.kind}'")
    if cfg.streams:
        n = cfg.streams * (cfg.streams + 2)
        out[p + "hc1"] = (n,)
        if s.ff:
            out[p + "hc2"] = (n,)
    if cfg.post_norm:
        out[p + "norm1_b"] = (D,)
        if s.ff:
            out[p + "norm2_b"] = (D,)
    if cfg.side_dim:
        out.update({p + "side_gate": (cfg.side_dim, D), p + "side_proj": (D, cfg.side_dim),
                    p + "side_norm": (D,)})
    if s.ff and s.ff_kind == "moe" and s.router == "logit_topk":
        out.update({p + "norm2": (D,), p + "router": (s.experts, D), p + "router_b": (s.experts,),
                    p + "w_up": (s.experts, s.ff, D), p + "w_down": (s.experts, D, s.ff)})
        if s.shared_ff:
            out.update({p + "ws_up": (s.shared_ff, D), p + "ws_down": (D, s.shared_ff)})
    elif s.ff and s.ff_kind in ("gated_gelu", "gated_silu"):
        out.update({p + "norm2": (D,), p + "w_gu": (2 * s.ff, D), p + "w_down": (D, s.ff)})
    elif s.ff and s.ff_kind == "gelu":
        out.update({p + "norm2": (D,), p + "w_up": (s.ff, D), p + "w_down": (D, s.ff)})
    elif s.ff and s.ff_kind == "moe" and s.router == "group_score":
        out.update({p + "norm2": (D,), p + "router": (s.experts, D),
                    p + "w_gu": (s.experts, 2 * s.ff, D), p + "w_down": (s.experts, D, s.ff)})
    elif s.ff and s.ff_kind == "moe":
        n = s.experts + s.identity
        out.update({p + "norm2": (D,), p + "router": (n + (1 if s.shared_ff else 0), D),
                    p + "correction": (n,), p + "w_gu": (s.experts, 2 * s.ff, D),
                    p + "w_down": (s.experts, D, s.ff)})
        if s.shared_ff:
            out.update({p + "ws_gu": (2 * s.shared_ff, D), p + "ws_down": (D, s.shared_ff)})
    elif s.ff:
        raise ValueError(f"unknown feed-forward kind '{s.ff_kind}'")
    return out


def layer_param_shapes(cfg: ModelConfig, i: int) -> Dict[str, tuple]:
    if cfg.is_hybrid:
        return hybrid_layer_shapes(cfg, i)
    d, f, hd = cfg.hidden_size, cfg.intermediate_size, cfg.head_dim
    p = f"layers.{i}."
    if cfg.arch == "gpt2":
        return {p + "ln1_w": (d,), p + "ln1_b": (d,), p + "wqkv": (3 * d, d), p + "bqkv": (3 * d,),
                p + "wo": (d, d), p + "bo": (d,), p + "ln2_w": (d,), p + "ln2_b": (d,),
                p + "w_fc": (f, d), p + "b_fc": (f,), p + "w_proj": (d, f), p + "b_proj": (d,)}
    s = {p + "attn_norm": (d,), p + "wqkv": (cfg.qkv_size, d), p + "wo": (d, cfg.q_size),
         p + "mlp_norm": (d,)}
    if cfg.is_moe:
        e = cfg.num_experts
        s.update({p + "router": (e, d), p + "w_gu": (e, 2 * f, d), p + "w_down": (e, d, f)})
    else:
        s.update({p + "w_gu": (2 * f, d), p + "w_down": (d, f)})
    return s


def global_param_shapes(cfg: ModelConfig, first: bool, last: bool) -> Dict[str, tuple]:
    d, v = cfg.hidden_size, cfg.vocab_size
    s: Dict[str, tuple] = {}
    if cfg.is_hybrid:
        # the loop entry re-reads the embedding output, so a stage that runs loop layers
        # holds the embedding too (hybrid designs run on one stage)
        s.update({"embed": (v, d), "final_norm": (d,), "lm_head": (v, d)})
        if cfg.loop and cfg.loop_entry:
            s.update({"loop_in": (d, 2 * d), "loop_step": (cfg.loop[2], d)})
        if cfg.learned_pos:
            s["pos_embed"] = (cfg.max_position, d)
        if cfg.post_norm:
            s["final_norm_b"] = (d,)
        if cfg.bigram:
            s["bigram"] = (cfg.bigram[0] + 1, d)
        if cfg.side_dim:
            s["side_embed"] = (v, len(cfg.layer_specs) * cfg.side_dim)
        return s
    if first or (last and cfg.tie_embeddings):
        s["embed"] = (v, d)
    if first and cfg.arch == "gpt2":
        s["pos_embed"] = (cfg.max_position, d)
    if last:
        s["final_norm"] = (d,)
        if cfg.arch == "gpt2":
            s["final_norm_b"] = (d,)
        if not cfg.tie_embeddings:
            s["lm_head"] = (v, d)
    return s


def stage_param_shapes(cfg: ModelConfig, layer_start: int, layer_end: int, first: bool,
                       last: bool, expert_range: Optional[tuple] = None) -> Dict[str, tuple]:
    s = global_param_shapes(cfg, first, last)
    for i in range(layer_start, layer_end):
        ls = layer_param_shapes(cfg, i)
        if expert_range is not None and cfg.is_moe:
            e0, e1 = expert_range
            for k in list(ls):
                if k.endswith(".w_gu") or k.endswith(".w_down"):
                    ls[k] = (e1 - e0,) + tuple(ls[k][1:])
        s.update(ls)
    return s


def _is_norm_weight(name: str) -> bool:
    return name.endswith(("attn_norm", "mlp_norm", "final_norm", "ln1_w", "ln2_w", "norm1",
                          "norm2", "q_norm", "k_norm", "c_norm", "o_norm", "side_norm"))


def _is_bias(name: str) -> bool:
    return name.endswith(("ln1_b", "ln2_b", "bqkv", "bo", "b_fc", "b_proj", "final_norm_b",
                          "norm1_b", "norm2_b"))


def random_init(shapes: Dict[str, tuple], device, dtype=torch.bfloat16, seed: int = 0,
                std: float = INIT_STD, norm_value: float = 1.0) -> Dict[str, torch.Tensor]:
    """Deterministic per-tensor init: each tensor's values depend only on (seed, name), so a
    pipeline stage generates exactly the slice the full model would hold."""
    out = {}
    dev = torch.device(device)
    hybrid = any(n.endswith(".norm1") for n in shapes)
    for name in sorted(shapes):
        shape = shapes[name]
        if hybrid and not _is_norm_weight(name) and not _is_bias(name):
            out[name] = _hybrid_init(name, shape, dev, dtype, seed)
        elif _is_norm_weight(name):
            # a design that stores its layer norms' weights as offsets starts them at zero
            v = norm_value if name.endswith(("norm1", "norm2", "final_norm")) else 1.0
            out[name] = torch.full(shape, v, dtype=dtype, device=dev)
        elif _is_bias(name):
            out[name] = torch.zeros(shape, dtype=dtype, device=dev)
        else:
            g = torch.Generator(device=dev)
            g.manual_seed((seed * 1_000_003 + _name_hash(name)) & 0x7FFF_FFFF_FFFF)
            t = torch.empty(shape, dtype=dtype, device=dev)
            t.normal_(0.0, std, generator=g)
            out[name] = t
    return out


def _hybrid_init(name: str, shape: tuple, dev, dtype, seed: int) -> torch.Tensor:
    """Random values for the hybrid family's tensors that a plain normal(0, 0.02) would make
    degenerate: head-mixing matrices near the identity (fp32), forget-gate lower bounds in
    [0, 0.9), gate biases and loop step vectors of unit-ish size, and input projections scaled
    like 1/sqrt(fan_in) so that normed queries, gates and recurrences see O(1) inputs."""
    g = torch.Generator(device="cpu")
    g.manual_seed((seed * 1_000_003 + _name_hash(name)) & 0x7FFF_FFFF_FFFF)
    if name.endswith(".talk"):
        t = torch.eye(shape[0]) + 0.2 * torch.randn(shape, generator=g)
        return t.to(dev, torch.float32)
    if name.endswith(".correction"):
        return (0.05 * torch.randn(shape, generator=g)).to(dev, torch.float32)
    if name.endswith(".router_b"):
        return (0.1 * torch.randn(shape, generator=g)).to(dev, torch.float32)
    if name.endswith((".hc1", ".hc2")):
        # read weights near 1/S, write weights near 1, a stream mix near the identity
        S = int(round((1 + shape[0]) ** 0.5)) - 1
        t = torch.cat([torch.full((S,), 1.0 / S) + 0.1 * torch.randn(S, generator=g),
                       1.0 + 0.2 * torch.randn(S, generator=g),
                       (torch.eye(S) + 0.15 * torch.randn(S, S, generator=g)).reshape(-1)])
        return t.to(dev, torch.float32)
    if name.endswith(".sink"):
        return torch.randn(shape, generator=g).to(dev, torch.float32)
    if name.endswith(".if_b"):
        # input gates around -1, forget gates around +3 (slow forgetting)
        H = shape[0] // 2
        t = torch.cat([-1.0 + 0.5 * torch.randn(H, generator=g),
                       3.0 + 1.0 * torch.randn(H, generator=g)])
        return t.to(dev, torch.float32)
    if name.endswith(".a_b"):
        # decays sigmoid(z)^(1/tau) spread between fast and slow channels
        return (1.0 + 2.0 * torch.randn(shape, generator=g)).to(dev, dtype)
    if name.endswith(".shift"):
        return torch.rand(shape, generator=g).to(dev, dtype)
    if name.endswith(".b_in"):
        # small: a large value bias is a constant added to every token, which would make a
        # random-init router send every token to the same experts
        return (0.02 * torch.randn(shape, generator=g)).to(dev, dtype)
    if name.endswith(".lower"):
        return (0.9 * torch.rand(shape, generator=g)).to(dev, dtype)
    if name.endswith((".f_b", "loop_step")):
        return (0.5 * torch.randn(shape, generator=g)).to(dev, dtype)
    return (torch.randn(shape, generator=g) / shape[-1] ** 0.5).to(dev, dtype)


def calm_random_mixers(cfg: ModelConfig, params: Dict[str, torch.Tensor]) -> None:
    """Random-init only. A fixed-decay linear attention reads SiLU-activated (mostly positive)
    queries, keys and values, so at random init its output has a large component shared by
    all tokens, which makes a random router send every token to the same experts (a trained
    model's routing is spread). Its output projection therefore starts small."""
    for i, s in enumerate(cfg.layer_specs):
        k = f"layers.{i}.wo"
        if s.kind == "lightning" and k in params:
            params[k].mul_(0.1)


def slice_experts(name: str, t: torch.Tensor, expert_range: Optional[tuple]) -> torch.Tensor:
    if expert_range is None or not (name.endswith(".w_gu") or name.endswith(".w_down")):
        return t
    if t.dim() != 3:
        return t
    if expert_range[0] == 0 and expert_range[1] == t.shape[0]:
        return t
    # a copy: a leading-dim slice is already contiguous, so .contiguous() would return a
    # view that keeps every expert's storage alive (each EP rank held all 8 experts)
    return t[expert_range[0]:expert_range[1]].clone()


def _name_hash(name: str) -> int:
    h = 1469598103934665603
    for ch in name.encode():
        h ^= ch
        h = (h * 1099511628211) & 0xFFFF_FFFF_FFFF_FFFF
    return h


def nbytes(params: Dict[str, torch.Tensor]) -> int:
    return sum(t.numel() * t.element_size() for t in params.values())


# ----------------------------------------------------------------------------- HF conversion
def from_hf_state_dict(cfg: ModelConfig, sd: Dict[str, torch.Tensor],
                       layers: Optional[Iterable[int]] = None, first: bool = True,
                       last: bool = True, dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Convert a HF LlamaForCausalLM / MixtralForCausalLM / GPT2LMHeadModel state dict."""
    layers = range(cfg.num_layers) if layers is None else layers
    out: Dict[str, torch.Tensor] = {}
    cv = lambda t: t.detach().to(dtype).contiguous()  # noqa: E731
    if cfg.arch == "gpt2":
        pre = "transformer."
        if first or (last and cfg.tie_embeddings):
            out["embed"] = cv(sd[pre + "wte.weight"])
        if first:
            out["pos_embed"] = cv(sd[pre + "wpe.weight"])
        if last:
            out["final_norm"] = cv(sd[pre + "ln_f.weight"])
            out["final_norm_b"] = cv(sd[pre + "ln_f.bias"])
        for i in layers:
            h = f"{pre}h.{i}."
            p = f"layers.{i}."
            # HF GPT-2 Conv1D stores [in, out]; ours is [out, in]
            out[p + "ln1_w"] = cv(sd[h + "ln_1.weight"]); out[p + "ln1_b"] = cv(sd[h + "ln_1.bias"])
            out[p + "wqkv"] = cv(sd[h + "attn.c_attn.weight"].t()); out[p + "bqkv"] = cv(sd[h + "attn.c_attn.bias"])
            out[p + "wo"] = cv(sd[h + "attn.c_proj.weight"].t()); out[p + "bo"] = cv(sd[h + "attn.c_proj.bias"])
            out[p + "ln2_w"] = cv(sd[h + "ln_2.weight"]); out[p + "ln2_b"] = cv(sd[h + "ln_2.bias"])
            out[p + "w_fc"] = cv(sd[h + "mlp.c_fc.weight"].t()); out[p + "b_fc"] = cv(sd[h + "mlp.c_fc.bias"])
            out[p + "w_proj"] = cv(sd[h + "mlp.c_proj.weight"].t()); out[p + "b_proj"] = cv(sd[h + "mlp.c_proj.bias"])
        return out
    if first:
        out["embed"] = cv(sd["model.embed_tokens.weight"])
    if last:
        out["final_norm"] = cv(sd["model.norm.weight"])
        if cfg.tie_embeddings:
            out["embed"] = cv(sd["model.embed_tokens.weight"])
        else:
            out["lm_head"] = cv(sd["lm_head.weight"])
    for i in layers:
        h = f"model.layers.{i}."
        p = f"layers.{i}."
        out[p + "attn_norm"] = cv(sd[h + "input_layernorm.weight"])
        out[p + "mlp_norm"] = cv(sd[h + "post_attention_layernorm.weight"])
        out[p + "wqkv"] = cv(torch.cat([sd[h + "self_attn.q_proj.weight"],
                                        sd[h + "self_attn.k_proj.weight"],
                                        sd[h + "self_attn.v_proj.weight"]], 0))
        out[p + "wo"] = cv(sd[h + "self_attn.o_proj.weight"])
        if cfg.is_moe:
            moe = h + "block_sparse_moe."
            if moe + "gate.weight" not in sd:
                moe = h + "mlp."
            out[p + "router"] = cv(sd[moe + "gate.weight"])
            gus, downs = [], []
            if moe + "experts.gate_up_proj" in sd:
                # fused expert tensors (transformers >= 5 MixtralExperts):
                # gate_up_proj [E, 2F, D] (gate rows then up rows), down_proj [E, D, F]
                gu = sd[moe + "experts.gate_up_proj"]
                dn = sd[moe + "experts.down_proj"]
                f = cfg.intermediate_size
                gus = [interleave_gate_up(gu[e, :f], gu[e, f:]) for e in range(cfg.num_experts)]
                downs = [dn[e] for e in range(cfg.num_experts)]
            else:
                for e in range(cfg.num_experts):
                    ex = f"{moe}experts.{e}."
                    if ex + "w1.weight" in sd:   # original Mixtral naming (w1 gate, w3 up, w2 down)
                        g, u, dn = sd[ex + "w1.weight"], sd[ex + "w3.weight"], sd[ex + "w2.weight"]
                    else:
                        g, u, dn = (sd[ex + "gate_proj.weight"], sd[ex + "up_proj.weight"],
                                    sd[ex + "down_proj.weight"])
                    gus.append(interleave_gate_up(g, u))
                    downs.append(dn)
            out[p + "w_gu"] = cv(torch.stack(gus))
            out[p + "w_down"] = cv(torch.stack(downs))
        else:
            out[p + "w_gu"] = cv(interleave_gate_up(sd[h + "mlp.gate_proj.weight"],
                                                    sd[h + "mlp.up_proj.weight"]))
            out[p + "w_down"] = cv(sd[h + "mlp.down_proj.weight"])
    return out


# ----------------------------------------------------------------------------- Buborax files
def from_buborax_state_dict(cfg: ModelConfig, sd, dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Convert a Buborax checkpoint (tensor names ``embed``, ``head``, ``final.norm``,
    ``loop.in``, ``loop.step``, ``l<i>.norm1|norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*``; linear
    weights [out, in]) into the in-memory layout of ``hybrid_layer_shapes``."""
    cv = lambda t: t.detach().to(dtype).contiguous()  # noqa: E731
    out = {"embed": cv(sd["embed"]), "lm_head": cv(sd["head"]), "final_norm": cv(sd["final.norm"])}
    if cfg.loop:
        out["loop_in"] = cv(sd["loop.in"])
        out["loop_step"] = cv(sd["loop.step"])
    for i, s in enumerate(cfg.layer_specs):
        a, p = f"l{i}.", f"layers.{i}."
        m = a + "mix."
        out[p + "norm1"] = cv(sd[a + "norm1"])
        H, d, dv = s.heads, s.dim, s.vdim
        if s.kind == "attention":
            out[p + "w_in"] = cv(torch.cat([sd[m + "q"], sd[m + "k"], sd[m + "g"]], 0))
            out[p + "q_norm"], out[p + "k_norm"] = cv(sd[m + "q.norm"]), cv(sd[m + "k.norm"])
            out[p + "talk"] = sd[m + "talk"].detach().float().contiguous()
        elif s.kind == "hgrn2":
            out[p + "w_in"] = cv(torch.cat([sd[m + "q"], sd[m + "f"], sd[m + "v"]], 0))
            out[p + "f_b"], out[p + "lower"] = cv(sd[m + "f.b"]), cv(sd[m + "lower"])
            out[p + "o_norm"] = cv(sd[m + "norm"])
        else:
            out[p + "w_in"] = cv(torch.cat([sd[m + "q"], sd[m + "dkv"]], 0))
            out[p + "c_norm"] = cv(sd[m + "dkv.norm"])
            uk = sd[m + "uk"].detach().reshape(H, d, s.kv_rank)
            out[p + "w_ukT"] = cv(uk.transpose(1, 2))
            out[p + "w_uv"] = cv(sd[m + "uv"].detach().reshape(H, dv, s.kv_rank))
        out[p + "wo"] = cv(sd[m + "o"])
        if s.ff:
            out[p + "norm2"] = cv(sd[a + "norm2"])
            out[p + "w_gu"] = cv(torch.cat([sd[a + "mlp.gate"], sd[a + "mlp.up"]], 0))
            out[p + "w_down"] = cv(sd[a + "mlp.down"])
    return out


# ----------------------------------------------------------------------------- Pulunex files
def from_pulunex_state_dict(cfg: ModelConfig, sd, dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Convert a Pulunex checkpoint (tensor names ``embed``, ``pos``, ``head``, ``final.norm``,
    ``l<i>.norm1|norm2|shift``, ``l<i>.mix.q|k|v`` with ``.b`` biases, ``l<i>.mix.talk|o``,
    ``l<i>.mlp.up|down`` or ``l<i>.mlp.router|correction|e<j>.gate|up|down|shared.*``; linear
    weights [out, in], norm weights single numbers) into ``hybrid_layer_shapes``' layout: a
    norm's number becomes a constant vector, projections that read the same input are stacked,
    the experts are stacked, and the shared expert's gate row is appended to the router."""
    D = cfg.hidden_size
    cv = lambda t: t.detach().to(dtype).contiguous()  # noqa: E731
    vec = lambda t: t.detach().to(dtype).reshape(1).expand(D).contiguous()  # noqa: E731
    out = {"embed": cv(sd["embed"]), "pos_embed": cv(sd["pos"]), "lm_head": cv(sd["head"]),
           "final_norm": vec(sd["final.norm"])}
    for i, s in enumerate(cfg.layer_specs):
        a, p = f"l{i}.", f"layers.{i}."
        m = a + "mix."
        out[p + "norm1"] = vec(sd[a + "norm1"])
        out[p + "shift"] = cv(sd[a + "shift"])
        parts = ["q"] if s.kv_from >= 0 else ["q", "k", "v"]
        out[p + "w_in"] = cv(torch.cat([sd[m + n] for n in parts], 0))
        out[p + "b_in"] = cv(torch.cat([sd[m + n + ".b"] for n in parts], 0))
        out[p + "talk"] = sd[m + "talk"].detach().float().contiguous()
        out[p + "wo"] = cv(sd[m + "o"])
        if not s.ff:
            continue
        f = a + "mlp."
        out[p + "norm2"] = vec(sd[a + "norm2"])
        if s.ff_kind == "gelu":
            out[p + "w_up"], out[p + "w_down"] = cv(sd[f + "up"]), cv(sd[f + "down"])
            continue
        rows = [sd[f + "router"]] + ([sd[f + "shared.sg"].reshape(1, D)] if s.shared_ff else [])
        out[p + "router"] = cv(torch.cat(rows, 0))
        out[p + "correction"] = sd[f + "correction"].detach().float().contiguous()
        out[p + "w_gu"] = cv(torch.stack([torch.cat([sd[f"{f}e{e}.gate"], sd[f"{f}e{e}.up"]], 0)
                                          for e in range(s.experts)]))
        out[p + "w_down"] = cv(torch.stack([sd[f"{f}e{e}.down"] for e in range(s.experts)]))
        if s.shared_ff:
            out[p + "ws_gu"] = cv(torch.cat([sd[f + "shared.gate"], sd[f + "shared.up"]], 0))
            out[p + "ws_down"] = cv(sd[f + "shared.down"])
    return out


# ----------------------------------------------------------------------------- Risutar files
def from_risutar_state_dict(cfg: ModelConfig, sd, dtype=torch.bfloat16):
    """Convert a Risutar checkpoint (tensor names ``embed``, ``bigram``, ``side.embed``,
    ``head``, ``final.norm`` (+ ``.b``), ``l<i>.norm1|norm2`` (+ ``.b``), ``l<i>.mix.*``,
    ``l<i>.mlp.*``, ``l<i>.side.gate|proj|norm``; linear weights [out, in]) into the layout of
    ``hybrid_layer_shapes``: projections that read the layer input are stacked, the experts are
    stacked, W_uk is stored per head and transposed (the absorb projection). Returns (config,
    tensors): widths the config file does not carry (the decay's inner width, the query
    latent's) are taken from the tensors' shapes."""
    from dataclasses import replace
    cv = lambda t: t.detach().to(dtype).contiguous()  # noqa: E731
    out = {"embed": cv(sd["embed"]), "lm_head": cv(sd["head"]),
           "final_norm": cv(sd["final.norm"]), "final_norm_b": cv(sd["final.norm.b"])}
    if cfg.bigram:
        out["bigram"] = cv(sd["bigram"])
    if cfg.side_dim:
        out["side_embed"] = cv(sd["side.embed"])
    specs = list(cfg.layer_specs)
    for i, s in enumerate(specs):
        a, p = f"l{i}.", f"layers.{i}."
        m = a + "mix."
        out[p + "norm1"], out[p + "norm1_b"] = cv(sd[a + "norm1"]), cv(sd[a + "norm1.b"])
        H, d, dv = s.heads, s.dim, s.vdim
        if s.kind == "gla":
            a1 = sd[m + "a1"]
            specs[i] = s = replace(s, decay_rank=int(a1.shape[0]))
            out[p + "w_in"] = cv(torch.cat([sd[m + "q"], sd[m + "k"], sd[m + "v"], sd[m + "g"],
                                            a1], 0))
            out[p + "w_a2"], out[p + "a_b"] = cv(sd[m + "a2"]), cv(sd[m + "a2.b"])
            out[p + "o_norm"] = cv(sd[m + "norm"])
        else:
            dq = sd[m + "dq"]
            specs[i] = s = replace(s, q_rank=int(dq.shape[0]))
            parts = [dq] + ([] if s.kv_from >= 0 else [sd[m + "dkv"]]) + [sd[m + "g"]]
            out[p + "w_in"] = cv(torch.cat(parts, 0))
            out[p + "q_norm"], out[p + "w_uq"] = cv(sd[m + "dq.norm"]), cv(sd[m + "uq"])
            if s.kv_from < 0:
                out[p + "c_norm"] = cv(sd[m + "dkv.norm"])
            uk = sd[m + "uk"].detach().reshape(H, d, s.kv_rank)
            out[p + "w_ukT"] = cv(uk.transpose(1, 2))
            out[p + "w_uv"] = cv(sd[m + "uv"].detach().reshape(H, dv, s.kv_rank))
        out[p + "wo"] = cv(sd[m + "o"])
        if cfg.side_dim:
            for n in ("gate", "proj", "norm"):
                out[p + "side_" + n] = cv(sd[f"{a}side.{n}"])
        if s.ff or a + "norm2" in sd:     # a second norm without a feed-forward still norms
            out[p + "norm2"], out[p + "norm2_b"] = cv(sd[a + "norm2"]), cv(sd[a + "norm2.b"])
        if not s.ff:
            continue
        f = a + "mlp."
        if s.ff_kind == "gated_silu":
            out[p + "w_gu"] = cv(torch.cat([sd[f + "gate"], sd[f + "up"]], 0))
            out[p + "w_down"] = cv(sd[f + "down"])
            continue
        out[p + "router"] = cv(sd[f + "router"])
        out[p + "router_b"] = sd[f + "router.b"].detach().float().contiguous()
        out[p + "w_up"] = cv(torch.stack([sd[f"{f}e{e}.up"] for e in range(s.experts)]))
        out[p + "w_down"] = cv(torch.stack([sd[f"{f}e{e}.down"] for e in range(s.experts)]))
        if s.shared_ff:
            out[p + "ws_up"], out[p + "ws_down"] = cv(sd[f + "shared.up"]), cv(sd[f + "shared.down"])
    return replace(cfg, layer_specs=tuple(specs)), out


# ----------------------------------------------------------------------------- Lapunex files
def from_lapunex_state_dict(cfg: ModelConfig, sd, dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Convert a Lapunex checkpoint (tensor names ``embed``, ``head``, ``final.norm``,
    ``l<i>.norm1|norm2``, ``l<i>.hc1|hc2.in|out|mix``, ``l<i>.mix.*`` (``left.*`` / ``right.*``
    in a parallel layer), ``l<i>.mlp.gate|up|down`` or ``l<i>.mlp.router|e<j>.gate|up|down``;
    linear weights [out, in]) into the layout of ``hybrid_layer_shapes``: all projections that
    read the mixer's input are stacked into one matrix, the two output projections of a
    parallel layer side by side into another, the experts are stacked, and a sublayer's
    hyper-connection tensors become one fp32 vector. Norm weights stay as stored (offsets from
    one; the kernels add the one in fp32)."""
    cv = lambda t: t.detach().to(dtype).contiguous()  # noqa: E731
    f32 = lambda t: t.detach().float().reshape(-1)  # noqa: E731
    out = {"embed": cv(sd["embed"]), "lm_head": cv(sd["head"]), "final_norm": cv(sd["final.norm"])}
    for i, s in enumerate(cfg.layer_specs):
        a, p = f"l{i}.", f"layers.{i}."
        m = a + "mix."
        out[p + "norm1"] = cv(sd[a + "norm1"])
        for q in ("1", "2") if cfg.streams else ():
            if q == "2" and not s.ff:
                continue
            h = f"{a}hc{q}."
            if tuple(sd[h + "mix"].shape) != (cfg.streams, cfg.streams):
                raise ValueError(f"{h}mix: not [{cfg.streams}, {cfg.streams}]")
            out[p + "hc" + q] = torch.cat([f32(sd[h + "in"]), f32(sd[h + "out"]),
                                           f32(sd[h + "mix"])]).contiguous()
        if s.kind == "lightning":
            out[p + "w_in"] = cv(torch.cat([sd[m + n] for n in "qkvg"], 0))
            out[p + "o_norm"] = cv(sd[m + "norm"])
            out[p + "wo"] = cv(sd[m + "o"])
        else:
            lt, rt = m + "left.", m + "right."
            out[p + "w_in"] = cv(torch.cat([sd[lt + n] for n in "qkvg"]
                                           + [sd[rt + n] for n in "qkvgif"], 0))
            out[p + "q_norm"], out[p + "k_norm"] = cv(sd[lt + "q.norm"]), cv(sd[lt + "k.norm"])
            out[p + "sink"] = f32(sd[lt + "sink"]).contiguous()
            out[p + "o_norm"] = cv(sd[rt + "norm"])
            out[p + "if_b"] = torch.cat([f32(sd[rt + "i.b"]), f32(sd[rt + "f.b"])]).contiguous()
            out[p + "wo"] = cv(torch.cat([sd[lt + "o"], sd[rt + "o"]], 1))
        if not s.ff:
            continue
        f = a + "mlp."
        out[p + "norm2"] = cv(sd[a + "norm2"])
        if s.ff_kind == "gated_silu":
            out[p + "w_gu"] = cv(torch.cat([sd[f + "gate"], sd[f + "up"]], 0))
            out[p + "w_down"] = cv(sd[f + "down"])
            continue
        out[p + "router"] = cv(sd[f + "router"])
        out[p + "w_gu"] = cv(torch.stack([torch.cat([sd[f"{f}e{e}.gate"], sd[f"{f}e{e}.up"]], 0)
                                          for e in range(s.experts)]))
        out[p + "w_down"] = cv(torch.stack([sd[f"{f}e{e}.down"] for e in range(s.experts)]))
    want = stage_param_shapes(cfg, 0, len(cfg.layer_specs), True, True)
    for k, shp in want.items():
        if k not in out or tuple(out[k].shape) != tuple(shp):
            got = tuple(out[k].shape) if k in out else None
            raise ValueError(f"{k}: the checkpoint gives {got}, the configuration {tuple(shp)}")
    return out
