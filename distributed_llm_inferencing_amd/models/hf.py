"""HF checkpoint import: ``save_pretrained`` directories (and hub-cache snapshots) of
LlamaForCausalLM / MixtralForCausalLM / GPT2LMHeadModel.

The reference loads checkpoints with ``AutoModelForCausalLM.from_pretrained(model_name,
cache_dir=MODEL_CACHE_DIR)`` (``worker/app.py:117-124``) and its sharder shards a loaded HF
model (``master/dashboard/management/commands/shard_model.py:37,55-96``). Here a checkpoint
directory is read without transformers at run time:

* ``config.json`` -> ``ModelConfig`` (``config_from_hf``);
* ``model.safetensors`` or ``model.safetensors.index.json`` + its shard files, read tensor by
  tensor through the C++ safetensors loader (mmap, no pickle) as ``from_hf_state_dict`` asks
  for them, so host memory holds the converted stage, not the checkpoint twice;
* ``layers`` / ``first`` / ``last`` select one pipeline stage's tensors (``shard-model
  --from-hf``, or a worker loading only its stage).

Directory forms accepted by ``find_hf_dir``: the directory itself, ``<root>/<name with / ->
_>/``, and the HF hub cache layout ``<root>/models--<org>--<name>/snapshots/<rev>/``.
"""
from __future__ import annotations

import json
from pathlib import Path
from typing import Dict, Iterable, Iterator, Optional, Tuple

import torch

from .configs import ModelConfig
from .weights import (from_buborax_state_dict, from_hf_state_dict, from_lapunex_state_dict,
                      from_pulunex_state_dict, from_risutar_state_dict)


def is_hf_dir(d) -> bool:
    d = Path(d)
    cj = d / "config.json"
    if not cj.exists():
        return False
    try:
        c = json.loads(cj.read_text())
    except (OSError, ValueError):
        return False
    return ("model_type" in c or c.get("architecture") in NATIVE_ARCHS) and ((d / "model.safetensors").exists()
                                  or (d / "model.safetensors.index.json").exists())


def find_hf_dir(root: str, name: str) -> Optional[Path]:
    """The HF checkpoint directory of ``name`` under ``root`` (see module docstring)."""
    r = Path(root)
    cands = [r / name.replace("/", "_"), r / name]
    hub = r / ("models--" + name.replace("/", "--"))
    snaps = hub / "snapshots"
    if snaps.is_dir():
        ref = hub / "refs" / "main"
        if ref.exists():
            cands.append(snaps / ref.read_text().strip())
        cands += sorted(snaps.iterdir(), key=lambda p: p.stat().st_mtime, reverse=True)
    for c in cands:
        if c.is_dir() and is_hf_dir(c):
            return c
    return None


NATIVE_ARCHS = ("Buborax", "Pulunex", "Risutar", "Lapunex")


def buborax_config(c: dict, name: Optional[str] = None) -> ModelConfig:
    """A Buborax ``config.json``: ``width``, ``vocab``, ``norm`` {eps, groups},
    ``residual_mult``, ``loop`` {start, stop, times} (optional) and ``layers``, a list of
    {type, mixer {...}, mlp {kind, ff} or null}. Every size and constant is read from it."""
    from .configs import LayerSpec, hybrid_config
    specs = []
    for L in c["layers"]:
        mx, kind = L["mixer"], L["type"]
        mlp = L.get("mlp")
        if mlp and mlp.get("kind", "dense") != "dense":
            raise ValueError(f"unsupported feed-forward kind '{mlp.get('kind')}'")
        ff = int(mlp["ff"]) if mlp else 0
        H, d = int(mx["heads"]), int(mx["dim"])
        # no mask: every earlier position is visible
        win = int((mx.get("mask") or {}).get("size") or (1 << 30))
        if kind == "attention":
            G = int(mx.get("kv_heads") or H)
            dv = int(mx.get("vdim", d))
            if dv != d or H % G:
                raise ValueError("attention: the values are the keys (vdim == dim) and heads "
                                 "must be a multiple of kv_heads")
            specs.append(LayerSpec("attention", heads=H, kv_heads=G, dim=d, vdim=dv,
                                   window=win, scale=float(mx.get("scale", d ** -0.5)), ff=ff))
        elif kind == "hgrn2":
            specs.append(LayerSpec("hgrn2", heads=H, dim=d, vdim=int(mx["vdim"]), ff=ff))
        elif kind == "latent_attention":
            rot = mx.get("rot") or {}
            dr = int(mx["rot_dim"])
            specs.append(LayerSpec("latent_attention", heads=H, kv_heads=1, dim=d,
                                   vdim=int(mx["vdim"]), window=win,
                                   scale=float(mx.get("scale", (d + dr) ** -0.5)), rot_dim=dr,
                                   kv_rank=int(mx["kv_rank"]), rot_dims=int(rot.get("dims", dr)),
                                   rot_base=float(rot.get("base", 10000.0)), ff=ff))
        else:
            raise ValueError(f"unsupported mixer type '{kind}'")
    lp = c.get("loop")
    loop = (int(lp["start"]), int(lp["stop"]), int(lp["times"])) if lp else ()
    if loop and not (0 <= loop[0] < loop[1] <= len(specs) and loop[2] >= 1):
        raise ValueError(f"bad loop {loop} for {len(specs)} layers")
    norm = c.get("norm") or {}
    return hybrid_config(name or c.get("_name_or_path") or "buborax", int(c["width"]),
                         int(c["vocab"]), specs, loop, int(norm.get("groups", 1)),
                         float(norm.get("eps", 1e-6)), float(c.get("residual_mult", 1.0)))


def pulunex_config(c: dict, name: Optional[str] = None) -> ModelConfig:
    """A Pulunex ``config.json``: ``width``, ``vocab``, ``max_positions``, ``embedding``
    {scale}, ``logit_scale``, ``norm`` {eps} and ``layers``, a list of {type, mixer {heads,
    kv_heads, dim, vdim, scale, mask {size}, kv_from}, mlp} with mlp null, {kind: dense, ff} or
    {kind: moe, expert {ff}, router {experts, identity, top}, shared {ff}}. Every size and
    constant is read from it."""
    from .configs import LayerSpec, hybrid_config
    specs = []
    for i, L in enumerate(c["layers"]):
        mx, kind = L["mixer"], L["type"]
        if kind != "attention":
            raise ValueError(f"unsupported mixer type '{kind}'")
        H, d = int(mx["heads"]), int(mx["dim"])
        G = int(mx.get("kv_heads") or H)
        if H % G:
            raise ValueError("attention: heads must be a multiple of kv_heads")
        src = mx.get("kv_from")
        src = -1 if src is None else int(src)
        if src >= 0:
            o = specs[src] if src < i else None
            if o is None or o.kv_from >= 0 or (o.kv_heads, o.dim, o.vdim) != (
                    G, d, int(mx.get("vdim", d))):
                raise ValueError(f"layer {i}: kv_from {src} must name an earlier layer with "
                                 "projections of its own and the same key / value sizes")
        ff = dict(ff=0)
        mlp = L.get("mlp")
        if mlp:
            fk = mlp.get("kind", "dense")
            if fk == "dense":
                ff = dict(ff=int(mlp["ff"]), ff_kind="gelu")
            elif fk == "moe":
                r = mlp["router"]
                ff = dict(ff=int(mlp["expert"]["ff"]), ff_kind="moe", experts=int(r["experts"]),
                          identity=int(r.get("identity") or 0), top=int(r["top"]),
                          shared_ff=int((mlp.get("shared") or {}).get("ff") or 0))
                if not 1 <= ff["top"] <= ff["experts"] + ff["identity"]:
                    raise ValueError(f"layer {i}: router.top {ff['top']} of "
                                     f"{ff['experts'] + ff['identity']} experts")
            else:
                raise ValueError(f"unsupported feed-forward kind '{fk}'")
        specs.append(LayerSpec("talk_attention", heads=H, kv_heads=G, dim=d,
                               vdim=int(mx.get("vdim", d)),
                               scale=float(mx.get("scale", d ** -0.5)),
                               chunk=int((mx.get("mask") or {}).get("size") or 0), kv_from=src,
                               shift=True, **ff))
    norm = c.get("norm") or {}
    return hybrid_config(name or c.get("_name_or_path") or "pulunex", int(c["width"]),
                         int(c["vocab"]), specs, norm_eps=float(norm.get("eps", 1e-6)),
                         arch="pulunex", max_position=int(c["max_positions"]),
                         embed_scale=float((c.get("embedding") or {}).get("scale", 1.0)),
                         logit_scale=float(c.get("logit_scale", 1.0)), learned_pos=True,
                         scalar_norm=True)


def risutar_config(c: dict, name: Optional[str] = None) -> ModelConfig:
    """A Risutar ``config.json``: ``width``, ``vocab``, ``norm`` {eps}, ``postln_alpha``,
    ``embedding`` {bigram {buckets, mul_prev, mul_cur}} (optional), ``token_side`` {dim}
    (optional) and ``layers``, a list of {type, mixer, mlp}: type ``gla`` with mixer {heads, dim,
    vdim, tau} or ``latent_attention`` with mixer {heads, dim, rot_dim, vdim, kv_rank, q_rank,
    scale, rot {base, dims}, kv_from}; mlp null, {kind: dense, ff} or {kind: moe, expert {ff},
    router {experts, top}, shared {ff}}. Sizes a config does not carry (the decay's inner
    width) come from the tensors' shapes at load time."""
    from .configs import LayerSpec, hybrid_config
    specs = []
    for i, L in enumerate(c["layers"]):
        mx, kind = L["mixer"], L["type"]
        ff = dict(ff=0)
        mlp = L.get("mlp")
        if mlp:
            fk = mlp.get("kind", "dense")
            if fk == "dense":
                ff = dict(ff=int(mlp["ff"]), ff_kind="gated_silu")
            elif fk == "moe":
                r = mlp["router"]
                ff = dict(ff=int(mlp["expert"]["ff"]), ff_kind="moe", router="logit_topk",
                          expert_act="gelu_erf", experts=int(r["experts"]), top=int(r["top"]),
                          shared_ff=int((mlp.get("shared") or {}).get("ff") or 0))
                if not 1 <= ff["top"] <= ff["experts"]:
                    raise ValueError(f"layer {i}: router.top {ff['top']} of {ff['experts']} experts")
            else:
                raise ValueError(f"unsupported feed-forward kind '{fk}'")
        H, d = int(mx["heads"]), int(mx["dim"])
        if kind == "gla":
            specs.append(LayerSpec("gla", heads=H, dim=d, vdim=int(mx.get("vdim", d)),
                                   tau=float(mx.get("tau", 1.0)),
                                   decay_rank=int(mx.get("decay_rank") or 0), **ff))
        elif kind == "latent_attention":
            rot = mx.get("rot") or {}
            dr = int(mx["rot_dim"])
            src = mx.get("kv_from")
            src = -1 if src is None else int(src)
            r = int(mx["kv_rank"])
            if src >= 0:
                o = specs[src] if src < i else None
                if (o is None or o.kind != "latent_attention" or o.kv_from >= 0
                        or (o.kv_rank, o.rot_dim) != (r, dr)):
                    raise ValueError(f"layer {i}: kv_from {src} must name an earlier latent-"
                                     "attention layer with a projection of its own and the "
                                     "same latent and rotated sizes")
            specs.append(LayerSpec("latent_attention", heads=H, kv_heads=1, dim=d,
                                   vdim=int(mx["vdim"]), window=1 << 30,
                                   scale=float(mx.get("scale", (d + dr) ** -0.5)), rot_dim=dr,
                                   kv_rank=r, rot_dims=int(rot.get("dims", dr)),
                                   rot_base=float(rot.get("base", 10000.0)),
                                   q_rank=int(mx.get("q_rank") or 0), head_gate=True,
                                   rot_half=True, kv_from=src, **ff))
        else:
            raise ValueError(f"unsupported mixer type '{kind}'")
    bg = (c.get("embedding") or {}).get("bigram")
    bigram = (int(bg["buckets"]), int(bg["mul_prev"]), int(bg["mul_cur"])) if bg else ()
    return hybrid_config(name or c.get("_name_or_path") or "risutar", int(c["width"]),
                         int(c["vocab"]), specs, norm_eps=float((c.get("norm") or {}).get("eps", 1e-5)),
                         arch="risutar", post_norm=True, postln_alpha=float(c.get("postln_alpha", 1.0)),
                         bigram=bigram, side_dim=int((c.get("token_side") or {}).get("dim") or 0))


def lapunex_config(c: dict, name: Optional[str] = None) -> ModelConfig:
    """A Lapunex ``config.json``: ``width``, ``vocab``, ``norm`` {eps}, ``embedding`` {scale},
    ``streams`` (optional: hyper-connected copies of the residual stream), ``loop`` {start,
    stop, times} (optional) and ``layers``, a list of {type, mixer, mlp}: type ``lightning``
    with mixer {heads, dim, vdim, decay [per head]} or ``parallel`` with mixer {left {heads,
    kv_heads, dim, vdim, scale, rot {base, dims, scaling {factor, original, fast, slow}}},
    right {heads, dim, vdim, gate_cap}, left_scale, right_scale}; mlp null, {kind: dense, ff}
    or {kind: moe, expert {ff, limit}, router {experts, top, scale, groups {count, keep}}}.
    Every size and constant is read from it."""
    from .configs import LayerSpec, hybrid_config
    specs = []
    for i, L in enumerate(c["layers"]):
        mx, kind = L["mixer"], L["type"]
        ff = dict(ff=0)
        mlp = L.get("mlp")
        if mlp:
            fk = mlp.get("kind", "dense")
            if fk == "dense":
                ff = dict(ff=int(mlp["ff"]), ff_kind="gated_silu")
            elif fk == "moe":
                r, gr = mlp["router"], mlp["router"].get("groups") or {}
                ff = dict(ff=int(mlp["expert"]["ff"]), ff_kind="moe", router="group_score",
                          expert_act="clamp_swish", experts=int(r["experts"]), top=int(r["top"]),
                          router_groups=int(gr.get("count") or 1),
                          router_keep=int(gr.get("keep") or gr.get("count") or 1),
                          router_scale=float(r.get("scale", 1.0)),
                          act_limit=float(mlp["expert"]["limit"]))
                E, ng, keep = ff["experts"], ff["router_groups"], ff["router_keep"]
                if E % ng or not 1 <= keep <= ng or not 1 <= ff["top"] <= keep * (E // ng):
                    raise ValueError(f"layer {i}: router of {E} experts in {ng} groups, "
                                     f"{keep} kept, top {ff['top']}")
            else:
                raise ValueError(f"unsupported feed-forward kind '{fk}'")
        if kind == "lightning":
            H = int(mx["heads"])
            decays = tuple(float(a) for a in mx["decay"])
            if len(decays) != H:
                raise ValueError(f"layer {i}: {len(decays)} decays for {H} heads")
            specs.append(LayerSpec("lightning", heads=H, dim=int(mx["dim"]),
                                   vdim=int(mx.get("vdim", mx["dim"])), decays=decays, **ff))
        elif kind == "parallel":
            l, r = mx["left"], mx["right"]
            Hl, d = int(l["heads"]), int(l["dim"])
            G = int(l.get("kv_heads") or Hl)
            if Hl % G:
                raise ValueError(f"layer {i}: heads must be a multiple of kv_heads")
            rot = l.get("rot") or {}
            sc = rot.get("scaling")
            dims = int(rot.get("dims") or 0)
            if dims % 2 or dims > d:
                raise ValueError(f"layer {i}: rot.dims {dims} of a head of {d}")
            left = LayerSpec(
                "sink_attention", heads=Hl, kv_heads=G, dim=d, vdim=int(l.get("vdim", d)),
                scale=float(l.get("scale", d ** -0.5)), rot_dims=dims,
                rot_base=float(rot.get("base", 10000.0)), window=1 << 30,
                rot_scaling=((float(sc["factor"]), float(sc["original"]), float(sc["fast"]),
                              float(sc["slow"])) if sc else ()))
            right = LayerSpec("mlstm", heads=int(r["heads"]), dim=int(r["dim"]),
                              vdim=int(r.get("vdim", r["dim"])), gate_cap=float(r["gate_cap"]))
            specs.append(LayerSpec("parallel", heads=max(Hl, right.heads), kv_heads=G,
                                   dim=max(d, right.dim), vdim=max(left.vdim, right.vdim),
                                   left=left, right=right,
                                   left_scale=float(mx.get("left_scale", 1.0)),
                                   right_scale=float(mx.get("right_scale", 1.0)), **ff))
        else:
            raise ValueError(f"unsupported mixer type '{kind}'")
    lp = c.get("loop")
    loop = (int(lp["start"]), int(lp["stop"]), int(lp["times"])) if lp else ()
    if loop and not (0 <= loop[0] < loop[1] <= len(specs) and loop[2] >= 1):
        raise ValueError(f"bad loop {loop} for {len(specs)} layers")
    return hybrid_config(name or c.get("_name_or_path") or "lapunex", int(c["width"]),
                         int(c["vocab"]), specs, loop,
                         norm_eps=float((c.get("norm") or {}).get("eps", 1e-5)), arch="lapunex",
                         embed_scale=float((c.get("embedding") or {}).get("scale", 1.0)),
                         streams=int(c.get("streams") or 0), norm_offset=1.0, loop_entry=False)


def config_from_hf(c: dict, name: Optional[str] = None) -> ModelConfig:
    """Map a ``config.json``: HF llama / mistral / mixtral / gpt2 model types, or one of the
    native layer-list designs (``architecture``: Buborax, Pulunex, Risutar, Lapunex)."""
    if c.get("architecture") == "Buborax":
        return buborax_config(c, name)
    if c.get("architecture") == "Pulunex":
        return pulunex_config(c, name)
    if c.get("architecture") == "Risutar":
        return risutar_config(c, name)
    if c.get("architecture") == "Lapunex":
        return lapunex_config(c, name)
    mt = c.get("model_type", "")
    name = name or c.get("_name_or_path") or mt
    if mt == "gpt2":
        d = int(c["n_embd"])
        return ModelConfig(
            name=name, arch="gpt2", hidden_size=d, num_layers=int(c["n_layer"]),
            num_heads=int(c["n_head"]), num_kv_heads=int(c["n_head"]),
            head_dim=d // int(c["n_head"]), intermediate_size=int(c.get("n_inner") or 4 * d),
            vocab_size=int(c["vocab_size"]), max_position=int(c.get("n_positions", 1024)),
            rope_theta=0.0, norm_eps=float(c.get("layer_norm_epsilon", 1e-5)),
            tie_embeddings=True, bos_token_id=int(c.get("bos_token_id", 50256)),
            eos_token_id=_eos(c, 50256))
    if mt not in ("llama", "mistral", "mixtral"):
        raise ValueError(f"unsupported HF model_type '{mt}' (llama, mistral, mixtral, gpt2)")
    d, nh = int(c["hidden_size"]), int(c["num_attention_heads"])
    rope = c.get("rope_theta")
    params = c.get("rope_parameters") or {}
    if rope is None:
        rope = params.get("rope_theta", 10000.0)
    # rope scaling (Llama-3.1 / 3.2 "llama3", "linear"): absorbed into the cos/sin table;
    # transformers 5 keeps it in rope_parameters, older configs in rope_scaling
    sc = dict(c.get("rope_scaling") or {})
    if not sc and params.get("rope_type", "default") not in ("default", None):
        sc = {k: v for k, v in params.items() if k != "rope_theta"}
    if sc:
        from ..ops.reference import rope_scaled_inv_freq
        import torch as _t
        rope_scaled_inv_freq(_t.ones(2, dtype=_t.float64), sc)     # refuse unknown types now
    max_pos = int(c.get("max_position_embeddings", 8192))
    # sliding-window attention (Mistral): full attention equals it while a sequence fits the
    # window, so the model's context is capped there instead of silently diverging past it
    sw = c.get("sliding_window")
    if sw and int(sw) < max_pos:
        import logging
        logging.getLogger(__name__).warning(
            "sliding_window=%s < max_position_embeddings=%s: context capped at the window "
            "(sliding-window attention is not implemented)", sw, max_pos)
        max_pos = int(sw)
    return ModelConfig(
        name=name, arch="llama", hidden_size=d, num_layers=int(c["num_hidden_layers"]),
        num_heads=nh, num_kv_heads=int(c.get("num_key_value_heads") or nh),
        head_dim=int(c.get("head_dim") or d // nh),
        intermediate_size=int(c["intermediate_size"]), vocab_size=int(c["vocab_size"]),
        max_position=max_pos, rope_theta=float(rope),
        rope_scaling=tuple(sorted((str(k), v) for k, v in sc.items()
                                  if isinstance(v, (int, float, str)))),
        norm_eps=float(c.get("rms_norm_eps", 1e-5)),
        num_experts=int(c.get("num_local_experts", 0)) if mt == "mixtral" else 0,
        top_k_experts=int(c.get("num_experts_per_tok", 2)),
        tie_embeddings=bool(c.get("tie_word_embeddings", False)),
        bos_token_id=int(c.get("bos_token_id") or 1), eos_token_id=_eos(c, 2))


def _eos(c: dict, default: int) -> int:
    e = c.get("eos_token_id", default)
    if isinstance(e, list):
        e = e[0] if e else default
    return int(default if e is None else e)


class LazyStateDict:
    """Mapping over every tensor of a (possibly multi-file) safetensors checkpoint; a tensor
    is read from disk (C++ loader, to host memory) when it is first asked for."""

    def __init__(self, d: Path):
        from ..runtime import SafetensorsFile
        self.dir = Path(d)
        idx = self.dir / "model.safetensors.index.json"
        if idx.exists():
            wm = json.loads(idx.read_text())["weight_map"]
            files = sorted(set(wm.values()))
        else:
            files = ["model.safetensors"]
            wm = None
        self._files = {f: SafetensorsFile(str(self.dir / f)) for f in files}
        self._where: Dict[str, str] = {}
        for f, st in self._files.items():
            for k in st.keys():
                self._where[k] = f
        if wm is not None:
            missing = [k for k in wm if k not in self._where]
            if missing:
                raise ValueError(f"{idx}: {len(missing)} indexed tensors missing, e.g. "
                                 f"{missing[0]}")

    def __contains__(self, k) -> bool:
        return k in self._where

    def __getitem__(self, k) -> torch.Tensor:
        f = self._where[k]
        return self._files[f].load([k])[k]

    def keys(self) -> Iterator[str]:
        return iter(self._where)

    def close(self) -> None:
        for st in self._files.values():
            st.close()


def load_hf_dir(d, device="cpu", dtype=torch.bfloat16, name: Optional[str] = None,
                layers: Optional[Iterable[int]] = None, first: bool = True,
                last: bool = True) -> Tuple[ModelConfig, Dict[str, torch.Tensor]]:
    """(config, our parameter dict on ``device``) from a HF checkpoint directory; with
    ``layers`` / ``first`` / ``last`` only that pipeline stage's tensors."""
    d = Path(d)
    cfg = config_from_hf(json.loads((d / "config.json").read_text()), name)
    sd = LazyStateDict(d)
    try:
        if cfg.arch == "pulunex":
            params = from_pulunex_state_dict(cfg, sd, dtype=dtype)
        elif cfg.arch == "risutar":
            cfg, params = from_risutar_state_dict(cfg, sd, dtype=dtype)
        elif cfg.arch == "lapunex":
            params = from_lapunex_state_dict(cfg, sd, dtype=dtype)
        elif cfg.is_hybrid:
            params = from_buborax_state_dict(cfg, sd, dtype=dtype)
        else:
            params = from_hf_state_dict(cfg, sd, layers=layers, first=first, last=last,
                                        dtype=dtype)
    finally:
        sd.close()
    dev = torch.device(device)
    if dev.type != "cpu":
        params = {k: v.to(dev, non_blocking=True) for k, v in params.items()}
        torch.cuda.synchronize(dev)
    return cfg, params
