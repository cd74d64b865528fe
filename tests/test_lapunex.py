"""Lapunex against the plain float64 oracle in ``lapunex_oracle.py``.

Every test builds its own small configuration and random weights, runs the framework (config
reader, weight conversion, engine, scheduler, block manager, state slots, runner, model, ops)
and compares with the oracle's whole-sequence functions. CPU cases run the PyTorch reference
ops in fp32; GPU cases run the HIP kernels in bf16 and fp32.
"""
import copy

import numpy as np
import pytest
import torch

import lapunex_oracle as O
from distributed_llm_inferencing_amd.engine import SamplingParams
from distributed_llm_inferencing_amd.engine.llm_engine import LLMEngine
from distributed_llm_inferencing_amd.models.hf import config_from_hf
from distributed_llm_inferencing_amd.models.weights import from_lapunex_state_dict
from distributed_llm_inferencing_amd.ops import hybrid as H

CASES = [("cpu", torch.float32),
         pytest.param("cuda", torch.float32, marks=pytest.mark.gpu),
         pytest.param("cuda", torch.bfloat16, marks=pytest.mark.gpu)]


def dense(ff=40):
    return {"kind": "dense", "ff": ff}


def moe(ff=12, experts=6, top=2, scale=1.3, limit=1.2, groups=(3, 2)):
    r = {"experts": experts, "top": top, "scale": scale}
    if groups:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": r}


def lightning(heads=2, dim=8, vdim=12, decay=None, mlp=None):
    decay = decay or [0.3 + 0.69 * (i + 1) / heads for i in range(heads)]
    return {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay},
            "mlp": mlp}


def rot(dims=4, base=50.0, scaling=(4.0, 24, 3.0, 1.0)):
    r = {"base": base, "dims": dims}
    if scaling:
        r["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return r


def left(heads=4, kv_heads=2, dim=8, vdim=6, scale=0.3, rot_=None):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
            "rot": rot() if rot_ is None else rot_}


def right(heads=2, dim=4, vdim=10, cap=8.0):
    return {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}


def parallel(l=None, r=None, ls=0.7, rs=1.2, mlp=None):
    return {"type": "parallel", "mixer": {"left": l or left(), "right": r or right(),
                                          "left_scale": ls, "right_scale": rs}, "mlp": mlp}


def config(layers, width=40, vocab=80, eps=2e-5, scale=3.0, streams=2, loop=None):
    c = {"architecture": "Lapunex", "width": width, "vocab": vocab, "norm": {"eps": eps},
         "embedding": {"scale": scale}, "layers": layers}
    if streams:
        c["streams"] = streams
    if loop:
        c["loop"] = dict(zip(("start", "stop", "times"), loop))
    return c


def without_routing(c):
    c = copy.deepcopy(c)
    for L in c["layers"]:
        if L["mlp"] and L["mlp"]["kind"] == "moe":
            L["mlp"] = dense(16)
    return c


FULL = config([lightning(mlp=dense()), parallel(mlp=moe()),
               lightning(heads=3, dim=4, vdim=4, mlp=moe(experts=4, top=1, groups=(2, 1))),
               parallel(l=left(heads=2, kv_heads=2, dim=16, vdim=4, rot_=rot(16, 10.0, None)),
                        r=right(heads=1, dim=16, vdim=8, cap=3.0), mlp=None),
               lightning(heads=1, dim=16, vdim=8, mlp=dense(24))], streams=4, loop=(1, 3, 3))


def engine(c, w, device, dtype, max_tokens=512, live=4, block_size=8, **kw):
    cfg = config_from_hf(c)
    params = from_lapunex_state_dict(cfg, {k: torch.as_tensor(v) for k, v in w.items()}, dtype=dtype)
    return LLMEngine(cfg, device=device, dtype=dtype, params=params, max_batch=live,
                     max_model_len=1 << 20, block_size=block_size,
                     num_blocks=-(-max_tokens // block_size) + live,
                     use_graphs=kw.pop("graphs", False), lookahead=kw.pop("lookahead", False), **kw)


def tol(dtype):
    return 2e-4 if dtype == torch.float32 else 8e-2


class Ref:
    """Oracle logits of a sequence with each position's closest routing decision."""

    def __init__(self, logits, margins):
        self.logits, self.margins = logits, np.asarray(margins)

    def __getitem__(self, k):
        return Ref(self.logits[k], self.margins[k])


def ref(tokens, c, w):
    return Ref(O.forward(c, w, tokens), O.route_margins(c, w, tokens))


def close(got, want, dtype, what="", slack=1.0):
    """Row error as a logit comparison sees it: mean removed, relative to the spread. In bf16
    a position whose routing was a close call (the rounded input may choose another expert)
    and the positions after it (they read its state and keys) only have to stay bounded; every
    position before, every position of a model without routing, and fp32 everywhere, is held
    to the strict bound."""
    loose = None
    if isinstance(want, Ref):
        if dtype == torch.bfloat16:
            loose = np.maximum.accumulate(want.margins < 0.03)
        want = want.logits
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    err = np.sqrt((d ** 2).mean(-1)) / want.std()
    if loose is not None and loose.any():
        assert err[loose].max() < 2.5, what
        err = err[~loose]
    if err.size:
        assert err.max() < slack * tol(dtype), \
            f"{what}: error {err.max():.3g} at row {int(err.argmax())}"


def replay(eng, tokens, cuts, rid="a"):
    """Feed ``tokens`` in portions ``cuts``; returns the logits of every position."""
    out, at = [], 0
    for n in cuts:
        last = at + n == len(tokens)
        lg = eng.replay_step([(rid, tokens[at:at + n])], [list(range(n))], [rid] if last else [])
        out.append(lg.float().cpu().numpy())
        at += n
    assert at == len(tokens)
    return np.concatenate(out)


def toks(n, vocab, seed=1):
    return np.random.default_rng(seed).integers(0, vocab, n).tolist()


def dev_t(a, device, dtype=torch.float32):
    return torch.as_tensor(np.asarray(a), dtype=dtype).to(device)


def i32(a, device):
    return torch.tensor(np.asarray(a), dtype=torch.int32, device=device)


def layer_params(c, w, device, dtype, i=0):
    from distributed_llm_inferencing_amd.models.mixers import derive_constants
    cfg = config_from_hf(c)
    params = from_lapunex_state_dict(cfg, {k: torch.as_tensor(v) for k, v in w.items()}, dtype=dtype)
    lp = {k[len(f"layers.{i}."):]: v.to(device) for k, v in params.items()
          if k.startswith(f"layers.{i}.")}
    derive_constants(cfg.layer_specs[i], lp, torch.device(device))
    return cfg.layer_specs[i], lp


def hidden(T, D, seed):
    return O.bf16_exact(np.random.default_rng(seed).standard_normal((T, D)))


# ------------------------------------------------------------------ single mechanisms (ops)
@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("S,D", [(3, 40), (1, 24), (2, 30), (5, 7), (8, 64)])
def test_stream_mix_read_and_norm(device, dtype, S, D):
    """A sublayer's write-back through the stream mix, the next sublayer's weighted read, the
    norm with weights stored as offsets from one; the plain sum of the streams."""
    rng = np.random.default_rng(S * 10 + D)
    T, eps = 6, 1e-3
    xs, y = rng.standard_normal((T, S, D)) * 2, rng.standard_normal((T, D))
    prev = np.concatenate([rng.standard_normal(S), rng.standard_normal(S),
                           (np.eye(S) + 0.3 * rng.standard_normal((S, S))).reshape(-1)])
    nxt = np.concatenate([rng.standard_normal(S), np.zeros(S), np.zeros(S * S)])
    wn = O.bf16_exact(rng.standard_normal(D) * 0.3)
    mix = prev[2 * S:].reshape(S, S)
    new = np.einsum("sr,tsd->trd", mix, xs) + prev[S:2 * S][None, :, None] * y[:, None, :]
    u = np.einsum("s,tsd->td", nxt[:S], new)
    xt = dev_t(xs, device)
    h = H.hyper_mix(xt, dev_t(y, device), dev_t(prev, device), dev_t(nxt, device),
                    dev_t(wn, device, dtype), eps, 1.0)
    a = 2e-5 if dtype == torch.float32 else 3e-2
    np.testing.assert_allclose(xt.cpu().numpy(), new, atol=2e-5, rtol=2e-5)
    np.testing.assert_allclose(h.float().cpu().numpy(), O.norm1p(u, wn, eps), atol=a, rtol=a)
    # read without a write-back; the streams stay as they are; fp32 sum without a norm
    ones = torch.ones(S, device=device)
    got = H.hyper_mix(xt, None, None, ones, None)
    assert got.dtype == torch.float32
    np.testing.assert_allclose(got.cpu().numpy(), new.sum(1), atol=3e-5, rtol=3e-5)
    np.testing.assert_allclose(xt.cpu().numpy(), new, atol=2e-5, rtol=2e-5)


def test_yarn_frequencies_follow_their_definition():
    from distributed_llm_inferencing_amd.models.mixers import yarn_frequencies
    for r in (rot(), rot(16, 10000.0, (6.0, 1024, 24.0, 2.0)), rot(6, 7.0, None),
              rot(32, 500.0, (2.5, 100, 9.0, 2.0)), rot(2, 100.0, (40.0, 4096, 1.0, 1.0))):
        sc = r.get("scaling")
        f, m = yarn_frequencies(r["dims"], r["base"],
                                tuple(sc[k] for k in ("factor", "original", "fast", "slow")) if sc else ())
        fo, mo = O.yarn_frequencies(r)
        np.testing.assert_allclose(f.numpy(), fo, rtol=1e-12)
        assert abs(m - mo) < 1e-12
    # a pair that turns often keeps its frequency, a slow one is divided by the factor
    f, _ = yarn_frequencies(16, 10000.0, (6.0, 1024.0, 24.0, 2.0))
    plain = 10000.0 ** (-2.0 * np.arange(8) / 16)
    assert f[0] == plain[0] and abs(float(f[-1]) - plain[-1] / 6.0) < 1e-15


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("l", [left(), left(heads=1, kv_heads=1, dim=16, vdim=4, rot_=rot(16, 10.0, None)),
                               left(heads=6, kv_heads=1, dim=4, vdim=10, rot_=rot(2)),
                               left(heads=3, kv_heads=3, dim=6, vdim=3, rot_={"base": 10.0, "dims": 0}),
                               left(heads=4, kv_heads=2, dim=32, vdim=16, rot_=rot(8, 1000.0, (8.0, 32, 4.0, 0.5)))],
                         ids=["gqa", "one_head", "mqa", "no_rotation", "matrix_core_sizes"])
def test_sink_attention_through_shuffled_pages(device, dtype, l):
    """Whole-row q / k norm, partial rotation with scaled frequencies, sink in the denominator,
    one gate per head, output scale: whole and in portions through pages in any order. The
    matrix memory is silenced (right_scale 0) so that the layer's output is the attention's."""
    from distributed_llm_inferencing_amd.models.mixers import StepView, parallel_mixer
    T, D, eps, bs = 37, 24, 1e-5, 4
    c = config([parallel(l=l, r=right(heads=1, dim=4, vdim=4), ls=0.8, rs=0.0)], width=D)
    w = O.random_weights(c, l["heads"])
    w["l0.mix.left.sink"] = O.bf16_exact(np.linspace(-1.0, 3.0, l["heads"]))   # a sink that counts
    spec, lp = layer_params(c, w, device, dtype)
    h = hidden(T, D, 3)
    want = 0.8 * O.sink_attention(h, w, "l0.mix.left.", l, eps)
    # the sink matters: without it the result differs visibly
    w0 = dict(w)
    w0["l0.mix.left.sink"] = np.full(l["heads"], -60.0)
    assert np.abs(0.8 * O.sink_attention(h, w0, "l0.mix.left.", l, eps) - want).max() > 0.05
    nblk = -(-T // bs)
    perm = np.random.default_rng(1).permutation(nblk + 3)[:nblk]
    G, d, dv = l["kv_heads"], l["dim"], l["vdim"]
    a = 2e-4 if dtype == torch.float32 else 5e-2
    for cuts in ([T], [5, 1, 2, T - 8], [1] * T):
        cache = (torch.zeros((nblk + 3) * bs, G * d, dtype=dtype, device=device),
                 torch.zeros((nblk + 3) * bs, G * dv, dtype=dtype, device=device),
                 torch.zeros(2, 1, 4, 4, device=device), torch.zeros(2, 1, 5, device=device))
        got, at = [], 0
        for n in cuts:
            step = StepView(i32([0, n], device), n, i32(np.arange(at, at + n), device),
                            i32([perm[t // bs] * bs + t % bs for t in range(at, at + n)], device),
                            i32(perm[None], device), bs, i32([1], device), at + n)
            got.append(parallel_mixer(spec, lp, dev_t(h[at:at + n], device, dtype), step, cache,
                                      eps).float().cpu().numpy())
            at += n
        np.testing.assert_allclose(np.concatenate(got), want, atol=a, rtol=a)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("H_,d,dv", [(2, 8, 12), (3, 5, 3), (1, 16, 64), (2, 32, 16), (1, 64, 70),
                                     (1, 128, 32), (2, 16, 63)])
@pytest.mark.parametrize("form", ["lightning", "mlstm"])
def test_recurrences_and_their_state(device, dtype, form, H_, d, dv):
    """Both recurrences over portions and single tokens of two interleaved sequences whose
    slots held stale states, against the oracle run over each whole sequence."""
    from distributed_llm_inferencing_amd.models.mixers import (StepView, lightning_mixer,
                                                               parallel_mixer)
    D, eps = 24, 1e-5
    if form == "lightning":
        lay = lightning(H_, d, dv, decay=[0.999 - 0.4 * i / H_ for i in range(H_)])
    else:   # the attention side silenced
        lay = parallel(l=left(heads=1, kv_heads=1, dim=4, vdim=4), r=right(H_, d, dv, cap=6.0),
                       ls=0.0, rs=1.3)
    c = config([lay], width=D)
    w = O.random_weights(c, 5 + d)
    spec, lp = layer_params(c, w, device, dtype)
    hs = {"a": hidden(40, D, 1), "b": hidden(9, D, 2)}
    if form == "lightning":
        want = {k: O.lightning(v, w, "l0.mix.", lay["mixer"], eps) for k, v in hs.items()}
    else:
        want = {k: 1.3 * O.mlstm(v, w, "l0.mix.right.", lay["mixer"]["right"], eps)
                for k, v in hs.items()}
    bs = 64
    if form == "lightning":
        cache = (torch.full((3, H_, d, dv), 3.0, device=device),)
    else:
        cache = (torch.zeros(3 * bs, 4, dtype=dtype, device=device),
                 torch.zeros(3 * bs, 4, dtype=dtype, device=device),
                 torch.full((3, H_, d, dv), 3.0, device=device),
                 torch.full((3, H_, d + 1), -2.0, device=device))

    def run(parts):             # parts: [(name, slot, start, n)]
        rows = np.concatenate([hs[nm][s:s + n] for nm, _, s, n in parts])
        lens = [n for *_, n in parts]
        cu = i32(np.concatenate([[0], np.cumsum(lens)]), device)
        pos = np.concatenate([np.arange(s, s + n) for _, _, s, n in parts])
        slots = [sl for _, sl, _, _ in parts]
        sm = np.concatenate([sl * bs + np.arange(s, s + n) for _, sl, s, n in parts])
        step = StepView(cu, max(lens), i32(pos, device), i32(sm, device),
                        i32([[sl] for sl in slots], device), bs, i32(slots, device),
                        int(pos.max()) + 1)
        fn = lightning_mixer if form == "lightning" else parallel_mixer
        return fn(spec, lp, dev_t(rows, device, dtype), step, cache, eps).float().cpu().numpy()

    a = 3e-4 if dtype == torch.float32 else 6e-2
    got = run([("a", 2, 0, 19), ("b", 0, 0, 1)])
    np.testing.assert_allclose(got[:19], want["a"][:19], atol=a, rtol=a)
    np.testing.assert_allclose(got[19:], want["b"][:1], atol=a, rtol=a)
    got = run([("b", 0, 1, 1), ("a", 2, 19, 2)])
    np.testing.assert_allclose(got[:1], want["b"][1:2], atol=a, rtol=a)
    np.testing.assert_allclose(got[1:], want["a"][19:21], atol=a, rtol=a)
    got = run([("a", 2, 21, 1), ("b", 0, 2, 7)])
    np.testing.assert_allclose(got[:1], want["a"][21:22], atol=a, rtol=a)
    np.testing.assert_allclose(got[1:], want["b"][2:], atol=a, rtol=a)
    got = run([("a", 2, 22, 18)])
    np.testing.assert_allclose(got, want["a"][22:], atol=a, rtol=a)
    st = cache[0] if form == "lightning" else cache[2]
    assert float(st[1].min()) == 3.0 and float(st[1].max()) == 3.0


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("form", ["lightning", "mlstm"])
def test_long_portions_of_wide_states(device, dtype, form):
    """Portions long enough, and states wide enough, that a head's state columns are dealt to
    several workgroups (the matrix memory's norm then runs as a kernel of its own): a long
    portion, single tokens, another portion, against the oracle over the whole sequence."""
    from distributed_llm_inferencing_amd.models.mixers import (StepView, lightning_mixer,
                                                               parallel_mixer)
    D, eps, T, H_, d, dv = 32, 1e-5, 110, 2, 128, 128
    if form == "lightning":
        lay = lightning(H_, d, dv, decay=[0.97, 0.6])
    else:
        lay = parallel(l=left(heads=1, kv_heads=1, dim=4, vdim=4), r=right(H_, d, dv, cap=6.0),
                       ls=0.0, rs=0.9)
    c = config([lay], width=D)
    w = O.random_weights(c, 3)
    spec, lp = layer_params(c, w, device, dtype)
    h = hidden(T, D, 5)
    want = (O.lightning(h, w, "l0.mix.", lay["mixer"], eps) if form == "lightning"
            else 0.9 * O.mlstm(h, w, "l0.mix.right.", lay["mixer"]["right"], eps))
    bs = 128
    cache = ((torch.full((2, H_, d, dv), 3.0, device=device),) if form == "lightning" else
             (torch.zeros(2 * bs, 4, dtype=dtype, device=device),
              torch.zeros(2 * bs, 4, dtype=dtype, device=device),
              torch.full((2, H_, d, dv), 3.0, device=device),
              torch.full((2, H_, d + 1), -2.0, device=device)))
    got, at = [], 0
    for n in (70, 1, 1, 38):
        step = StepView(i32([0, n], device), n, i32(np.arange(at, at + n), device),
                        i32(bs + np.arange(at, at + n), device), i32([[1]], device), bs,
                        i32([1], device), at + n)
        fn = lightning_mixer if form == "lightning" else parallel_mixer
        got.append(fn(spec, lp, dev_t(h[at:at + n], device, dtype), step, cache,
                      eps).float().cpu().numpy())
        at += n
    a = 3e-4 if dtype == torch.float32 else 6e-2
    np.testing.assert_allclose(np.concatenate(got), want, atol=a, rtol=a)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("mlp", [moe(), moe(top=1), moe(experts=3, top=3, groups=(1, 1)),
                                 moe(groups=None), moe(experts=10, top=3, groups=(5, 3)),
                                 moe(ff=7, experts=9, top=3, groups=(3, 1), scale=0.4, limit=0.3),
                                 moe(experts=6, top=2, groups=(6, 2))],
                         ids=["usual", "top1", "all_experts", "no_groups", "five_groups",
                              "one_group_kept", "groups_of_one"])
def test_router_and_experts(device, dtype, mlp):
    """Softmax scores, group-limited choice, scaled un-renormalised weights, clamped experts."""
    from distributed_llm_inferencing_amd.models.mixers import moe_ff
    D, T = 24, 33
    c = config([lightning(mlp=mlp)], width=D)
    w = O.random_weights(c, 7)
    spec, lp = layer_params(c, w, device, dtype)
    h = hidden(T, D, 9)
    ids, wt, margin = O.route(h, w, "l0.mlp.", mlp["router"])
    assert margin.min() > 1e-4                        # no test rests on a tie
    tw, ti, _ = H.score_router(dev_t(h, device, dtype), lp["router"], None, spec.top, 0,
                               spec.router_groups, spec.router_keep, spec.router_scale)
    assert np.array_equal(np.sort(ti.cpu().numpy(), -1), np.sort(ids, -1))
    order = np.argsort(ti.cpu().numpy(), -1), np.argsort(ids, -1)
    np.testing.assert_allclose(np.take_along_axis(tw.cpu().numpy(), order[0], -1),
                               np.take_along_axis(wt, order[1], -1), atol=1e-5)
    got = moe_ff(spec, lp, dev_t(h, device, dtype)).cpu().numpy()
    a = 1e-4 if dtype == torch.float32 else 4e-2
    np.testing.assert_allclose(got, O.moe_ff(h, w, "l0.mlp.", mlp), atol=a, rtol=a)
    # the clamp is active somewhere, or the test would not see it
    g = h @ w["l0.mlp.e0.gate"].T
    assert (g > mlp["expert"]["limit"]).any()


# ------------------------------------------------------------------ whole models
@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("lay", [lightning(mlp=None), lightning(mlp=dense()), lightning(mlp=moe()),
                                 parallel(mlp=None), parallel(mlp=dense()), parallel(mlp=moe(top=1))],
                         ids=["lightning", "lightning_dense", "lightning_moe", "parallel",
                              "parallel_dense", "parallel_moe"])
def test_one_layer_models(lay, device, dtype):
    c = config([lay])
    w = O.random_weights(c, 11)
    t = toks(21, c["vocab"])
    eng = engine(c, w, device, dtype)
    close(replay(eng, t, [21]), ref(t, c, w), dtype, "one layer")


@pytest.mark.parametrize("device,dtype", CASES)
def test_layer_trace_matches_the_oracle(device, dtype):
    # in bf16 a routing close call moves a whole row and all rows after it: no routing there
    FULL = globals()["FULL"] if dtype == torch.float32 else without_routing(globals()["FULL"])
    w = O.random_weights(FULL, 2)
    t = toks(14, FULL["vocab"], 4)
    trace = []
    O.forward(FULL, w, t, trace)
    eng = engine(FULL, w, device, dtype)
    eng.model.layer_trace = []
    replay(eng, t, [14])
    assert len(eng.model.layer_trace) == len(trace) == 9          # 1 + 2 * 3 + 2 runs
    for i, (got, want) in enumerate(zip(eng.model.layer_trace, trace)):
        d = np.abs(got.cpu().numpy() - want).max(-1)
        lim = 1e-3 if dtype == torch.float32 else 3e-2 * np.abs(want).max()
        assert d.max() < lim, f"layer {i}"


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("routed", [True, False])
def test_prefill_equals_decode_equals_portions(device, dtype, routed):
    FULL = globals()["FULL"] if routed else without_routing(globals()["FULL"])
    w = O.random_weights(FULL, 1)
    t = toks(45, FULL["vocab"], 3)
    want = ref(t, FULL, w)
    for cuts in ([45], [1] * 45, [2] * 22 + [1], [7, 2, 9, 1, 1, 3, 16, 2, 4],
                 [30] + [1] * 15, [8, 8, 8, 8, 8, 5], [17, 16, 12]):
        eng = engine(FULL, w, device, dtype)
        close(replay(eng, t, cuts), want, dtype, f"cuts {cuts[:4]}")


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("routed", [True, False])
def test_mixed_batches_and_reuse_of_pages_and_slots(device, dtype, routed):
    """Unequal requests in one step (portions beside single tokens) against each alone, in a
    pool so small that pages and state slots are freed and taken again."""
    FULL = globals()["FULL"] if routed else without_routing(globals()["FULL"])
    w = O.random_weights(FULL, 4)
    V = FULL["vocab"]
    seqs = {k: toks(n, V, s) for k, n, s in (("a", 30, 1), ("b", 9, 2), ("c", 17, 3), ("d", 5, 4),
                                             ("e", 26, 5), ("f", 12, 6))}
    want = {k: ref(t, FULL, w) for k, t in seqs.items()}
    eng = engine(FULL, w, device, dtype, max_tokens=88, live=3)
    plan = [[("a", 6), ("b", 1)], [("a", 1), ("b", 2), ("c", 17)], [("a", 10), ("b", 6)],
            [("a", 13), ("d", 2)], [("d", 3), ("e", 20)], [("e", 1), ("f", 1)],
            [("e", 5), ("f", 9)], [("f", 2)]]
    at = {k: 0 for k in seqs}
    got = {k: [] for k in seqs}
    for step in plan:
        entries, wantidx, end = [], [], []
        for k, n in step:
            entries.append((k, seqs[k][at[k]:at[k] + n]))
            wantidx.append(list(range(n)))
            at[k] += n
            if at[k] == len(seqs[k]):
                end.append(k)
        lg = eng.replay_step(entries, wantidx, end).float().cpu().numpy()
        o = 0
        for k, n in step:
            got[k].append(lg[o:o + n])
            o += n
    for k in seqs:
        assert at[k] == len(seqs[k])
        close(np.concatenate(got[k]), want[k], dtype, f"request {k}")
    assert eng.bm.num_free == eng.bm.num_blocks and eng.state_slots.num_free == 3


@pytest.mark.parametrize("device,dtype", CASES)
def test_other_sizes_and_degenerate_values(device, dtype):
    """Sizes that differ where a usual model makes them equal, values of 1, one stream, no
    streams at all (a plain residual), no loop, a loop of one pass, a loop over everything."""
    cs = [
        config([parallel(l=left(heads=1, kv_heads=1, dim=4, vdim=3, rot_=rot(2)),
                         r=right(heads=1, dim=3, vdim=5, cap=1.0), ls=1.0, rs=1.0,
                         mlp=moe(ff=5, experts=2, top=2, groups=(1, 1), scale=1.0)),
                lightning(heads=1, dim=3, vdim=5, mlp=dense(7))],
               width=20, vocab=31, scale=1.0, streams=1),
        config([lightning(heads=5, dim=4, vdim=2, mlp=moe(experts=8, top=3, groups=(2, 1))),
                parallel(l=left(heads=6, kv_heads=3, dim=2, vdim=7, rot_=rot(2, 3.0, None)),
                         r=right(heads=3, dim=6, vdim=2), mlp=None),
                parallel(l=left(heads=2, kv_heads=1, dim=6, vdim=2, rot_=rot(6)),
                         r=right(heads=2, dim=2, vdim=3, cap=30.0), ls=2.0, rs=0.1, mlp=dense(9))],
               width=28, vocab=40, scale=7.0, streams=0, loop=(0, 3, 2)),
        config([parallel(mlp=dense()), lightning(mlp=None)], width=64, vocab=50, eps=1e-2,
               streams=4, loop=(1, 2, 1)),
        # nothing a multiple of 4: no kernel may take a vector path it is not aligned for
        config([parallel(l=left(heads=3, kv_heads=1, dim=6, vdim=3, rot_=rot(2)),
                         r=right(heads=3, dim=5, vdim=7), mlp=moe(ff=5, experts=3, top=2, groups=(3, 2))),
                lightning(heads=3, dim=5, vdim=7, mlp=dense(9)),
                lightning(heads=1, dim=7, vdim=9, decay=[1.0], mlp=None)],
               width=30, vocab=33, streams=2, loop=(1, 3, 3)),
        config([lightning(mlp=dense(12)), lightning(heads=2, dim=16, vdim=8, mlp=None)],
               width=32, vocab=37, streams=0),
    ]
    for n, c in enumerate(cs):
        w = O.random_weights(c, 20 + n)
        t = toks(19, c["vocab"], n)
        want = ref(t, c, w)
        eng = engine(c, w, device, dtype, block_size=4)
        close(replay(eng, t, [19]), want, dtype, f"config {n} whole")
        close(replay(eng, t, [3, 1, 2, 13]), want, dtype, f"config {n} portions")


@pytest.mark.parametrize("device,dtype", CASES)
def test_states_wider_than_a_workgroup(device, dtype):
    """States whose columns exceed what one workgroup keeps in registers (d a power of two) or
    in LDS (any other d): the columns are dealt to several workgroups in every step kind."""
    att = left(heads=2, kv_heads=1, dim=32, vdim=16, rot_=rot(8))
    cs = [config([lightning(heads=1, dim=128, vdim=320, mlp=None),
                  parallel(l=att, r=right(heads=1, dim=128, vdim=384), mlp=dense(64))],
                 width=64, vocab=90),
          config([lightning(heads=1, dim=200, vdim=192, mlp=None),
                  parallel(l=att, r=right(heads=1, dim=200, vdim=192), mlp=None)],
                 width=64, vocab=90, streams=0)]
    for n, c in enumerate(cs):
        w = O.random_weights(c, 3)
        t = toks(24, c["vocab"], 2)
        want = ref(t, c, w)
        eng = engine(c, w, device, dtype, max_tokens=128)
        close(replay(eng, t, [24]), want, dtype, f"config {n} whole")
        close(replay(eng, t, [17] + [1] * 7), want, dtype, f"config {n} decoded")


def standout_model():
    """One parallel layer whose attention finds one key: keys and queries share their
    projection and norm weights (one key head per query head), so among unit-RMS rows a key
    that points along the last token's query scores highest, and a large score scale makes it
    dominate (no rotation here: the first rotated pair always turns by one radian a position,
    which would favour the query's own key). The far token's embedding is the last token's plus a vector the query projection
    does not see: the same key direction, another value."""
    l = left(heads=2, kv_heads=2, dim=8, vdim=6, scale=6.0, rot_={"base": 10.0, "dims": 0})
    c = config([parallel(l=l, r=right(heads=1, dim=4, vdim=4), ls=1.0, rs=0.05)], width=24,
               vocab=64, streams=0)
    w = O.random_weights(c, 9)
    w["l0.mix.left.k"] = w["l0.mix.left.q"].copy()
    w["l0.mix.left.k.norm"] = w["l0.mix.left.q.norm"].copy()
    w["l0.mix.left.sink"] = np.zeros(2)
    w["l0.mix.left.v"] = w["l0.mix.left.v"] * 3.0
    w["l0.mix.left.g"] = w["l0.mix.left.g"] * 0.0                 # gates half open
    w["l0.mix.left.o"] = w["l0.mix.left.o"] * 6.0                 # the mixer outweighs the residual
    A = w["l0.mix.left.q"] * (1.0 + w["l0.norm1"])[None, :]      # what a key sees of the input
    null = np.linalg.svd(A)[2][A.shape[0]:]                       # [8, 24] directions it ignores
    delta = null.T @ np.random.default_rng(3).standard_normal(null.shape[0])
    w["embed"][61] = O.bf16_exact(w["embed"][62] + 1.5 * delta)
    return c, w


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("far", [1, 7, 8, 9, 250])
def test_far_keys_and_page_borders_stand_out(far, device, dtype):
    """One key, ``far`` positions back (around a page border, or hundreds away), dominates the
    last query's scores. The position's logits then depend on that one key being found."""
    c, w = standout_model()
    n = far + 6
    t = toks(n, 60, far)
    t[n - 1 - far] = 61                                   # a token used nowhere else
    t[n - 1] = 62
    want = ref(t, c, w)
    t2 = list(t)
    t2[n - 1 - far] = 60
    moved = np.abs(O.forward(c, w, t2)[-1] - want.logits[-1]).max()
    assert moved > 0.05
    eng = engine(c, w, device, dtype)
    close(replay(eng, t, [n]), want, dtype, "whole")
    close(replay(eng, t, [n - 3, 1, 1, 1]), want, dtype, "decoded")
    close(replay(eng, t, [n - 1 - far, 1] + ([far - 1] if far > 1 else []) + [1]), want, dtype,
          "cut at the key")


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("routed", [True, False])
def test_first_tokens_and_long_decode(device, dtype, routed):
    FULL = globals()["FULL"] if routed else without_routing(globals()["FULL"])
    w = O.random_weights(FULL, 6)
    t = toks(150, FULL["vocab"], 8)
    want = ref(t, FULL, w)
    eng = engine(FULL, w, device, dtype)
    got = replay(eng, t, [1, 1, 1, 2] + [1] * 145)
    close(got[:6], want[:6], dtype, "first tokens")
    close(got, want, dtype, "long decode", slack=1.0 if dtype == torch.float32 else 2.0)
    # the same slot and pages again, starting from a stale state
    t2 = toks(12, FULL["vocab"], 9)
    close(replay(eng, t2, [1] * 12), ref(t2, FULL, w), dtype, "reused")


@pytest.mark.parametrize("device,dtype,graphs", [
    ("cpu", torch.float32, False),
    pytest.param("cuda", torch.float32, False, marks=pytest.mark.gpu),
    pytest.param("cuda", torch.bfloat16, True, marks=pytest.mark.gpu)])
def test_greedy_generation_through_the_engine(device, dtype, graphs):
    """``LLMEngine.generate``: scheduler, chunked prefill, decode steps (captured graphs and
    lookahead on the GPU) against greedy decoding with the oracle. In bf16 the model has no
    routed layers: a routing close call would legitimately change the continuation."""
    c = copy.deepcopy(FULL) if dtype == torch.float32 else without_routing(FULL)
    w = O.random_weights(c, 12)
    w["head"] = w["head"] * 4.0                          # clear winners
    prompts = [toks(n, c["vocab"], s) for n, s in ((11, 1), (3, 2), (25, 3))]
    eng = engine(c, w, device, dtype, graphs=graphs, lookahead=graphs, max_prefill_tokens=16)
    outs = eng.generate(prompts, SamplingParams(max_new_tokens=8, do_sample=False, ignore_eos=True))
    for p, o in zip(prompts, outs):
        seq = list(p)
        assert len(o.output_ids) == 8
        for tok in o.output_ids:
            lg = O.forward(c, w, seq)[-1]
            best = int(lg.argmax())
            if tok != best:              # a near tie may fall the other way in reduced precision
                assert lg[best] - lg[tok] < (1e-3 if dtype == torch.float32 else 0.3)
            seq.append(tok)


def test_config_reader_reads_every_size():
    cfg = config_from_hf(FULL)
    assert cfg.arch == "lapunex" and cfg.is_hybrid and cfg.has_state
    assert (cfg.hidden_size, cfg.vocab_size, cfg.embed_scale, cfg.norm_eps) == (40, 80, 3.0, 2e-5)
    assert cfg.streams == 4 and cfg.loop == (1, 3, 3) and not cfg.loop_entry
    assert [li for li, _, first in cfg.layer_runs() if not first] == [0, 1, 2, 1, 2, 1, 2, 3, 4]
    s = cfg.layer_specs
    assert [x.kind for x in s] == ["lightning", "parallel", "lightning", "parallel", "lightning"]
    assert (s[0].heads, s[0].dim, s[0].vdim, s[0].ff_kind, s[0].ff) == (2, 8, 12, "gated_silu", 40)
    assert len(s[0].decays) == 2
    l, r = s[1].left, s[1].right
    assert (l.heads, l.kv_heads, l.dim, l.vdim, l.scale, l.rot_dims, l.rot_base) == (4, 2, 8, 6, 0.3, 4, 50.0)
    assert l.rot_scaling == (4.0, 24.0, 3.0, 1.0) and s[3].left.rot_scaling == ()
    assert (r.heads, r.dim, r.vdim, r.gate_cap) == (2, 4, 10, 8.0)
    assert (s[1].left_scale, s[1].right_scale) == (0.7, 1.2)
    assert (s[1].router, s[1].expert_act, s[1].experts, s[1].top, s[1].router_groups,
            s[1].router_keep, s[1].router_scale, s[1].act_limit) == ("group_score", "clamp_swish", 6, 2, 3, 2, 1.3, 1.2)
    assert s[3].ff == 0 and cfg.cache_row_width(1) == 2 * (8 + 6) and cfg.cache_row_width(0) == 0
    # the configuration survives the dictionary form the workers exchange
    from distributed_llm_inferencing_amd.models.configs import ModelConfig
    assert ModelConfig.from_dict(cfg.to_dict()) == cfg
    params = from_lapunex_state_dict(cfg, {k: torch.as_tensor(v) for k, v in
                                           O.random_weights(FULL, 0).items()})
    assert params["layers.1.hc2"].shape == (24,) and params["layers.1.hc2"].dtype == torch.float32
    assert params["layers.1.wo"].shape == (40, 4 * 6 + 2 * 10)
    bad = copy.deepcopy(FULL)
    bad["layers"][1]["mlp"]["router"]["groups"]["count"] = 4      # 6 experts in 4 groups
    with pytest.raises(ValueError):
        config_from_hf(bad)
    bad = copy.deepcopy(FULL)
    bad["layers"][0]["mixer"]["decay"] = [0.5]
    with pytest.raises(ValueError):
        config_from_hf(bad)


def test_registry_model_random_init_generates():
    eng = LLMEngine("lapunex-tiny", device="cpu", dtype=torch.float32, max_batch=2,
                    max_model_len=64, block_size=8, num_blocks=24, use_graphs=False)
    outs = eng.generate([[1, 2, 3], [4, 5, 6, 7, 8]], SamplingParams(max_new_tokens=4, do_sample=False,
                                                                    ignore_eos=True))
    assert all(len(o.output_ids) == 4 for o in outs)


@pytest.mark.gpu
@pytest.mark.parametrize("width,lay,n", [
    (128, lightning(heads=2, dim=16, vdim=32, mlp=moe(ff=64, experts=4, top=2, groups=(2, 1))), 70),
    (64, parallel(l=left(heads=4, kv_heads=2, dim=32, vdim=16, rot_=rot(8)),
                  r=right(heads=2, dim=16, vdim=16), mlp=moe(ff=128, experts=3, top=1, groups=None)), 33),
    (128, lightning(heads=1, dim=32, vdim=64, mlp=dense(192)), 41),
    (192, parallel(l=left(heads=8, kv_heads=2, dim=64, vdim=32, scale=0.12, rot_=rot(16, 1000.0)),
                   r=right(heads=2, dim=64, vdim=64),
                   mlp=moe(ff=64, experts=8, top=3, groups=(4, 3))), 300)],
    ids=["lightning_moe", "parallel_moe_top1", "dense", "matrix_core_attention"])
def test_tuned_layouts_and_matrix_core_attention(width, lay, n):
    """Sizes the tuned GEMM tiles and the matrix-core attention take: the dense feed-forward's
    activation runs as a GEMM epilogue, the experts as grouped GEMMs, the attention (sink,
    head gates, output scale) on the MFMA kernel, also split over keys for single tokens at a
    long context; whole prompts, portions and single tokens."""
    c = config([lay, lay], width=width, vocab=96)
    w = O.random_weights(c, width + n)
    t = toks(n, 96, n)
    want = ref(t, c, w)
    eng = engine(c, w, "cuda", torch.bfloat16, max_tokens=640)
    assert "ff_tuned" in eng.model.layers[0]
    close(replay(eng, t, [n]), want, torch.bfloat16, "whole")
    close(replay(eng, t, [n - 9, 2, 1, 1, 5]), want, torch.bfloat16, "portions")
    close(replay(eng, t, [n - 20] + [1] * 20), want, torch.bfloat16, "decoded")


def test_checkpoint_folder_through_the_replay_command(tmp_path, monkeypatch, capsys):
    """A checkpoint folder (config.json + model.safetensors in bfloat16) read by the C++
    safetensors loader, and the trace replay command driving the engine: two requests in mixed
    steps, logits written per step."""
    import io
    import json
    from safetensors.torch import save_file
    from distributed_llm_inferencing_amd.cli import main as cli_main
    c = config([lightning(mlp=moe()), parallel(mlp=dense())], loop=(0, 2, 2))
    w = O.random_weights(c, 21)
    model = tmp_path / "model"
    model.mkdir()
    (model / "config.json").write_text(json.dumps(c))
    save_file({k: torch.as_tensor(v).to(torch.bfloat16).contiguous() for k, v in w.items()},
              str(model / "model.safetensors"))
    ta, tb = toks(21, c["vocab"], 1), toks(9, c["vocab"], 2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": ta[:13], "want": [0, 12]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": ta[13:14], "want": [0]},
                                     {"id": "b", "tokens": tb, "want": [3, 8]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": ta[14:], "want": []}], "end": ["a"]}]
    monkeypatch.setattr("sys.stdin", io.StringIO("\n".join(json.dumps(s) for s in steps) + "\n"))
    out = tmp_path / "out"
    rc = cli_main(["trace-run", "--model", str(model), "--dtype", "float32", "--out", str(out),
                   "--max-tokens", "128", "--device", "cpu"])
    assert rc == 0
    assert [ln for ln in capsys.readouterr().out.splitlines() if ln.startswith("done")] == \
        ["done 0", "done 1", "done 2"]
    ra, rb = O.forward(c, w, ta), O.forward(c, w, tb)
    V = c["vocab"]
    got0 = np.fromfile(out / "0.f32", dtype="<f4").reshape(-1, V)
    got1 = np.fromfile(out / "1.f32", dtype="<f4").reshape(-1, V)
    close(got0, ra[[0, 12]], torch.float32, "step 0")
    close(got1, np.stack([ra[13], rb[3], rb[8]]), torch.float32, "step 1")
    assert not (out / "2.f32").exists()
