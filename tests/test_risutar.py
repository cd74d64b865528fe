"""Risutar against the plain float64 oracle in ``risutar_oracle.py``.

Every test builds its own small configuration and random weights, runs the framework (config
reader, weight conversion, engine, scheduler, block manager, state slots, runner, model, ops)
and compares with the oracle's whole-sequence functions. CPU cases run the PyTorch reference
ops in fp32; GPU cases run the HIP kernels in bf16 and fp32.
"""
import copy

import numpy as np
import pytest
import torch

import risutar_oracle as O
from distributed_llm_inferencing_amd.engine import SamplingParams
from distributed_llm_inferencing_amd.engine.llm_engine import LLMEngine
from distributed_llm_inferencing_amd.models.hf import config_from_hf
from distributed_llm_inferencing_amd.models.weights import from_risutar_state_dict
from distributed_llm_inferencing_amd.ops import hybrid as H

CASES = [("cpu", torch.float32),
         pytest.param("cuda", torch.float32, marks=pytest.mark.gpu),
         pytest.param("cuda", torch.bfloat16, marks=pytest.mark.gpu)]


def dense(ff=40):
    return {"kind": "dense", "ff": ff}


def moe(ff=12, experts=5, top=2, shared=20):
    m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def gla(heads=2, dim=8, vdim=12, tau=6.0, mlp=None):
    return {"type": "gla", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau},
            "mlp": mlp}


def latent(heads=3, dim=8, rot=4, vdim=10, kv_rank=12, q_rank=14, scale=0.3, base=100.0,
           kv_from=None, mlp=None):
    mx = {"heads": heads, "dim": dim, "rot_dim": rot, "vdim": vdim, "kv_rank": kv_rank,
          "q_rank": q_rank, "scale": scale, "rot": {"base": base, "dims": rot}}
    if kv_from is not None:
        mx["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": mx, "mlp": mlp}


def config(layers, width=40, vocab=80, eps=2e-6, alpha=2.5, bigram=(53, 11, 3), side=6):
    c = {"architecture": "Risutar", "width": width, "vocab": vocab, "norm": {"eps": eps},
         "postln_alpha": alpha, "layers": layers}
    if bigram:
        c["embedding"] = {"bigram": dict(zip(("buckets", "mul_prev", "mul_cur"), bigram))}
    if side:
        c["token_side"] = {"dim": side}
    return c


def without_routing(c):
    c = copy.deepcopy(c)
    for L in c["layers"]:
        if L["mlp"] and L["mlp"]["kind"] == "moe":
            L["mlp"] = dense(16)
    return c


FULL = config([gla(mlp=dense()), latent(mlp=moe()), latent(kv_from=1, mlp=moe(top=3, shared=0)),
               gla(heads=3, dim=4, vdim=4, tau=2.0, mlp=moe(experts=3, top=1)),
               latent(heads=2, dim=16, rot=8, vdim=4, kv_rank=8, q_rank=5, mlp=None),
               gla(heads=1, dim=16, vdim=8, mlp=dense(24))])


def engine(c, w, device, dtype, max_tokens=512, live=4, block_size=8, **kw):
    cfg, params = from_risutar_state_dict(config_from_hf(c), w, dtype=dtype)
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
    return Ref(O.forward(c, w, tokens).numpy(), O.route_margins(c, w, tokens))


def close(got, want, dtype, what="", slack=1.0):
    """Row error as a logit comparison sees it: mean removed, relative to the spread. In bf16
    a position whose routing was a close call (the rounded input may choose another expert,
    which with one expert per token swaps the whole feed-forward output) and the positions
    after it (they read its state and keys) only have to stay bounded; every position before,
    every position of a model without routing, and fp32 everywhere, is held to the strict
    bound."""
    loose = None
    if isinstance(want, Ref):
        if dtype == torch.bfloat16:
            loose = np.maximum.accumulate(want.margins < 0.02)
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
    return torch.tensor(a, dtype=torch.int32, device=device)


# ------------------------------------------------------------------ single mechanisms (ops)
@pytest.mark.parametrize("device,dtype", CASES)
def test_bigram_embedding_and_the_previous_token_state(device, dtype):
    """Hashed bigram rows; the token before a portion's first row comes from the sequence's
    slot, a sequence's first token takes the table's last row whatever the slot held."""
    c = config([gla()], vocab=70, bigram=(17, 29, 5))
    w = O.random_weights(c, 3)
    a, b = toks(9, 70, 1), toks(4, 70, 2)
    want_a, want_b = O.embed(c, w, a).numpy(), O.embed(c, w, b).numpy()
    state = i32([55, 66, 44], device)                       # stale contents of reused slots
    table, bg = dev_t(w["embed"], device, dtype), dev_t(w["bigram"], device, dtype)

    def run(ids, slots, lens, first_pos):
        cu = i32(np.concatenate([[0], np.cumsum(lens)]), device)
        pos = i32(np.concatenate([np.arange(p, p + n) for p, n in zip(first_pos, lens)]), device)
        idt = i32(ids, device)
        prev = H.prev_tokens(idt, state, i32(slots, device), cu, max(lens), pos)
        x, xs = H.embedding_bigram(idt, prev, table, bg, 17, 29, 5)
        assert xs.dtype == dtype
        np.testing.assert_allclose(xs.float().cpu().numpy(), x.cpu().numpy(),
                                   atol=0 if dtype == torch.float32 else 2e-2, rtol=1e-2)
        return x.cpu().numpy()

    got = run(a[:5] + b[:1], [2, 0], [5, 1], [0, 0])
    np.testing.assert_allclose(got[:5], want_a[:5], atol=1e-6)
    np.testing.assert_allclose(got[5:], want_b[:1], atol=1e-6)
    got = run(b[1:4] + a[5:6], [0, 2], [3, 1], [1, 5])
    np.testing.assert_allclose(got[:3], want_b[1:4], atol=1e-6)
    np.testing.assert_allclose(got[3:], want_a[5:6], atol=1e-6)
    got = run(a[6:9], [2], [3], [6])
    np.testing.assert_allclose(got, want_a[6:9], atol=1e-6)
    assert state.tolist() == [b[3], 66, a[8]]


@pytest.mark.parametrize("device,dtype", CASES)
def test_norm_after_the_sum_and_normed_side_input(device, dtype):
    rng = np.random.default_rng(0)
    T, D, eps = 7, 36, 1e-3
    x, y = rng.standard_normal((T, D)) * 3 + 1, rng.standard_normal((T, D))
    wn, bn = rng.random(D) + 0.5, rng.standard_normal(D)
    want = O.layer_norm(torch.tensor(1.7 * x + y), torch.tensor(wn), torch.tensor(bn), eps).numpy()
    xt = dev_t(x, device)
    h = H.postnorm(xt, dev_t(y, device), dev_t(wn, device, dtype), dev_t(bn, device, dtype), eps,
                   keep=1.7)
    a = 1e-5 if dtype == torch.float32 else 3e-2
    wq, bq = dev_t(wn, device, dtype).double().cpu(), dev_t(bn, device, dtype).double().cpu()
    want = O.layer_norm(torch.tensor(1.7 * x + y), wq, bq, eps).numpy()
    np.testing.assert_allclose(xt.cpu().numpy(), want, atol=1e-5, rtol=1e-5)
    np.testing.assert_allclose(h.float().cpu().numpy(), want, atol=a, rtol=a)
    # selected rows only, the stream untouched
    rows = torch.tensor([5, 0, 5], device=device)
    x2 = dev_t(x, device)
    h = H.postnorm(x2, None, dev_t(wn, device, dtype), dev_t(bn, device, dtype), eps, rows_idx=rows)
    np.testing.assert_allclose(x2.cpu().numpy(), x, atol=1e-6)
    np.testing.assert_allclose(h.float().cpu().numpy(),
                               O.layer_norm(torch.tensor(x), wq, bq, eps).numpy()[[5, 0, 5]],
                               atol=a, rtol=a)
    # x += y / rms(y) * w
    x3 = dev_t(x, device)
    h = H.add_rmsnormed(x3, dev_t(y, device), dev_t(wn, device, dtype), eps)
    want = x + (O.rms_div(torch.tensor(y), eps) * wq).numpy()
    np.testing.assert_allclose(x3.cpu().numpy(), want, atol=1e-5, rtol=1e-5)
    np.testing.assert_allclose(h.float().cpu().numpy(), want, atol=a, rtol=a)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("H_,d,dv,tau", [(2, 8, 12, 6.0), (3, 5, 3, 1.0), (1, 16, 64, 16.0),
                                         (2, 32, 16, 3.0), (1, 64, 70, 2.0), (1, 128, 32, 9.0)])
def test_gated_linear_attention_and_its_state(device, dtype, H_, d, dv, tau):
    """The recurrence over portions and single tokens of two interleaved sequences whose
    slots held stale states, against the oracle run over each whole sequence."""
    rng = np.random.default_rng(H_ * 100 + d)
    D, ra, eps = 24, 5, 1e-5
    m = {"heads": H_, "dim": d, "vdim": dv, "tau": tau}
    c = config([{"type": "gla", "mixer": m, "mlp": None}], width=D)
    w = {k[len("l0.mix."):]: v for k, v in O.random_weights(c, 5, decay_rank=ra).items()
         if k.startswith("l0.mix.")}
    w["o"] = torch.eye(H_ * dv, dtype=torch.float64)
    ha = O.bf16_exact(torch.randn(40, D, dtype=torch.float64))
    hb = O.bf16_exact(torch.randn(9, D, dtype=torch.float64))
    want = {"a": O.gla(m, w, "", ha, eps).numpy(), "b": O.gla(m, w, "", hb, eps).numpy()}
    hs = {"a": ha, "b": hb}
    state = torch.full((3, H_, d, dv), 3.0, device=device)
    w_in = torch.cat([w["q"], w["k"], w["v"], w["g"], w["a1"]], 0)

    def run(parts):             # parts: [(name, slot, start, n)]
        rows = torch.cat([hs[nm][s:s + n] for nm, _, s, n in parts])
        proj = dev_t(rows @ w_in.T, device)
        a1 = O.bf16_exact(proj[:, 2 * H_ * (d + dv):].cpu()) if dtype == torch.bfloat16 \
            else proj[:, 2 * H_ * (d + dv):].double().cpu()
        z = dev_t(a1 @ w["a2"].T, device)
        lens = [n for *_, n in parts]
        cu = i32(np.concatenate([[0], np.cumsum(lens)]), device)
        pos = i32(np.concatenate([np.arange(s, s + n) for _, _, s, n in parts]), device)
        return H.gla(proj, z, dev_t(w["a2.b"], device, dtype), tau, dev_t(w["norm"], device, dtype),
                     eps, state, i32([sl for _, sl, _, _ in parts], device), cu, max(lens), pos,
                     H_, d, dv).float().cpu().numpy()

    a = 2e-4 if dtype == torch.float32 else 4e-2
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
    assert float(state[1].min()) == 3.0 and float(state[1].max()) == 3.0


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("H_,d,dr,dv,r,rq", [(3, 8, 4, 10, 12, 14), (1, 16, 2, 4, 6, 3),
                                            (4, 32, 32, 16, 32, 24), (6, 4, 8, 4, 8, 8)])
def test_latent_attention_own_and_borrowed_cache(device, dtype, H_, d, dr, dv, r, rq):
    """Query latent, rotate-half rotation, absorbed attention over the cached latent through
    pages in any order, one gate per head; a second layer attends the first one's cache."""
    from distributed_llm_inferencing_amd.models.configs import LayerSpec
    from distributed_llm_inferencing_amd.models.mixers import (StepView, derive_constants,
                                                               latent_attention_mixer)
    T, D, eps, bs = 37, 24, 1e-5, 4
    lay = latent(H_, d, dr, dv, r, rq, scale=0.35, base=50.0)
    c = config([lay, latent(H_, d, dr, dv, r, rq, scale=0.2, base=50.0, kv_from=0)], width=D)
    w = O.random_weights(c, H_)
    for i in (0, 1):
        w[f"l{i}.mix.o"] = torch.eye(H_ * dv, dtype=torch.float64)
    cfg, params = from_risutar_state_dict(config_from_hf(c), w, dtype=dtype)
    h0 = O.bf16_exact(torch.randn(T, D, dtype=torch.float64))
    h1 = O.bf16_exact(torch.randn(T, D, dtype=torch.float64))
    kv = O.latent_kv(lay["mixer"], w, "l0.mix.", h0, eps)
    want0 = O.latent_attention(c["layers"][0]["mixer"], w, "l0.mix.", h0, eps, kv).numpy()
    want1 = O.latent_attention(c["layers"][1]["mixer"], w, "l1.mix.", h1, eps, kv).numpy()
    nblk = -(-T // bs)
    perm = np.random.default_rng(1).permutation(nblk + 3)[:nblk]
    cache = torch.zeros((nblk + 3) * bs, r + dr, dtype=dtype, device=device)
    a = 2e-4 if dtype == torch.float32 else 5e-2
    for cuts in ([T], [5, 1, 2, T - 8]):
        cache.zero_()
        got0, got1, at = [], [], 0
        for n in cuts:
            step = StepView(i32([0, n], device), n, i32(np.arange(at, at + n), device),
                            i32([perm[t // bs] * bs + t % bs for t in range(at, at + n)], device),
                            i32(perm[None], device), bs, None)
            for i, (hh, got) in enumerate(((h0, got0), (h1, got1))):
                spec = cfg.layer_specs[i]
                lp = {k[len(f"layers.{i}."):]: v.to(device) for k, v in params.items()
                      if k.startswith(f"layers.{i}.")}
                derive_constants(spec, lp, torch.device(device))
                y = latent_attention_mixer(spec, lp, dev_t(hh[at:at + n], device, dtype), step,
                                           (cache,), eps)
                got.append(y.float().cpu().numpy())
            at += n
        np.testing.assert_allclose(np.concatenate(got0), want0, atol=a, rtol=a)
        np.testing.assert_allclose(np.concatenate(got1), want1, atol=a, rtol=a)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("mlp", [moe(), moe(top=1), moe(experts=3, top=3), moe(shared=0),
                                 moe(ff=7, experts=9, top=4, shared=5)],
                         ids=["usual", "top1", "all_experts", "no_shared", "odd_sizes"])
def test_router_and_experts(device, dtype, mlp):
    """Biased logits, top-k by logit, weights renormalised among the k, exact-GELU experts,
    the always-on shared expert."""
    from distributed_llm_inferencing_amd.models.mixers import derive_constants, moe_ff
    D, T = 24, 33
    c = config([gla(mlp=mlp)], width=D)
    w = O.random_weights(c, 7)
    cfg, params = from_risutar_state_dict(config_from_hf(c), w, dtype=dtype)
    spec = cfg.layer_specs[0]
    lp = {k[len("layers.0."):]: v.to(device) for k, v in params.items() if k.startswith("layers.0.")}
    derive_constants(spec, lp, torch.device(device))
    h = O.bf16_exact(torch.randn(T, D, dtype=torch.float64))
    ids, wt = O.route(mlp, w, "l0.mlp.", h)
    tw, ti = H.logit_router(dev_t(h, device, dtype), lp["router"], lp["router_b"], spec.top)
    assert np.array_equal(ti.cpu().numpy(), ids.numpy())
    np.testing.assert_allclose(tw.cpu().numpy(), wt.numpy(), atol=1e-5)
    got = moe_ff(spec, lp, dev_t(h, device, dtype)).cpu().numpy()
    a = 1e-4 if dtype == torch.float32 else 4e-2
    np.testing.assert_allclose(got, O.moe_ff(mlp, w, "l0.mlp.", h).numpy(), atol=a, rtol=a)


# ------------------------------------------------------------------ whole models
@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("lay", [gla(mlp=None), gla(mlp=dense()), gla(mlp=moe()),
                                 latent(mlp=None), latent(mlp=dense()), latent(mlp=moe(top=1))],
                         ids=["gla", "gla_dense", "gla_moe", "latent", "latent_dense", "latent_moe"])
def test_one_layer_models(lay, device, dtype):
    c = config([lay])
    w = O.random_weights(c, 11)
    t = toks(21, c["vocab"])
    eng = engine(c, w, device, dtype)
    close(replay(eng, t, [21]), ref(t, c, w), dtype, "one layer")


@pytest.mark.parametrize("device,dtype", CASES)
def test_layer_trace_matches_the_oracle(device, dtype):
    w = O.random_weights(FULL, 2)
    t = toks(14, FULL["vocab"], 4)
    trace = []
    O.forward(FULL, w, t, trace)
    eng = engine(FULL, w, device, dtype)
    eng.model.layer_trace = []
    replay(eng, t, [14])
    # a routing close call in bf16 moves a whole row: compare where it does not
    for i, (got, want) in enumerate(zip(eng.model.layer_trace, trace)):
        d = np.abs(got.cpu().numpy() - want.numpy()).max(-1)
        lim = 1e-3 if dtype == torch.float32 else 0.25
        assert np.median(d) < lim and (dtype == torch.bfloat16 or d.max() < lim), f"layer {i}"


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("routed", [True, False])
def test_prefill_equals_decode_equals_portions(device, dtype, routed):
    FULL = globals()["FULL"] if routed else without_routing(globals()["FULL"])
    w = O.random_weights(FULL, 1)
    t = toks(45, FULL["vocab"], 3)
    want = ref(t, FULL, w)
    for cuts in ([45], [1] * 45, [2] * 22 + [1], [7, 2, 9, 1, 1, 3, 16, 2, 4],
                 [30] + [1] * 15, [8, 8, 8, 8, 8, 5]):
        eng = engine(FULL, w, device, dtype)
        close(replay(eng, t, cuts), want, dtype, f"cuts {cuts[:4]}")


@pytest.mark.parametrize("device,dtype", CASES)
def test_mixed_batches_and_reuse_of_pages_and_slots(device, dtype):
    """Unequal requests in one step (portions beside single tokens) against each alone, in a
    pool so small that pages and state slots are freed and taken again."""
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
    """Sizes that differ where a usual model makes them equal, and values of 1."""
    cs = [
        config([latent(heads=1, dim=4, rot=2, vdim=3, kv_rank=5, q_rank=9, mlp=moe(ff=5, experts=2, top=2, shared=3)),
                gla(heads=1, dim=3, vdim=5, tau=1.0, mlp=dense(7))],
               width=20, vocab=31, alpha=1.0, bigram=(7, 1, 1), side=1),
        config([gla(heads=5, dim=4, vdim=2, tau=30.0, mlp=moe(experts=7, top=6)),
                latent(heads=5, dim=2, rot=6, vdim=7, kv_rank=3, q_rank=2, mlp=None),
                latent(heads=2, dim=6, rot=6, vdim=2, kv_rank=3, q_rank=11, kv_from=1, mlp=dense(9))],
               width=28, vocab=40, alpha=0.5, bigram=None, side=0),
        config([latent(mlp=dense()), gla(mlp=None)], width=64, vocab=50, eps=1e-2, alpha=7.0,
               bigram=(1, 3, 2), side=13),
        # nothing a multiple of 4: no kernel may take a vector path it is not aligned for
        config([latent(heads=3, dim=5, rot=2, vdim=3, kv_rank=7, q_rank=5, mlp=moe(ff=5, experts=3, top=2, shared=7)),
                gla(heads=3, dim=5, vdim=7, tau=3.0, mlp=dense(9)),
                latent(heads=1, dim=3, rot=2, vdim=9, kv_rank=7, q_rank=3, kv_from=0, mlp=None)],
               width=30, vocab=33, alpha=1.5, bigram=(5, 2, 9), side=3),
    ]
    for n, c in enumerate(cs):
        w = O.random_weights(c, 20 + n, decay_rank=1 + 3 * n)
        t = toks(19, c["vocab"], n)
        want = ref(t, c, w)
        eng = engine(c, w, device, dtype, block_size=4)
        close(replay(eng, t, [19]), want, dtype, f"config {n} whole")
        close(replay(eng, t, [3, 1, 2, 13]), want, dtype, f"config {n} portions")


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("far", [1, 7, 8, 9, 250])
def test_far_keys_and_page_borders_stand_out(far, device, dtype):
    """One key, ``far`` positions back (around a page border, or hundreds away), is made to
    dominate the last query's scores: its token's embedding is solved so that its cached latent
    points along the last token's absorbed query. The position's logits then depend on that
    one key being found."""
    c = config([latent(heads=2, dim=8, rot=4, vdim=6, kv_rank=10, q_rank=8, scale=1.5, mlp=None)],
               width=24, vocab=64, bigram=None, side=0)
    w = O.random_weights(c, 9)
    w["l0.mix.uk"] = w["l0.mix.uk"] * 3.0
    w["l0.mix.uv"] = w["l0.mix.uv"] * 3.0
    m, eps = c["layers"][0]["mixer"], c["norm"]["eps"]
    cq = O.rms_div(w["embed"][62] @ w["l0.mix.dq"].T, eps) * w["l0.mix.dq.norm"]
    q0 = (cq @ w["l0.mix.uq"].T).reshape(2, 12)[0, :8]
    qa = w["l0.mix.uk"].reshape(2, 8, 10)[0].T @ q0          # the query as the latent sees it
    h = torch.linalg.pinv(w["l0.mix.dkv"][:10]) @ (qa / w["l0.mix.dkv.norm"])
    w["embed"][61] = O.bf16_exact(h / h.pow(2).mean().sqrt())
    n = far + 6
    t = toks(n, 60, far)
    t[n - 1 - far] = 61                                   # a token used nowhere else
    t[n - 1] = 62
    want = ref(t, c, w)
    # the attention really concentrates: removing the far token changes the last logits
    t2 = list(t)
    t2[n - 1 - far] = 60
    moved = np.abs(O.forward(c, w, t2).numpy()[-1] - want.logits[-1]).max()
    assert moved > 0.05
    eng = engine(c, w, device, dtype)
    close(replay(eng, t, [n]), want, dtype, "whole")
    close(replay(eng, t, [n - 3, 1, 1, 1]), want, dtype, "decoded")


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
    # 150 steps of six layers: bf16 rounding of the activations adds up along the states
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
    lookahead on the GPU) against greedy decoding with the oracle."""
    c = copy.deepcopy(FULL)
    w = O.random_weights(c, 12)
    w["head"] = w["head"] * 4.0                          # clear winners
    prompts = [toks(n, c["vocab"], s) for n, s in ((11, 1), (3, 2), (25, 3))]
    eng = engine(c, w, device, dtype, graphs=graphs, lookahead=graphs, max_prefill_tokens=16)
    outs = eng.generate(prompts, SamplingParams(max_new_tokens=8, do_sample=False, ignore_eos=True))
    for p, o in zip(prompts, outs):
        seq = list(p)
        assert len(o.output_ids) == 8
        for tok in o.output_ids:
            lg = O.forward(c, w, seq).numpy()[-1]
            best = int(lg.argmax())
            if tok != best:              # a near tie may fall the other way in reduced precision
                assert lg[best] - lg[tok] < (1e-3 if dtype == torch.float32 else 0.3)
            seq.append(tok)


def test_config_reader_reads_every_size():
    cfg = config_from_hf(FULL)
    assert cfg.arch == "risutar" and cfg.is_hybrid and cfg.has_state
    assert (cfg.hidden_size, cfg.vocab_size, cfg.postln_alpha, cfg.norm_eps) == (40, 80, 2.5, 2e-6)
    assert cfg.bigram == (53, 11, 3) and cfg.side_dim == 6
    s = cfg.layer_specs
    assert [x.kind for x in s] == ["gla", "latent_attention", "latent_attention", "gla",
                                   "latent_attention", "gla"]
    assert (s[0].heads, s[0].dim, s[0].vdim, s[0].tau, s[0].ff_kind, s[0].ff) == (2, 8, 12, 6.0, "gated_silu", 40)
    assert (s[1].kv_rank, s[1].q_rank, s[1].rot_dim, s[1].rot_dims, s[1].rot_base, s[1].scale) == (12, 14, 4, 4, 100.0, 0.3)
    assert s[1].rot_half and s[1].head_gate and s[1].kv_from == -1 and s[2].kv_from == 1
    assert (s[2].router, s[2].expert_act, s[2].experts, s[2].top, s[2].shared_ff) == ("logit_topk", "gelu_erf", 5, 3, 0)
    assert s[4].ff == 0 and cfg.cache_row_width(2) == 0 and cfg.cache_row_width(1) == 16
    cfg2, params = from_risutar_state_dict(cfg, O.random_weights(FULL, 0, decay_rank=3))
    assert cfg2.layer_specs[0].decay_rank == 3 and params["layers.0.w_a2"].shape == (16, 3)
    bad = copy.deepcopy(FULL)
    bad["layers"][2]["mixer"]["kv_from"] = 0
    with pytest.raises(ValueError):
        config_from_hf(bad)


def test_registry_model_random_init_generates():
    eng = LLMEngine("risutar-tiny", device="cpu", dtype=torch.float32, max_batch=2,
                    max_model_len=64, block_size=8, num_blocks=24, use_graphs=False)
    outs = eng.generate([[1, 2, 3], [4, 5, 6, 7, 8]], SamplingParams(max_new_tokens=4, do_sample=False,
                                                                    ignore_eos=True))
    assert all(len(o.output_ids) == 4 for o in outs)


@pytest.mark.gpu
@pytest.mark.parametrize("width,lay,n", [
    (128, gla(heads=2, dim=16, vdim=32, mlp=moe(ff=64, experts=4, top=2, shared=128)), 70),
    (64, latent(heads=2, dim=16, rot=16, vdim=16, kv_rank=16, q_rank=32, mlp=moe(ff=128, experts=3, top=1, shared=0)), 33),
    (128, gla(heads=1, dim=32, vdim=64, mlp=dense(192)), 41),
    (192, latent(heads=4, dim=32, rot=32, vdim=16, kv_rank=64, q_rank=64, mlp=moe(ff=64, experts=8, top=3, shared=64)), 300)],
    ids=["moe_shared", "moe_top1", "dense", "moe_matrix_core_heads"])
def test_tuned_feed_forward_layout_at_several_sizes(gpu, width, lay, n):
    """Sizes the tuned GEMM tiles take: the activations run as GEMM epilogues (exact GELU for
    the ungated experts and the shared one, SiLU * up over the interleaved dense weight) and the
    experts as grouped GEMMs; whole prompts, portions and single tokens."""
    c = config([lay, lay], width=width, vocab=96)
    w = O.random_weights(c, width + n)
    t = toks(n, 96, n)
    want = ref(t, c, w)
    eng = engine(c, w, "cuda", torch.bfloat16, max_tokens=640)
    assert "ff_tuned" in eng.model.layers[0]
    close(replay(eng, t, [n]), want, torch.bfloat16, "whole")
    close(replay(eng, t, [n - 9, 2, 1, 1, 5]), want, torch.bfloat16, "portions")


@pytest.mark.gpu
def test_exact_gelu_gemm_epilogue(gpu):
    from distributed_llm_inferencing_amd import ops
    g = torch.Generator().manual_seed(0)
    for M in (3, 40, 700):
        x = (torch.randn(M, 128, generator=g) * 1.5).to(torch.bfloat16).cuda()
        wt = (torch.randn(192, 128, generator=g) / 8).to(torch.bfloat16).cuda()
        got = ops.linear(x, wt, epi="gelu_erf").float().cpu()
        want = torch.nn.functional.gelu(x.double().cpu() @ wt.double().cpu().T)
        np.testing.assert_allclose(got.numpy(), want.numpy(), atol=2e-2, rtol=2e-2)
