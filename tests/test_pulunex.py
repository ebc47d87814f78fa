"""Pulunex against the plain float64 oracle in ``pulunex_oracle.py``.

Every test builds its own small configuration and random weights, runs the framework (config
reader, weight conversion, engine, scheduler, block manager, state slots, runner, model, ops)
and compares with the oracle's whole-sequence functions. CPU cases run the PyTorch reference
ops in fp32; GPU cases run the HIP kernels in bf16 and fp32.
"""
import copy

import numpy as np
import pytest
import torch

import pulunex_oracle as O
from distributed_llm_inferencing_amd.engine import SamplingParams
from distributed_llm_inferencing_amd.engine.llm_engine import LLMEngine
from distributed_llm_inferencing_amd.models.hf import config_from_hf
from distributed_llm_inferencing_amd.models.weights import from_pulunex_state_dict
from distributed_llm_inferencing_amd.ops import hybrid as H

CASES = [("cpu", torch.float32),
         pytest.param("cuda", torch.float32, marks=pytest.mark.gpu),
         pytest.param("cuda", torch.bfloat16, marks=pytest.mark.gpu)]


def dense(ff=40):
    return {"kind": "dense", "ff": ff}


def moe(ff=12, experts=5, identity=2, top=2, shared=20):
    m = {"kind": "moe", "expert": {"ff": ff},
         "router": {"experts": experts, "identity": identity, "top": top}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def layer(heads=4, kv=2, dim=8, vdim=12, size=7, scale=0.4, mlp=None, kv_from=None):
    mx = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale}
    if size:
        mx["mask"] = {"size": size}
    if kv_from is not None:
        mx["kv_from"] = kv_from
    return {"type": "attention", "mixer": mx, "mlp": mlp}


def config(layers, width=40, vocab=80, positions=200, eps=1e-5, emb=3.0, logit=0.7):
    return {"architecture": "Pulunex", "width": width, "vocab": vocab, "max_positions": positions,
            "embedding": {"scale": emb}, "logit_scale": logit, "norm": {"eps": eps},
            "layers": layers}


FULL = config([layer(mlp=dense()), layer(mlp=moe()), layer(size=5, mlp=moe(top=3, shared=0)),
               layer(kv_from=1, mlp=moe(identity=0)), layer(size=5, kv_from=2, mlp=None),
               layer(heads=2, kv=1, dim=16, vdim=4, size=11, mlp=dense(24))])


def engine(c, w, device, dtype, max_tokens=512, live=4, block_size=8, **kw):
    cfg = config_from_hf(c)
    sd = {k: torch.tensor(v) for k, v in w.items()}
    params = from_pulunex_state_dict(cfg, sd, dtype=dtype)
    return LLMEngine(cfg, device=device, dtype=dtype, params=params, max_batch=live,
                     max_model_len=1 << 20, block_size=block_size,
                     num_blocks=-(-max_tokens // block_size) + live,
                     use_graphs=kw.pop("graphs", False), lookahead=kw.pop("lookahead", False), **kw)


def tol(dtype):
    return 2e-4 if dtype == torch.float32 else 6e-2


class Ref:
    """Oracle logits of a sequence with each position's closest routing decision."""

    def __init__(self, logits, margins):
        self.logits, self.margins = logits, np.asarray(margins)

    def __getitem__(self, k):
        return Ref(self.logits[k], self.margins[k])


def ref(tokens, c, w):
    m = []
    return Ref(O.forward(tokens, c, w, margins=m), m)


def close(got, want, dtype, what=""):
    """Row error as a logit comparison sees it: mean removed, relative to the spread. In bf16
    a position whose routing was a close call (the rounded input may choose another expert)
    is held to a looser bound; every other position, and fp32 everywhere, to the strict one."""
    loose = None
    if isinstance(want, Ref):
        if dtype == torch.bfloat16:
            loose = want.margins < 0.005
        want = want.logits
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    err = np.sqrt((d ** 2).mean(-1)) / want.std()
    if loose is not None and loose.any():
        assert err[loose].max() < 8 * tol(dtype), what
        err = err[~loose]
    assert err.max() < tol(dtype), f"{what}: error {err.max():.3g} at row {int(err.argmax())}"


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
    return torch.tensor(np.asarray(a), dtype=dtype, device=device)


# ------------------------------------------------------------------ single mechanisms (ops)
@pytest.mark.parametrize("device,dtype", CASES)
def test_token_shift_op_and_its_state(device, dtype):
    """Rows mixed with their predecessors; the predecessor of a portion's first row comes from
    the slot, position 0 starts from zeros whatever the slot held, slots are independent."""
    rng = np.random.default_rng(0)
    D = 24
    hs = rng.standard_normal((9, D))
    other = rng.standard_normal((4, D))
    mu = rng.random(D)
    want = O.token_shift(hs, mu)
    want_o = O.token_shift(other, mu)
    state = torch.full((3, D), 7.0, device=device)          # stale contents of reused slots
    mu_t = dev_t(mu, device, dtype)

    def run(rows, slots, lens, first_pos):
        cu = torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int32, device=device)
        pos = np.concatenate([np.arange(p, p + n) for p, n in zip(first_pos, lens)])
        return H.token_shift(dev_t(rows, device), mu_t, state,
                             torch.tensor(slots, dtype=torch.int32, device=device), cu,
                             max(lens), torch.tensor(pos, dtype=torch.int32, device=device)
                             ).float().cpu().numpy()

    a = 1e-6 if dtype == torch.float32 else 2e-2
    got = run(np.vstack([hs[:5], other[:1]]), [2, 0], [5, 1], [0, 0])
    np.testing.assert_allclose(got[:5], want[:5], atol=a)
    np.testing.assert_allclose(got[5:], want_o[:1], atol=a)
    got = run(np.vstack([other[1:4], hs[5:6]]), [0, 2], [3, 1], [1, 5])
    np.testing.assert_allclose(got[:3], want_o[1:4], atol=a)
    np.testing.assert_allclose(got[3:], want[5:6], atol=a)
    got = run(hs[6:9], [2], [3], [6])
    np.testing.assert_allclose(got, want[6:9], atol=a)
    np.testing.assert_allclose(state[2].cpu().numpy(), hs[8], atol=1e-6)
    np.testing.assert_allclose(state[1].cpu().numpy(), 7.0)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("H_,G,d,dv,size", [(4, 2, 8, 12, 7), (6, 1, 4, 4, 3), (3, 3, 16, 5, 1),
                                            (2, 2, 32, 32, 64)])
def test_block_attention_with_mixed_scores(device, dtype, H_, G, d, dv, size):
    """talk_prepare + window_attention through a paged cache against the oracle's attention:
    biases, unit-RMS q / k, mixing before the softmax, grouped values, block mask."""
    rng = np.random.default_rng(H_ * 10 + G)
    T, D, eps, bs = 23, 20, 1e-5, 4
    mx = {"heads": H_, "kv_heads": G, "dim": d, "vdim": dv, "scale": 0.6, "mask": {"size": size}}
    w = {"m.q": rng.standard_normal((H_ * d, D)), "m.q.b": rng.standard_normal(H_ * d),
         "m.k": rng.standard_normal((G * d, D)), "m.k.b": rng.standard_normal(G * d),
         "m.v": rng.standard_normal((G * dv, D)), "m.v.b": rng.standard_normal(G * dv),
         "m.talk": np.eye(H_) + 0.4 * rng.standard_normal((H_, H_)), "m.o": np.eye(H_ * dv)}
    us = rng.standard_normal((T, D))
    want = O.block_attention(us, mx, w, "m.", eps, O.keys_values(us, mx, w, "m.", eps))
    proj = np.concatenate([us @ w["m.q"].T, us @ w["m.k"].T, us @ w["m.v"].T], 1)
    bias = np.concatenate([w["m.q.b"], w["m.k.b"], w["m.v.b"]])
    nblk = -(-T // bs)
    perm = rng.permutation(nblk + 3)[:nblk]                  # pages in any order
    kc = torch.zeros((nblk + 3) * bs, G * d, dtype=dtype, device=device)
    vc = torch.zeros((nblk + 3) * bs, G * dv, dtype=dtype, device=device)
    slots = torch.tensor([perm[t // bs] * bs + t % bs for t in range(T)], dtype=torch.int32,
                         device=device)
    q = H.talk_prepare(dev_t(proj, device), dev_t(bias, device, dtype),
                       dev_t(w["m.talk"], device), eps, H_, G, d, dv, kc, vc, slots, True)
    o = H.window_attention(q, kc, vc, G * d, dv, H_, G,
                           torch.tensor([0, T], dtype=torch.int32, device=device), T,
                           torch.arange(T, dtype=torch.int32, device=device),
                           torch.tensor(perm[None], dtype=torch.int32, device=device), bs,
                           1 << 30, 0.6, chunk=size, k_groups=1)
    a = 1e-4 if dtype == torch.float32 else 6e-2
    np.testing.assert_allclose(o.float().cpu().numpy(), want, atol=a, rtol=a)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("mlp", [moe(), moe(identity=0, top=1), moe(experts=3, identity=5, top=4),
                                 moe(shared=0), moe(ff=7, experts=9, top=3, shared=5)],
                         ids=["usual", "top1", "mostly_identity", "no_shared", "odd_sizes"])
def test_router_and_experts(device, dtype, mlp):
    """Softmax over all experts, choice with the correction, weights without it and not
    renormalised, identity experts, the shared expert's gate."""
    rng = np.random.default_rng(5)
    D, T = 24, 17
    c = config([layer(mlp=mlp)], width=D)
    w = O.random_weights(c, seed=4)
    cfg = config_from_hf(c)
    p = from_pulunex_state_dict(cfg, {k: torch.tensor(v) for k, v in w.items()}, dtype=dtype)
    lp = {k[len("layers.0."):]: v.to(device) for k, v in p.items() if k.startswith("layers.0.")}
    h = torch.tensor(rng.standard_normal((T, D)), dtype=dtype, device=device)
    hq = h.float().cpu().numpy().astype(np.float64)
    r = mlp["router"]
    ng = 1 if mlp.get("shared") else 0
    tw, ti, gates = H.score_router(h, lp["router"], lp["correction"].float(), r["top"], ng)
    for t in range(T):
        s = O.softmax(w["l0.mlp.router"] @ hq[t])
        ch = s + w["l0.mlp.correction"]
        picked = sorted(range(len(s)), key=lambda e: (-ch[e], e))[:r["top"]]
        gap = np.sort(ch)[::-1]
        if dtype == torch.float32 or gap[r["top"] - 1] - gap[r["top"]] > 0.02:
            assert sorted(ti[t].tolist()) == sorted(picked), t
            for j, e in enumerate(ti[t].tolist()):
                assert abs(float(tw[t, j]) - s[e]) < (1e-5 if dtype == torch.float32 else 2e-2)
    shared = (lp["ws_gu"], lp["ws_down"], gates) if ng else None
    got = H.moe_experts_f32(h, lp["w_gu"], lp["w_down"], tw, ti, shared).float().cpu().numpy()
    want = np.stack([O.routed_ff(hq[t], mlp, w, "l0.mlp.") for t in range(T)])
    if dtype == torch.float32:
        np.testing.assert_allclose(got, want, atol=2e-4, rtol=2e-4)
    else:
        assert np.abs(got - want).max() < 0.08 * np.abs(want).max()


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("lay", [layer(mlp=None), layer(mlp=dense()), layer(mlp=moe()),
                                 layer(heads=6, kv=1, dim=4, vdim=4, size=0, mlp=None)],
                         ids=["attention", "dense_ff", "routed_ff", "no_mask"])
def test_one_layer_models(lay, device, dtype):
    c = config([lay])
    w = O.random_weights(c, seed=3)
    t = toks(21, c["vocab"])
    close(replay(engine(c, w, device, dtype), t, [21]), ref(t, c, w), dtype)


# ------------------------------------------------------------------ schedules
@pytest.mark.parametrize("device,dtype", CASES)
def test_prefill_equals_decode_equals_portions(device, dtype):
    w = O.random_weights(FULL, seed=5)
    t = toks(45, FULL["vocab"], 2)
    want = ref(t, FULL, w)
    eng = engine(FULL, w, device, dtype)
    close(replay(eng, t, [45]), want, dtype, "whole")
    close(replay(eng, t, [1] * 45), want, dtype, "token by token")
    close(replay(eng, t, [20] + [1] * 25), want, dtype, "prefill + decode")
    for cuts in ([2] * 22 + [1], [3, 7, 2, 16, 2, 2, 13], [8, 8, 8, 8, 8, 5], [44, 1]):
        close(replay(eng, t, cuts), want, dtype, f"portions {cuts[:4]}")
    assert eng.bm.num_free == eng.bm.num_blocks and eng.state_slots.num_free == 4


@pytest.mark.parametrize("device,dtype", CASES)
def test_mixed_batches_and_reuse_of_pages_and_slots(device, dtype):
    """Unequal requests side by side (portions beside single tokens), more requests than
    state slots over time, a pool too small for all of them at once."""
    w = O.random_weights(FULL, seed=6)
    seqs = {f"r{i}": toks(n, FULL["vocab"], 10 + i) for i, n in enumerate((37, 5, 22, 1, 30, 18, 9))}
    want = {k: ref(v, FULL, w) for k, v in seqs.items()}
    eng = engine(FULL, w, device, dtype, max_tokens=128, live=3)
    got = {k: [] for k in seqs}
    at = {k: 0 for k in seqs}
    waiting, live = list(seqs), []
    rng = np.random.default_rng(0)
    step = 0
    while waiting or live:
        while waiting and len(live) < 3:
            live.append(waiting.pop(0))
        entries, wants, end = [], [], []
        for k in live:
            if step % 3 == 2 and k == live[0] and len(live) > 1:
                continue                                   # a request may sit a step out
            n = min(len(seqs[k]) - at[k], int(rng.choice([1, 1, 2, 5, 11])))
            entries.append((k, seqs[k][at[k]:at[k] + n]))
            wants.append(list(range(n)))
            at[k] += n
            if at[k] == len(seqs[k]):
                end.append(k)
        lg = eng.replay_step(entries, wants, end).float().cpu().numpy()
        o = 0
        for (k, part) in entries:
            got[k].append(lg[o:o + len(part)])
            o += len(part)
        live = [k for k in live if k not in end]
        step += 1
    for k in seqs:
        close(np.concatenate(got[k]), want[k], dtype, k)
    assert eng.bm.num_free == eng.bm.num_blocks and eng.state_slots.num_free == 3


@pytest.mark.parametrize("device,dtype", CASES)
def test_other_sizes_and_degenerate_values(device, dtype):
    """Values a usual configuration makes equal or 1: one kv head, as many kv heads as heads,
    one head, blocks of one position, blocks longer than the sequence, vdim != dim, top 1,
    no identity experts, scales of 1, a chain of layers on one donor's cache, two donors."""
    variants = [
        config([layer(heads=1, kv=1, dim=8, vdim=8, size=1, mlp=dense(8))], emb=1.0, logit=1.0),
        config([layer(heads=3, kv=3, dim=4, vdim=20, size=1000, mlp=moe(top=1, identity=0)),
                layer(heads=3, kv=3, dim=4, vdim=20, size=2, kv_from=0, mlp=None),
                layer(heads=3, kv=3, dim=4, vdim=20, size=3, kv_from=0, mlp=dense(16))],
               width=24, vocab=33, emb=0.5, logit=3.0),
        config([layer(mlp=None), layer(heads=8, kv=4, dim=4, vdim=2, size=6, mlp=moe(experts=2, identity=1, top=3)),
                layer(kv_from=0, mlp=moe(ff=40, shared=8)),
                layer(heads=8, kv=4, dim=4, vdim=2, size=9, kv_from=1, mlp=None)],
               width=32, eps=1e-3),
    ]
    for i, c in enumerate(variants):
        w = O.random_weights(c, seed=20 + i)
        t = toks(19, c["vocab"], i)
        eng = engine(c, w, device, dtype)
        want = ref(t, c, w)
        close(replay(eng, t, [19]), want, dtype, f"variant {i} whole")
        close(replay(eng, t, [4, 1, 1, 6, 2, 5]), want, dtype, f"variant {i} portions")


# ------------------------------------------------------------------ edges made visible
def _echo_model(size, block):
    """One attention layer whose query for token 1 matches the key of token 2 and nothing else:
    no position vectors, no shift, no biases, keys = minus the queries' projection, opposite
    embeddings for the two tokens, a large score scale. Whether a far token 2 is visible then
    decides the probe's logits."""
    c = config([layer(heads=2, kv=1, dim=16, vdim=16, size=size, scale=1.5, mlp=None)],
               width=32, vocab=40, positions=700)
    w = O.random_weights(c, seed=9)
    w["pos"][:] = 0.0
    w["l0.shift"][:] = 0.0
    w["l0.mix.q.b"][:] = 0.0
    w["l0.mix.k.b"][:] = 0.0
    w["l0.mix.q"] = -np.concatenate([w["l0.mix.k"], w["l0.mix.k"]], 0)
    w["l0.mix.talk"] = np.eye(2)
    w["embed"][1] = -w["embed"][2]
    w["l0.mix.v"] *= 4.0
    return c, w


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("size", [8, 12, 333])
def test_block_edges_and_far_keys_stand_out(size, device, dtype):
    """The marked key at the first position of the probe's block (just inside), at the last
    position of the block before (just outside), far back inside a long block, and at page
    borders; the probe inside a prompt, as a prompt's cut, and decoded alone."""
    block = 8
    c, w = _echo_model(size, block)
    n = 2 * size + 5 if size < 100 else 340
    base = [3 + (i % 30) for i in range(n)]
    probes = [n - 1, (n - 1) // size * size, size - 1, size, min(n - 1, size + block)]
    for probe in sorted(set(p for p in probes if 1 <= p < n)):
        first = probe // size * size
        for key in {first, first - 1, first + 1, probe - 1, (probe // block) * block,
                    (probe // block) * block - 1, 0}:
            if not 0 <= key < probe:
                continue
            t = list(base)
            t[key], t[probe] = 2, 1
            want = O.forward(t[:probe + 1], c, w)
            seen, hidden = want[probe], O.forward([3] * probe + [1], c, w)[probe]
            eng = engine(c, w, device, dtype, max_tokens=1024, block_size=block)
            for cuts in ([probe + 1], [probe, 1], [key + 1, probe - key - 1, 1] if probe - key > 1 else [probe, 1]):
                got = replay(eng, t[:probe + 1], cuts)
                close(got[probe:], want[probe:probe + 1], dtype, f"size {size} probe {probe} key {key} {cuts}")
            if key >= first:             # the marked key must matter when it is visible
                assert np.abs(seen - hidden).max() > 0.1 * np.abs(seen).max()


@pytest.mark.parametrize("device,dtype", CASES)
def test_first_tokens_and_long_decode(device, dtype):
    c = config([layer(size=5, mlp=moe()), layer(size=16, kv_from=0, mlp=dense())])
    w = O.random_weights(c, seed=12)
    t = toks(70, c["vocab"], 4)
    want = ref(t, c, w)
    eng = engine(c, w, device, dtype)
    close(replay(eng, t, [1, 1, 2, 1] + [1] * 65), want, dtype, "from the first token on")
    close(replay(eng, t[:3], [3]), want[:3], dtype, "three tokens")
    close(replay(eng, t[:1], [1]), want[:1], dtype, "one token")
    # a request that is ended by a later step which brings no tokens at all
    lg = eng.replay_step([("z", t[:5])], [[4]], [])
    assert eng.replay_step([], [], ["z"]).shape[0] == 0
    close(lg.float().cpu().numpy(), want[4:5], dtype, "ended by an empty step")
    assert eng.bm.num_free == eng.bm.num_blocks and eng.state_slots.num_free == 4


# ------------------------------------------------------------------ generation entry point
@pytest.mark.parametrize("device,dtype,graphs", [
    ("cpu", torch.float32, False),
    pytest.param("cuda", torch.float32, False, marks=pytest.mark.gpu),
    pytest.param("cuda", torch.bfloat16, True, marks=pytest.mark.gpu)])
def test_greedy_generation_through_the_engine(device, dtype, graphs):
    """LLMEngine.generate (scheduler admission, chunked prefill, decode steps / captured
    graphs, sampler at temperature 0) against the oracle's argmax continuation; unequal prompts
    in one batch, more requests than slots."""
    w = O.random_weights(FULL, seed=7)
    prompts = [toks(n, FULL["vocab"], 30 + n) for n in (9, 1, 17, 4, 12)]
    new = 12
    eng = engine(FULL, w, device, dtype, max_tokens=512, live=3, graphs=graphs,
                 lookahead=graphs, max_prefill_tokens=16)
    outs = eng.generate(prompts, SamplingParams(max_new_tokens=new, do_sample=False,
                                                ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert len(o.output_ids) == new
        seq = list(p)
        for k, tok in enumerate(o.output_ids):
            lg = O.forward(seq, FULL, w)[-1]
            best = int(lg.argmax())
            if tok != best:
                # a near tie may flip in reduced precision; anything else is a fault
                gap = (lg[best] - lg[tok]) / lg.std()
                assert gap < (1e-3 if dtype == torch.float32 else 0.15), (k, tok, best, gap)
            seq.append(tok)
    assert eng.bm.num_free == eng.bm.num_blocks and eng.state_slots.num_free == 3


def test_config_reader_reads_every_size():
    c = copy.deepcopy(FULL)
    cfg = config_from_hf(c)
    assert cfg.is_hybrid and cfg.arch == "pulunex"
    assert (cfg.hidden_size, cfg.vocab_size, cfg.max_position) == (40, 80, 200)
    assert (cfg.embed_scale, cfg.logit_scale, cfg.norm_eps) == (3.0, 0.7, 1e-5)
    s = cfg.layer_specs
    assert (s[0].heads, s[0].kv_heads, s[0].dim, s[0].vdim, s[0].chunk, s[0].scale) == (4, 2, 8, 12, 7, 0.4)
    assert (s[0].ff_kind, s[0].ff) == ("gelu", 40)
    assert (s[1].ff_kind, s[1].ff, s[1].experts, s[1].identity, s[1].top, s[1].shared_ff) == (
        "moe", 12, 5, 2, 2, 20)
    assert s[2].top == 3 and s[2].shared_ff == 0 and s[3].identity == 0
    assert (s[3].kv_from, s[4].kv_from, s[4].ff, s[5].kv_from) == (1, 2, 0, -1)
    assert all(x.shift and x.has_state for x in s) and cfg.has_state
    assert cfg.cache_row_width(3) == 0 and cfg.cache_row_width(1) == 2 * (8 + 12)
    c["layers"][3]["mixer"]["kv_from"] = 4                   # a donor must come earlier
    with pytest.raises(ValueError):
        config_from_hf(c)
    c = copy.deepcopy(FULL)
    c["layers"][0]["mlp"]["kind"] = "maxout"
    with pytest.raises(ValueError):
        config_from_hf(c)


def test_registry_model_random_init_generates():
    eng = LLMEngine("pulunex-tiny", device="cpu", dtype=torch.float32, max_batch=2,
                    max_model_len=64, block_size=8, num_blocks=24, use_graphs=False)
    outs = eng.generate([[5, 6, 7], [9]], SamplingParams(max_new_tokens=5, do_sample=False,
                                                        ignore_eos=True))
    assert [len(o.output_ids) for o in outs] == [5, 5]


@pytest.mark.gpu
def test_model_on_matrix_core_sized_heads(gpu):
    """Head sizes the MFMA attention takes (multiples of 32 / 16) and feed-forward sizes the
    tuned GEMM tiles take (fused activation epilogues, grouped expert GEMMs); prompts long
    enough for several query tiles, blocks that end inside a tile."""
    c = config([layer(heads=4, kv=2, dim=32, vdim=48, size=40, mlp=moe(ff=64, shared=128)),
                layer(heads=4, kv=2, dim=32, vdim=48, size=19, kv_from=0, mlp=dense(64)),
                layer(heads=4, kv=2, dim=32, vdim=48, size=64, mlp=moe(ff=64, identity=0, shared=0))],
               width=64, vocab=96)
    w = O.random_weights(c, seed=31)
    t = toks(75, c["vocab"], 8)
    want = ref(t, c, w)
    eng = engine(c, w, "cuda", torch.bfloat16, block_size=16)
    assert all("ff_tuned" in lp for lp in eng.model.layers)
    close(replay(eng, t, [75]), want, torch.bfloat16, "whole")
    close(replay(eng, t, [33, 2, 17] + [1] * 23), want, torch.bfloat16, "portions + decode")


def _paged_case(lens, starts, H, Gk, G, dq, dv, block, seed):
    """Random queries of portions [start, start + len) per sequence over shuffled pages; key
    rows hold Gk heads of dq, value rows G heads of dv."""
    g = torch.Generator().manual_seed(seed)
    S = len(lens)
    nblk = [-(-(s + n) // block) for s, n in zip(starts, lens)]
    total = sum(nblk) + 3
    perm = torch.randperm(total, generator=g).tolist()
    tables = torch.zeros(S, max(nblk), dtype=torch.int32)
    at = 0
    for s in range(S):
        tables[s, :nblk[s]] = torch.tensor(perm[at:at + nblk[s]], dtype=torch.int32)
        at += nblk[s]
    kc = torch.randn(total * block, Gk * dq, generator=g).to(torch.bfloat16)
    vc = torch.randn(total * block, G * dv, generator=g).to(torch.bfloat16)
    q = torch.randn(sum(lens), H * dq, generator=g).to(torch.bfloat16)
    cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32)
    pos = torch.cat([torch.arange(s, s + n, dtype=torch.int32) for s, n in zip(starts, lens)])
    return q, kc, vc, cu, pos, tables


@pytest.mark.gpu
@pytest.mark.parametrize("H_,G,dq,dv,size", [(4, 2, 64, 48, 40), (6, 2, 128, 64, 96),
                                             (16, 4, 256, 128, 19), (3, 1, 32, 16, 1),
                                             (8, 8, 512, 32, 1000), (12, 3, 96, 80, 33),
                                             (24, 2, 64, 32, 50), (32, 8, 256, 128, 300)])
@pytest.mark.parametrize("decode", [False, True])
def test_matrix_core_attention_with_blocks_and_shared_key_rows(gpu, H_, G, dq, dv, size, decode):
    """The MFMA form with the block mask and one key head per cache row against the PyTorch
    reference: prompt portions whose query tiles straddle block edges, and decode rows with long
    contexts (key splits), at block edges, one after an edge, and at position 0."""
    from distributed_llm_inferencing_amd.ops import reference as R
    if decode:
        starts = [size - 1, size, 2 * size + size // 2, 0, 777, 5 * size - 1]
        lens = [1] * len(starts)
    else:
        lens, starts = [37, 1, 16, 50, 2], [0, 63, 48, 200, size]
    block = 16
    q, kc, vc, cu, pos, bt = _paged_case(lens, starts, H_, 1, G, dq, dv, block, seed=H_ + dq)
    scale = 1.0 / dq ** 0.5
    want = R.window_attention(q, kc, vc, dq, dv, H_, G, cu, pos, bt, block, 1 << 30, scale,
                              out_dtype=torch.float32, chunk=size, k_groups=1)
    d = lambda t: t.to(gpu)      # noqa: E731
    args = (d(q), d(kc), d(vc), dq, dv, H_, G, d(cu), max(lens), d(pos), d(bt), block, 1 << 30,
            scale)
    assert H.MFMA_ATTENTION
    got = H.window_attention(*args, chunk=size, k_groups=1).float().cpu()
    H.MFMA_ATTENTION = False
    try:
        scalar = H.window_attention(*args, chunk=size, k_groups=1).float().cpu()
    finally:
        H.MFMA_ATTENTION = True
    lim = 0.03 * want.abs().max().item() + 0.02
    assert (scalar - want).abs().max() < lim
    assert (got - want).abs().max() < lim
    assert size == 1 or not torch.equal(got, scalar)      # the two kernels really differ


@pytest.mark.gpu
@pytest.mark.parametrize("width,lay,n", [
    (192, layer(heads=6, kv=2, dim=32, vdim=32, size=24,
                mlp=moe(ff=128, experts=12, identity=4, top=2, shared=64)), 70),
    (320, layer(heads=5, kv=1, dim=64, vdim=16, size=9,
                mlp=moe(ff=64, experts=3, identity=1, top=3, shared=0)), 41),
    (128, layer(heads=2, kv=2, dim=16, vdim=16, size=50, mlp=dense(192)), 33),
    (64, layer(heads=2, kv=1, dim=32, vdim=32, size=4,
               mlp=moe(ff=64, experts=2, identity=1, top=2, shared=64)), 1100)],
    ids=["w192_12experts", "w320_top3", "w128_dense", "long_prompt_2experts"])
def test_tuned_feed_forward_layout_at_several_sizes(gpu, width, lay, n):
    """The feed-forwards on the tuned GEMM tiles (fused activation epilogues, grouped expert
    GEMMs incl. the prompt-sized form) at widths that are multiples of 64 but not powers of
    two, expert counts that are not, top 3, and single-row decode steps."""
    c = config([lay, copy.deepcopy(lay)], width=width, vocab=64, positions=1200)
    c["layers"][1]["mixer"]["kv_from"] = 0
    w = O.random_weights(c, seed=width)
    t = toks(n, c["vocab"], 5)
    want = ref(t, c, w)
    eng = engine(c, w, "cuda", torch.bfloat16, max_tokens=1280, block_size=16)
    assert all("ff_tuned" in lp for lp in eng.model.layers)
    close(replay(eng, t, [n]), want, torch.bfloat16, "whole")
    if n < 100:
        close(replay(eng, t, [n - 9, 2] + [1] * 7), want, torch.bfloat16, "portions + decode")
