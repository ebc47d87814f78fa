"""Buborax (hybrid design) against the plain float64 oracle in ``buborax_oracle.py``.

Every test builds its own small configuration and random weights, runs the framework (config
reader, weight conversion, engine, scheduler, block manager, state slots, runner, model, ops)
and compares logits with the oracle's whole-sequence forward. CPU cases run the PyTorch
reference ops in fp32; GPU cases run the HIP kernels in bf16 and fp32.
"""
import copy

import numpy as np
import pytest
import torch

import buborax_oracle as O
from distributed_llm_inferencing_amd.engine import SamplingParams
from distributed_llm_inferencing_amd.engine.llm_engine import LLMEngine
from distributed_llm_inferencing_amd.models.hf import config_from_hf
from distributed_llm_inferencing_amd.models.weights import from_buborax_state_dict

CASES = [("cpu", torch.float32),
         pytest.param("cuda", torch.float32, marks=pytest.mark.gpu),
         pytest.param("cuda", torch.bfloat16, marks=pytest.mark.gpu)]


def attn(heads=4, kv=2, dim=16, win=6, scale=0.3, ff=48):
    return {"type": "attention", "mlp": {"kind": "dense", "ff": ff} if ff else None,
            "mixer": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": dim,
                      "mask": {"size": win}, "scale": scale}}


def hgrn(heads=2, dim=8, vdim=12, ff=48):
    return {"type": "hgrn2", "mlp": {"kind": "dense", "ff": ff} if ff else None,
            "mixer": {"heads": heads, "dim": dim, "vdim": vdim}}


def latent(heads=3, dim=8, rot_dim=8, vdim=12, rank=16, win=7, scale=0.25, dims=4, base=300.0,
           ff=0):
    return {"type": "latent_attention", "mlp": {"kind": "dense", "ff": ff} if ff else None,
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim,
                      "kv_rank": rank, "mask": {"size": win}, "scale": scale,
                      "rot": {"base": base, "dims": dims}}}


def config(layers, width=48, vocab=96, loop=None, groups=3, mult=0.6, eps=1e-5):
    c = {"architecture": "Buborax", "width": width, "vocab": vocab, "layers": layers,
         "norm": {"eps": eps, "groups": groups}, "residual_mult": mult}
    if loop:
        c["loop"] = dict(zip(("start", "stop", "times"), loop))
    return c


FULL = config([attn(), hgrn(), latent(), hgrn(heads=3, dim=16, vdim=8, ff=0), attn(kv=4, win=9)],
              loop=(1, 4, 2))


def engine(c, w, device, dtype, max_tokens=512, live=4, block_size=8, **kw):
    cfg = config_from_hf(c)
    sd = {k: torch.tensor(v) for k, v in w.items()}
    params = from_buborax_state_dict(cfg, sd, dtype=dtype)
    return LLMEngine(cfg, device=device, dtype=dtype, params=params, max_batch=live,
                     max_model_len=1 << 20, block_size=block_size,
                     num_blocks=-(-max_tokens // block_size) + live, use_graphs=kw.pop("graphs", False),
                     lookahead=kw.pop("lookahead", False), **kw)


def tol(dtype):
    return 2e-4 if dtype == torch.float32 else 6e-2


def close(got, want, dtype, what=""):
    """Row error the way a logit comparison should see it: mean removed, relative to the
    oracle logits' spread."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    err = np.sqrt((d ** 2).mean(-1)) / want.std()
    assert err.max() < tol(dtype), f"{what}: error {err.max():.3g} at row {int(err.argmax())}"


def replay(eng, tokens, cuts, rid="a", want_all=True):
    """Feed ``tokens`` in portions ``cuts``; returns logits of every position."""
    out, at = [], 0
    for n in cuts:
        part = tokens[at:at + n]
        last = at + n == len(tokens)
        lg = eng.replay_step([(rid, part)], [list(range(n))], [rid] if last else [])
        out.append(lg.float().cpu().numpy())
        at += n
    assert at == len(tokens)
    return np.concatenate(out)


def toks(n, vocab, seed=1):
    return np.random.default_rng(seed).integers(0, vocab, n).tolist()


# ------------------------------------------------------------------ single mechanisms
@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("layer", [attn(ff=0), attn(heads=6, kv=1, dim=8, win=3, ff=0),
                                   hgrn(ff=0), hgrn(heads=1, dim=24, vdim=5, ff=0),
                                   hgrn(heads=2, dim=64, vdim=20, ff=0),
                                   hgrn(heads=1, dim=128, vdim=72, ff=0),
                                   latent(), latent(heads=1, dim=4, rot_dim=6, vdim=3, rank=5,
                                                    win=4, dims=6),
                                   attn(heads=2, kv=2, dim=8, win=50, ff=40)],
                         ids=["attn", "attn_mqa", "hgrn2", "hgrn2_1head", "hgrn2_d64", "hgrn2_d128",
                              "latent", "latent_odd",
                              "ff"])
def test_mechanism_alone(layer, device, dtype):
    c = config([layer], groups=1, mult=1.0)
    w = O.random_weights(c, seed=3)
    t = toks(21, c["vocab"])
    eng = engine(c, w, device, dtype)
    close(replay(eng, t, [21]), O.forward(c, w, t), dtype, layer["type"])


@pytest.mark.parametrize("device,dtype", CASES)
def test_group_norm_and_gated_ff_ops(device, dtype):
    from distributed_llm_inferencing_amd.ops import hybrid as H
    g = np.random.default_rng(0)
    x = g.standard_normal((5, 60))
    y = g.standard_normal((5, 60))
    wn = 1 + 0.1 * g.standard_normal(60)
    xt = torch.tensor(x, dtype=torch.float32, device=device)
    h = H.resadd_groupnorm(xt, torch.tensor(y, dtype=torch.float32, device=device),
                           torch.tensor(wn, device=device).to(dtype), 4, 1e-5, mult=0.5)
    wn_r = torch.tensor(wn).to(dtype).double().numpy()
    want = np.stack([O.group_norm(r, wn_r, 4, 1e-5) for r in x + 0.5 * y])
    assert np.abs(xt.cpu().numpy() - (x + 0.5 * y)).max() < 1e-5
    assert np.abs(h.float().cpu().numpy() - want).max() < (1e-5 if dtype == torch.float32 else 3e-2)
    gu = g.standard_normal((5, 2 * 28))
    act = H.gelu_mul(torch.tensor(gu, dtype=torch.float32, device=device), 28, dtype)
    want = O.gelu_tanh(gu[:, :28]) * gu[:, 28:]
    assert np.abs(act.float().cpu().numpy() - want).max() < (1e-5 if dtype == torch.float32 else 3e-2)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("shape", [(7, 33, 50), (70, 130, 96), (3, 64, 128), (129, 20, 8),
                                   (70, 33, 128), (5, 509, 64), (300, 81, 192), (1, 7, 256)])
def test_linear_any_shapes(shape, device, dtype):
    from distributed_llm_inferencing_amd.ops import hybrid as H
    M, N, K = shape
    g = torch.Generator().manual_seed(M)
    x = torch.randn(M, K, generator=g).to(dtype)
    w = torch.randn(N, K, generator=g).to(dtype)
    y = H.linear_any(x.to(device), w.to(device))
    want = x.double() @ w.double().t()
    assert y.dtype == torch.float32
    assert (y.cpu().double() - want).abs().max() < 1e-3 * K ** 0.5
    xh = torch.randn(M, 3, K, generator=g).to(dtype)
    wh = torch.randn(3, N, K, generator=g).to(dtype)
    out = torch.zeros(M, 3, N + 5, dtype=dtype, device=device)
    H.head_linear(xh.to(device), wh.to(device), out)
    want = torch.einsum("thk,hnk->thn", xh.double(), wh.double())
    lim = 1e-3 * K ** 0.5 if dtype == torch.float32 else 0.02 * K ** 0.5 + 0.05
    assert (out[:, :, :N].cpu().double() - want).abs().max() < lim
    assert float(out[:, :, N:].abs().max()) == 0.0


# ------------------------------------------------------------------ whole model, schedules
@pytest.mark.parametrize("device,dtype", CASES)
def test_prefill_equals_decode_equals_portions(device, dtype):
    w = O.random_weights(FULL, seed=5)
    t = toks(45, FULL["vocab"], 2)
    want = O.forward(FULL, w, t)
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
    want = {k: O.forward(FULL, w, v) for k, v in seqs.items()}
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
            left = len(seqs[k]) - at[k]
            n = min(left, int(rng.choice([1, 1, 2, 5, 11])))
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
    """Values the usual configuration makes equal or 1: one group, no loop, a loop run once,
    a loop over the first layer, no feed-forward anywhere, multiplier 1, rotation over all of
    the rotated part, heads == kv_heads == 1."""
    variants = [
        config([hgrn(), attn(heads=1, kv=1, dim=8, win=1)], groups=1, mult=1.0),
        config([latent(dims=8), hgrn(ff=0)], loop=(0, 1, 3), groups=2),
        config([attn(ff=0), latent(ff=32), hgrn()], loop=(0, 3, 1), width=40, vocab=50, groups=5),
        config([hgrn(heads=4, dim=4, vdim=4), attn(heads=8, kv=4, dim=4, win=1000)],
               loop=(1, 2, 2), width=32, groups=8, mult=0.3),
    ]
    for i, c in enumerate(variants):
        w = O.random_weights(c, seed=20 + i)
        t = toks(19, c["vocab"], i)
        eng = engine(c, w, device, dtype)
        want = O.forward(c, w, t)
        close(replay(eng, t, [19]), want, dtype, f"variant {i} whole")
        close(replay(eng, t, [4, 1, 1, 6, 2, 5]), want, dtype, f"variant {i} portions")


# ------------------------------------------------------------------ edges made visible
def _echo_model(win, block):
    """One attention layer whose key projection is minus its query projection, a large score
    scale, and a token pair with opposite embeddings (698 / 699): the key of a 699 matches the
    query of a 698 and outweighs every other key (the query's own key points the other way),
    so whether one far 699 is seen or not changes the logits of a 698 at once."""
    c = config([attn(heads=2, kv=2, dim=16, win=win, scale=2.0, ff=0)], groups=1, mult=1.0,
               vocab=700, width=32)
    w = O.random_weights(c, seed=9)
    w["l0.mix.k"] = -w["l0.mix.q"]
    w["embed"][699] = -w["embed"][698]
    w["l0.mix.k.norm"] = w["l0.mix.q.norm"].copy()
    w["l0.mix.talk"] = np.eye(2)
    return c, w


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("win", [8, 16, 333])
def test_window_edges_and_far_keys_stand_out(win, device, dtype):
    """The probe token sits just inside (distance win-1) or just outside (win) the window of
    the last position, among otherwise distinct tokens; whole prompt, decoded, and with the
    probe at a page border."""
    block = 8
    c, w = _echo_model(win, block)
    for dist in (win - 1, win):
        for n in (win + 5, win + block, 2 * win + 3):
            t = list(range(1, n + 1))
            t[n - 1 - dist] = 699
            t[n - 1] = 698
            want = O.forward(c, w, t)
            eng = engine(c, w, device, dtype, max_tokens=1024, block_size=block)
            close(replay(eng, t, [n])[-1:], want[-1:], dtype, f"prompt d={dist} n={n}")
            close(replay(eng, t, [n - 3, 1, 1, 1])[-1:], want[-1:], dtype, f"decode d={dist}")
            close(replay(eng, t, [n - 1 - dist, 1, dist - 1, 1] if dist > 1 else [n - 2, 1, 1])[-1:],
                  want[-1:], dtype, f"cut at the probe d={dist}")
    # seen and unseen differ visibly in the oracle itself, or the test shows nothing
    t_in, t_out = list(range(1, win + 6)), list(range(1, win + 6))
    t_in[-1] = t_out[-1] = 698
    t_in[-1 - (win - 1)] = 699
    t_out[-1 - win] = 699
    a, b = O.forward(c, w, t_in)[-1], O.forward(c, w, t_out)[-1]
    assert np.abs(a - b).max() > 0.2 * a.std()


@pytest.mark.parametrize("device,dtype", CASES)
def test_first_tokens_and_long_decode(device, dtype):
    c = config([attn(win=5), hgrn(), latent(win=4)], loop=(1, 3, 2))
    w = O.random_weights(c, seed=12)
    t = toks(70, c["vocab"], 4)
    want = O.forward(c, w, t)
    eng = engine(c, w, device, dtype)
    close(replay(eng, t, [1, 1, 2, 1] + [1] * 65), want, dtype, "from the first token on")
    close(replay(eng, t[:3], [3]), want[:3], dtype, "three tokens")
    close(replay(eng, t[:1], [1]), want[:1], dtype, "one token")


# ------------------------------------------------------------------ generation entry point
@pytest.mark.parametrize("device,dtype,graphs", [
    ("cpu", torch.float32, False),
    pytest.param("cuda", torch.float32, False, marks=pytest.mark.gpu),
    pytest.param("cuda", torch.bfloat16, True, marks=pytest.mark.gpu)])
def test_greedy_generation_through_the_engine(device, dtype, graphs):
    """LLMEngine.generate (scheduler admission, prefill, decode steps / captured graphs,
    sampler at temperature 0) against the oracle's argmax continuation; unequal prompts in
    one batch, more requests than slots."""
    w = O.random_weights(FULL, seed=7, scale=1.5)
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
            lg = O.forward(FULL, w, seq)[-1]
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
    assert cfg.is_hybrid and cfg.hidden_size == 48 and cfg.vocab_size == 96
    assert cfg.loop == (1, 4, 2) and cfg.norm_groups == 3 and cfg.residual_mult == 0.6
    assert [r[0] for r in cfg.layer_runs()] == [0, 1, 2, 3, 1, 2, 3, 4]
    s = cfg.layer_specs
    assert (s[0].heads, s[0].kv_heads, s[0].window, s[0].ff) == (4, 2, 6, 48)
    assert (s[2].kv_rank, s[2].rot_dim, s[2].rot_dims, s[2].rot_base) == (16, 8, 4, 300.0)
    assert s[3].ff == 0 and s[3].has_state
    c["layers"][0]["type"] = "convolution"
    with pytest.raises(ValueError):
        config_from_hf(c)


# ------------------------------------------------------------------ MFMA attention kernel
def _paged_case(lens, starts, H, G, dq, dv, block, shared_kv, seed, dtype=torch.bfloat16):
    """Random queries of portions [start, start+len) per sequence over shuffled pages."""
    g = torch.Generator().manual_seed(seed)
    S = len(lens)
    ctx = [s + n for s, n in zip(starts, lens)]
    nblk = [-(-c // block) for c in ctx]
    total = sum(nblk) + 3
    perm = torch.randperm(total, generator=g).tolist()
    tables = torch.zeros(S, max(nblk), dtype=torch.int32)
    at = 0
    for s in range(S):
        tables[s, :nblk[s]] = torch.tensor(perm[at:at + nblk[s]], dtype=torch.int32)
        at += nblk[s]
    kw = G * dq
    k_cache = torch.randn(total * block, kw, generator=g).to(dtype)
    v_cache = k_cache if shared_kv else torch.randn(total * block, G * dv, generator=g).to(dtype)
    T = sum(lens)
    q = torch.randn(T, H * dq, generator=g).to(dtype)
    cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32)
    pos = torch.cat([torch.arange(s, s + n, dtype=torch.int32) for s, n in zip(starts, lens)])
    return q, k_cache, v_cache, cu, pos, tables


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,dq,dv,win,talk,shared", [
    (4, 2, 32, 32, 24, True, False), (8, 8, 64, 64, 100, True, False),
    (32, 8, 128, 128, 70, True, False), (5, 1, 96, 64, 33, False, True),
    (16, 1, 160, 144, 64, False, True), (3, 3, 32, 32, 1, True, False),
    (4, 2, 32, 48, 5000, True, False), (40, 5, 32, 32, 50, False, False)])
def test_mfma_window_attention_matches_reference(gpu, H, G, dq, dv, win, talk, shared):
    from distributed_llm_inferencing_amd.ops import hybrid as Hy
    from distributed_llm_inferencing_amd.ops import reference as R
    lens, starts = [37, 1, 16, 5, 1], [0, 63, 48, 200, 0]
    block = 16
    q, kc, vc, cu, pos, bt = _paged_case(lens, starts, H, G, dq, dv, block, shared, seed=H + dq)
    g = torch.Generator().manual_seed(1)
    T = q.shape[0]
    slopes = torch.pow(2.0, -8.0 * torch.arange(1, H + 1) / H).float() if talk else None
    tk = (torch.eye(H) + 0.3 * torch.randn(H, H, generator=g)).to(torch.bfloat16).float() if talk else None
    gate = torch.randn(T, H * dv + 7, generator=g)[:, :H * dv] if talk else None
    scale = 1.0 / dq ** 0.5
    want = R.window_attention(q, kc, vc, dq, dv, H, G, cu, pos, bt, block, win, scale, slopes, tk,
                              gate, out_dtype=torch.float32)
    d = lambda t: None if t is None else t.to(gpu)      # noqa: E731
    args = (d(q), d(kc), d(kc) if shared else d(vc), dq, dv, H, G, d(cu), max(lens), d(pos),
            d(bt), block, win, scale, d(slopes), d(tk), d(gate))
    assert Hy.MFMA_ATTENTION
    got = Hy.window_attention(*args).float().cpu()
    Hy.MFMA_ATTENTION = False
    try:
        scalar = Hy.window_attention(*args).float().cpu()
    finally:
        Hy.MFMA_ATTENTION = True
    lim = 0.03 * want.abs().max().item() + 0.02
    assert (scalar - want).abs().max() < lim
    assert (got - want).abs().max() < lim
    assert not torch.equal(got, scalar) or H * dq < 64      # the two kernels really differ


@pytest.mark.gpu
@pytest.mark.parametrize("H,dq,dv,win", [(32, 96, 64, 300), (5, 64, 32, 40), (16, 160, 144, 1000)])
def test_mfma_decode_rows_of_shared_kv_heads(gpu, H, dq, dv, win):
    """Decode steps (one token a sequence) of heads that share one cached row per position,
    values = the row's first columns: the kernel's rows-are-heads form, with key splits."""
    from distributed_llm_inferencing_amd.ops import hybrid as Hy
    from distributed_llm_inferencing_amd.ops import reference as R
    starts = [0, 700, 31, 299, 300, 1, 64]
    lens = [1] * len(starts)
    q, kc, _, cu, pos, bt = _paged_case(lens, starts, H, 1, dq, dv, 16, True, seed=H)
    scale = dq ** -0.5
    want = R.window_attention(q, kc, kc, dq, dv, H, 1, cu, pos, bt, 16, win, scale,
                              out_dtype=torch.float32)
    d = lambda t: t.to(gpu)      # noqa: E731
    got = Hy.window_attention(d(q), d(kc), d(kc), dq, dv, H, 1, d(cu), 1, d(pos), d(bt), 16, win,
                              scale).float().cpu()
    assert (got - want).abs().max() < 0.03 * want.abs().max().item() + 0.02


@pytest.mark.gpu
def test_model_on_mfma_sized_heads(gpu):
    """A whole model whose head sizes take the MFMA attention path, cut in portions."""
    c = config([attn(heads=4, kv=2, dim=32, win=20, ff=64), hgrn(heads=2, dim=16, vdim=32),
                latent(heads=4, dim=16, rot_dim=16, vdim=16, rank=48, win=18, dims=8)],
               width=64, groups=2, loop=(0, 2, 2))
    w = O.random_weights(c, seed=31)
    t = toks(60, c["vocab"], 5)
    want = O.forward(c, w, t)
    eng = engine(c, w, "cuda", torch.bfloat16)
    close(replay(eng, t, [60]), want, torch.bfloat16, "whole")
    close(replay(eng, t, [17, 1, 1, 30, 2, 9]), want, torch.bfloat16, "portions")


@pytest.mark.parametrize("device,dtype", CASES[:2])
def test_generation_under_preemption(device, dtype):
    """A pool too small for the batch: sequences are preempted (blocks and state slot given
    back), re-admitted and recomputed from position 0; the tokens stay the oracle's."""
    w = O.random_weights(FULL, seed=8, scale=1.5)
    prompts = [toks(n, FULL["vocab"], 50 + n) for n in (14, 11, 16)]
    new = 14
    eng = engine(FULL, w, device, dtype, max_tokens=56, live=3)
    outs = eng.generate(prompts, SamplingParams(max_new_tokens=new, do_sample=False,
                                                ignore_eos=True))
    assert eng.scheduler.num_preempted > 0
    for p, o in zip(prompts, outs):
        seq = list(p)
        for tok in o.output_ids:
            lg = O.forward(FULL, w, seq)[-1]
            best = int(lg.argmax())
            assert tok == best or (lg[best] - lg[tok]) / lg.std() < 1e-3
            seq.append(tok)
        assert len(o.output_ids) == new
    assert eng.bm.num_free == eng.bm.num_blocks and eng.state_slots.num_free == 3


def test_registry_model_random_init_generates():
    """The registry's test-size hybrid (``buborax-tiny``) through the plain entry point: random
    init by name, prompts as text (byte tokenizer), sampled generation, deterministic per seed."""
    outs = []
    for _ in range(2):
        eng = LLMEngine("buborax-tiny", device="cpu", dtype=torch.float32, max_batch=4,
                        max_model_len=64, block_size=8, num_blocks=64, seed=3)
        o = eng.generate(["hybrid", "layers"], SamplingParams(max_new_tokens=6, seed=11,
                                                              ignore_eos=True))
        assert all(len(x.output_ids) == 6 for x in o)
        assert all(0 <= t < eng.cfg.vocab_size for x in o for t in x.output_ids)
        outs.append([x.output_ids for x in o])
    assert outs[0] == outs[1]
