"""Plain, slow implementation of the Pulunex design, used only as the tests' oracle.

Everything is float64 numpy on whole sequences (no cache, no state: a sequence is recomputed
from its first token), one function per mechanism. It shares no code with the package.

``cfg`` is the parsed config.json, ``w`` a dict name -> float64 array. The design:

* x_t = embed[token_t] * embedding.scale + pos[t];
* every layer: x += mixer(shift(norm(x))), then x += ff(norm(x)) when the layer has one;
* norm(v) = v / sqrt(mean(v^2) + eps) * g with ONE learned number g per norm;
* shift: the mixer reads u_t = h_t + (h_{t-1} - h_t) * mu (h_{-1} = 0), mu a learned vector;
* the mixer is softmax attention inside blocks of ``mask.size`` positions counted from the
  start of the sequence, without positional rotation, with biased q / k / v projections,
  unit-RMS queries and keys, scores mixed across heads before the softmax, grouped key /
  value heads, and optionally the keys and values of an earlier layer;
* the feed-forward is gelu_tanh(up) -> down, or a routed mixture of gated-SiLU experts with
  identity experts and an always-on shared expert behind a sigmoid gate;
* logits = head norm(x) * logit_scale.
"""
import math

import numpy as np


def unit_rms(v, eps):
    return v / math.sqrt(float(np.mean(v * v)) + eps)


def scalar_norm(v, g, eps):
    return unit_rms(v, eps) * float(g)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softmax(s):
    e = np.exp(s - s.max())
    return e / e.sum()


def embed(tokens, cfg, w):
    sc = cfg["embedding"]["scale"]
    return np.stack([w["embed"][t] * sc + w["pos"][p] for p, t in enumerate(tokens)])


def token_shift(hs, mu):
    """hs [T, D]: row t becomes h_t + (h_{t-1} - h_t) * mu, with the rows as they came in."""
    prev = np.vstack([np.zeros_like(hs[:1]), hs[:-1]])
    return hs + (prev - hs) * mu


def keys_values(us, mx, w, pre, eps):
    """Unit-RMS keys [T, G, d] and values [T, G, dv] of a layer that owns its projections."""
    T = us.shape[0]
    G, d, dv = mx["kv_heads"], mx["dim"], mx["vdim"]
    k = (us @ w[pre + "k"].T + w[pre + "k.b"]).reshape(T, G, d)
    v = (us @ w[pre + "v"].T + w[pre + "v.b"]).reshape(T, G, dv)
    kn = np.empty_like(k)
    for t in range(T):
        for g in range(G):
            kn[t, g] = unit_rms(k[t, g], eps)
    return kn, v


def block_attention(us, mx, w, pre, eps, kv):
    """us [T, D] mixer inputs of one sequence; kv = (keys, values) to attend. Returns [T, D]."""
    T = us.shape[0]
    H, G, d, dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    size = (mx.get("mask") or {}).get("size") or max(T, 1)      # no mask: one block
    scale = mx["scale"]
    kn, v = kv
    q = (us @ w[pre + "q"].T + w[pre + "q.b"]).reshape(T, H, d)
    talk = w[pre + "talk"]
    rep = H // G
    out = np.zeros((T, H * dv))
    for i in range(T):
        first = (i // size) * size
        js = list(range(first, i + 1))
        raw = np.empty((H, len(js)))
        for h in range(H):
            qh = unit_rms(q[i, h], eps)
            for n, j in enumerate(js):
                raw[h, n] = float(qh @ kn[j, h // rep]) * scale
        mixed = talk @ raw
        for h in range(H):
            p = softmax(mixed[h])
            o = np.zeros(dv)
            for n, j in enumerate(js):
                o += p[n] * v[j, h // rep]
            out[i, h * dv:(h + 1) * dv] = o
    return out @ w[pre + "o"].T


def gated_expert(h, w, pre):
    return w[pre + "down"] @ (silu(w[pre + "gate"] @ h) * (w[pre + "up"] @ h))


def routed_ff(h, mlp, w, pre, margin=None):
    """``margin`` (a one-element list) is lowered to the gap between the last chosen and the
    first rejected choice score: how close the routing of this token was to another outcome."""
    r = mlp["router"]
    E, I, top = r["experts"], r.get("identity", 0), r["top"]
    s = softmax(w[pre + "router"] @ h)
    choice = s + w[pre + "correction"]
    order = sorted(range(E + I), key=lambda e: (-choice[e], e))
    picked = order[:top]
    if margin is not None and top < E + I:
        margin[0] = min(margin[0], choice[order[top - 1]] - choice[order[top]])
    out = np.zeros_like(h)
    for e in picked:
        out += s[e] * (h if e >= E else gated_expert(h, w, f"{pre}e{e}."))
    if mlp.get("shared"):
        gate = sigmoid(float(w[pre + "shared.sg"].reshape(-1) @ h))
        out += gate * gated_expert(h, w, pre + "shared.")
    return out


def feed_forward(h, mlp, w, pre, margin=None):
    if mlp["kind"] == "dense":
        return w[pre + "down"] @ gelu_tanh(w[pre + "up"] @ h)
    return routed_ff(h, mlp, w, pre, margin)


def forward(tokens, cfg, w, trace=None, margins=None):
    """Logits [T, V] of one sequence; ``trace`` (a list) receives x after every layer,
    ``margins`` (a list) one number per position: its closest routing decision."""
    eps = cfg["norm"]["eps"]
    marg = [[math.inf] for _ in tokens]
    x = embed(tokens, cfg, w)
    kvs = {}
    for i, L in enumerate(cfg["layers"]):
        mx, pre = L["mixer"], f"l{i}.mix."
        hs = np.stack([scalar_norm(r, w[f"l{i}.norm1"], eps) for r in x])
        us = token_shift(hs, w[f"l{i}.shift"])
        src = mx.get("kv_from")
        if src is None:
            kvs[i] = keys_values(us, mx, w, pre, eps)
            src = i
        x = x + block_attention(us, mx, w, pre, eps, kvs[src])
        if L.get("mlp"):
            x = x + np.stack([feed_forward(scalar_norm(r, w[f"l{i}.norm2"], eps), L["mlp"], w,
                                           f"l{i}.mlp.", marg[t]) for t, r in enumerate(x)])
        if trace is not None:
            trace.append(x.copy())
    if margins is not None:
        margins.extend(m[0] for m in marg)
    hs = np.stack([scalar_norm(r, w["final.norm"], eps) for r in x])
    return hs @ w["head"].T * cfg.get("logit_scale", 1.0)


def tensor_shapes(cfg):
    """Name -> shape of every tensor a checkpoint of ``cfg`` holds."""
    D, V = cfg["width"], cfg["vocab"]
    out = {"embed": (V, D), "pos": (cfg["max_positions"], D), "final.norm": (), "head": (V, D)}
    for i, L in enumerate(cfg["layers"]):
        mx, p = L["mixer"], f"l{i}."
        H, G, d, dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
        out.update({p + "norm1": (), p + "shift": (D,), p + "mix.q": (H * d, D),
                    p + "mix.q.b": (H * d,), p + "mix.talk": (H, H), p + "mix.o": (D, H * dv)})
        if mx.get("kv_from") is None:
            out.update({p + "mix.k": (G * d, D), p + "mix.k.b": (G * d,),
                        p + "mix.v": (G * dv, D), p + "mix.v.b": (G * dv,)})
        mlp = L.get("mlp")
        if not mlp:
            continue
        out[p + "norm2"] = ()
        if mlp["kind"] == "dense":
            out.update({p + "mlp.up": (mlp["ff"], D), p + "mlp.down": (D, mlp["ff"])})
            continue
        r, F = mlp["router"], mlp["expert"]["ff"]
        n = r["experts"] + r.get("identity", 0)
        out.update({p + "mlp.router": (n, D), p + "mlp.correction": (n,)})
        for e in range(r["experts"]):
            out.update({f"{p}mlp.e{e}.gate": (F, D), f"{p}mlp.e{e}.up": (F, D),
                        f"{p}mlp.e{e}.down": (D, F)})
        if mlp.get("shared"):
            Fs = mlp["shared"]["ff"]
            out.update({p + "mlp.shared.gate": (Fs, D), p + "mlp.shared.up": (Fs, D),
                        p + "mlp.shared.down": (D, Fs), p + "mlp.shared.sg": (1, D)})
    return out


def random_weights(cfg, seed=0):
    """Random float64 weights, exactly representable in bfloat16 (so that a bf16 and an fp32
    copy of the checkpoint hold the same numbers), sized so that every mechanism matters:
    biases, shift vectors, router corrections and head mixing are all well away from their
    neutral values."""
    rng = np.random.default_rng(seed)

    def bf(a):
        a = np.asarray(a, np.float32)
        u = a.view(np.uint32)
        u = ((u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000).astype(np.uint32)
        return u.view(np.float32).astype(np.float64)

    w = {}
    for name, shape in tensor_shapes(cfg).items():
        if name.endswith(("norm1", "norm2", "final.norm")):
            v = 0.7 + 0.6 * rng.random(shape)
        elif name.endswith(".shift"):
            v = rng.random(shape)
        elif name.endswith(".talk"):
            v = np.eye(shape[0]) + 0.3 * rng.standard_normal(shape)
        elif name.endswith(".correction"):
            v = 0.1 * rng.standard_normal(shape)
        elif name.endswith(".b"):
            v = 0.3 * rng.standard_normal(shape)
        elif name == "pos":
            v = 0.5 * rng.standard_normal(shape)
        elif name == "embed":
            v = rng.standard_normal(shape) / cfg["embedding"]["scale"]
        elif name.endswith("mlp.router"):
            v = 2.0 * rng.standard_normal(shape) / math.sqrt(shape[-1])
        else:
            v = rng.standard_normal(shape) / math.sqrt(shape[-1])
        w[name] = bf(v).reshape(shape)
    return w
