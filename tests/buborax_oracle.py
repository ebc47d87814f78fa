"""Plain, slow implementation of the Buborax design, used only as the tests' oracle.

Everything is float64 numpy, one token at a time where the design is sequential, one function
per mechanism. It shares no code with the package: the tests compare the framework's ops, model
and engine against these functions.

Model description (``cfg`` is the parsed config.json, ``w`` a dict name -> float64 array):

* residual stream x; every layer is x += m * mixer(gnorm(x)), then x += m * ff(gnorm(x));
* gnorm: the vector is cut into ``groups`` equal parts, each divided by its own
  sqrt(mean(part^2) + eps), the whole multiplied by a weight;
* layers [start, stop) repeat ``times`` times with the same weights; before each pass
  x = W_in [x; x0] + step[pass] with x0 the embedding output; every pass keeps a cache or state of
  its own (here: whole sequences are recomputed, so there is no cache at all).
"""
import math

import numpy as np


def rms(v, eps):
    return v / math.sqrt(float(np.mean(v * v)) + eps)


def group_norm(x, weight, groups, eps):
    n = x.shape[0] // groups
    out = np.empty_like(x)
    for g in range(groups):
        out[g * n:(g + 1) * n] = rms(x[g * n:(g + 1) * n], eps)
    return out * weight


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def softmax(s):
    e = np.exp(s - s.max())
    return e / e.sum()


def dense_ff(h, w, pre):
    return w[pre + "down"] @ (gelu_tanh(w[pre + "gate"] @ h) * (w[pre + "up"] @ h))


def attention_mixer(hs, mx, w, pre, eps):
    """hs: [T, D] inputs of one sequence (positions 0..T-1). Returns [T, D]."""
    T = hs.shape[0]
    H, G, d = mx["heads"], mx["kv_heads"], mx["dim"]
    win, scale = mx["mask"]["size"], mx["scale"]
    q = (hs @ w[pre + "q"].T).reshape(T, H, d)
    kraw = (hs @ w[pre + "k"].T).reshape(T, G, d)
    gate = sigmoid(hs @ w[pre + "g"].T)
    qn = np.empty_like(q)
    kn = np.empty_like(kraw)
    for t in range(T):
        for h in range(H):
            qn[t, h] = rms(q[t, h], eps) * w[pre + "q.norm"]
        for g in range(G):
            kn[t, g] = rms(kraw[t, g], eps) * w[pre + "k.norm"]
    talk = w[pre + "talk"]
    out = np.zeros((T, H * d))
    for i in range(T):
        lo = max(0, i - win + 1)
        probs = np.zeros((H, i + 1 - lo))
        for h in range(H):
            g = h // (H // G)
            slope = 2.0 ** (-8.0 * (h + 1) / H)
            s = np.array([qn[i, h] @ kn[j, g] * scale - slope * (i - j) for j in range(lo, i + 1)])
            probs[h] = softmax(s)
        mixed = talk @ probs
        for h in range(H):
            g = h // (H // G)
            out[i, h * d:(h + 1) * d] = mixed[h] @ kraw[lo:i + 1, g]
    return (out * gate) @ w[pre + "o"].T


def hgrn2_mixer(hs, mx, w, pre, eps):
    T = hs.shape[0]
    H, d, dv = mx["heads"], mx["dim"], mx["vdim"]
    qz = hs @ w[pre + "q"].T
    q = (qz * sigmoid(qz)).reshape(T, H, d)
    v = (hs @ w[pre + "v"].T).reshape(T, H, dv)
    low = w[pre + "lower"]
    f = (low + (1.0 - low) * sigmoid(hs @ w[pre + "f"].T + w[pre + "f.b"])).reshape(T, H, d)
    S = np.zeros((H, d, dv))
    out = np.zeros((T, H * dv))
    for t in range(T):
        for h in range(H):
            S[h] = f[t, h][:, None] * S[h] + np.outer(1.0 - f[t, h], v[t, h])
            o = S[h].T @ q[t, h]
            out[t, h * dv:(h + 1) * dv] = rms(o, eps) * w[pre + "norm"]
    return out @ w[pre + "o"].T


def rotate_interleaved(v, pos, dims, base):
    out = v.copy()
    for i in range(dims // 2):
        a = pos * base ** (-2.0 * i / dims)
        c, s = math.cos(a), math.sin(a)
        x, y = v[2 * i], v[2 * i + 1]
        out[2 * i] = x * c - y * s
        out[2 * i + 1] = y * c + x * s
    return out


def latent_attention_mixer(hs, mx, w, pre, eps):
    T = hs.shape[0]
    H, d, dr, dv, r = mx["heads"], mx["dim"], mx["rot_dim"], mx["vdim"], mx["kv_rank"]
    win, scale = mx["mask"]["size"], mx["scale"]
    rot = mx["rot"]
    q = (hs @ w[pre + "q"].T).reshape(T, H, d + dr)
    dkv = hs @ w[pre + "dkv"].T
    c = np.stack([rms(dkv[t, :r], eps) * w[pre + "dkv.norm"] for t in range(T)])
    krot = np.stack([rotate_interleaved(dkv[t, r:], t, rot["dims"], rot["base"])
                     for t in range(T)])
    ku = (c @ w[pre + "uk"].T).reshape(T, H, d)
    vv = (c @ w[pre + "uv"].T).reshape(T, H, dv)
    out = np.zeros((T, H * dv))
    for i in range(T):
        lo = max(0, i - win + 1)
        for h in range(H):
            qr = rotate_interleaved(q[i, h, d:], i, rot["dims"], rot["base"])
            s = np.array([(q[i, h, :d] @ ku[j, h] + qr @ krot[j]) * scale
                          for j in range(lo, i + 1)])
            out[i, h * dv:(h + 1) * dv] = softmax(s) @ vv[lo:i + 1, h]
    return out @ w[pre + "o"].T


MIXERS = {"attention": attention_mixer, "hgrn2": hgrn2_mixer,
          "latent_attention": latent_attention_mixer}


def layer_runs(cfg):
    """[(layer index, pass number or None, first of its pass)] in execution order."""
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return [(i, None, False) for i in range(n)]
    runs = [(i, None, False) for i in range(lp["start"])]
    for t in range(lp["times"]):
        for i in range(lp["start"], lp["stop"]):
            runs.append((i, t, i == lp["start"]))
    return runs + [(i, None, False) for i in range(lp["stop"], n)]


def forward(cfg, w, tokens, return_layers=False):
    """Logits [T, vocab] of one whole sequence (and the residual after every layer run)."""
    eps, groups, m = cfg["norm"]["eps"], cfg["norm"]["groups"], cfg["residual_mult"]
    x = w["embed"][np.asarray(tokens)]
    x0 = x.copy()
    layers = []
    for i, t, first in layer_runs(cfg):
        L = cfg["layers"][i]
        pre = "l%d." % i
        if first:
            x = np.concatenate([x, x0], axis=1) @ w["loop.in"].T + w["loop.step"][t]
        hs = np.stack([group_norm(r, w[pre + "norm1"], groups, eps) for r in x])
        x = x + m * MIXERS[L["type"]](hs, L["mixer"], w, pre + "mix.", eps)
        if L.get("mlp"):
            hs = np.stack([group_norm(r, w[pre + "norm2"], groups, eps) for r in x])
            x = x + m * np.stack([dense_ff(h, w, pre + "mlp.") for h in hs])
        layers.append(x.copy())
    hs = np.stack([group_norm(r, w["final.norm"], groups, eps) for r in x])
    logits = hs @ w["head"].T
    return (logits, np.stack(layers)) if return_layers else logits


def random_weights(cfg, seed=0, scale=1.0):
    """Random float64 weights with the design's tensor names, rounded to bfloat16 values so the
    framework (bf16 storage) and the oracle see the same numbers."""
    import torch
    g = np.random.default_rng(seed)
    D, V = cfg["width"], cfg["vocab"]
    w = {}

    def mat(o, i, gain=1.0):
        return g.standard_normal((o, i)) * gain * scale / math.sqrt(i)

    w["embed"] = g.standard_normal((V, D))
    w["head"] = mat(V, D)
    w["final.norm"] = 1.0 + 0.1 * g.standard_normal(D)
    lp = cfg.get("loop")
    if lp:
        w["loop.in"] = mat(D, 2 * D, 1.4)
        w["loop.step"] = 0.3 * g.standard_normal((lp["times"], D))
    for i, L in enumerate(cfg["layers"]):
        p, mx = "l%d." % i, L["mixer"]
        w[p + "norm1"] = 1.0 + 0.1 * g.standard_normal(D)
        if L["type"] == "attention":
            H, G, d = mx["heads"], mx["kv_heads"], mx["dim"]
            w[p + "mix.q"], w[p + "mix.k"] = mat(H * d, D), mat(G * d, D)
            w[p + "mix.q.norm"] = 1.0 + 0.2 * g.standard_normal(d)
            w[p + "mix.k.norm"] = 1.0 + 0.2 * g.standard_normal(d)
            w[p + "mix.talk"] = np.eye(H) + 0.3 * g.standard_normal((H, H))
            w[p + "mix.g"], w[p + "mix.o"] = mat(H * d, D), mat(D, H * d)
        elif L["type"] == "hgrn2":
            H, d, dv = mx["heads"], mx["dim"], mx["vdim"]
            w[p + "mix.q"], w[p + "mix.f"], w[p + "mix.v"] = mat(H * d, D), mat(H * d, D), mat(H * dv, D)
            w[p + "mix.f.b"] = g.standard_normal(H * d)
            w[p + "mix.lower"] = g.uniform(0.0, 0.9, H * d)
            w[p + "mix.norm"] = 1.0 + 0.2 * g.standard_normal(dv)
            w[p + "mix.o"] = mat(D, H * dv)
        else:
            H, d, dr, dv, r = mx["heads"], mx["dim"], mx["rot_dim"], mx["vdim"], mx["kv_rank"]
            w[p + "mix.q"], w[p + "mix.dkv"] = mat(H * (d + dr), D), mat(r + dr, D)
            w[p + "mix.dkv.norm"] = 1.0 + 0.2 * g.standard_normal(r)
            w[p + "mix.uk"], w[p + "mix.uv"] = mat(H * d, r), mat(H * dv, r)
            w[p + "mix.o"] = mat(D, H * dv)
        if L.get("mlp"):
            F = L["mlp"]["ff"]
            w[p + "norm2"] = 1.0 + 0.1 * g.standard_normal(D)
            w[p + "mlp.gate"], w[p + "mlp.up"], w[p + "mlp.down"] = mat(F, D), mat(F, D), mat(D, F)
    return {k: torch.tensor(v).to(torch.bfloat16).double().numpy() for k, v in w.items()}
