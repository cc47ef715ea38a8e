"""A plain, slow statement of the Pemolorn design in float64 numpy: one function per mechanism, whole sequences at once, no
cache, no batching.  It shares nothing with the served model; the tests compare the engine against it.

Notation: T tokens of one sequence at positions 0 .. T - 1 (or `pos`), D the model width, H query heads over G key / value heads.
"""
import math

import numpy as np


def rms(x, eps):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def short_conv(u, w):
    """u [T, C], w [C, taps]: y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros before the start."""
    T, C = u.shape
    taps = w.shape[1]
    padded = np.concatenate([np.zeros((taps - 1, C)), u])
    return sum(padded[j:j + T] * w[:, j] for j in range(taps))


def rotate_pairs(x, pos, dims, base):
    """x [T, heads, dim]: neighbours (2i, 2i + 1) of the first `dims` dimensions of each head turn by pos * base^(-2i / dims)."""
    out = x.copy()
    for i in range(dims // 2):
        a = np.asarray(pos, dtype=np.float64) * base ** (-2.0 * i / dims)
        c, s = np.cos(a)[:, None], np.sin(a)[:, None]
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * c - v * s
        out[..., 2 * i + 1] = v * c + u * s
    return out


def sink_softmax_sum(scores, values, sink):
    """One query: softmax over `scores` with exp(sink) added to the denominator, weighted sum of `values` [n, dv]."""
    m = max(float(np.max(scores)) if len(scores) else -math.inf, sink)
    e = np.exp(np.asarray(scores) - m)
    return (e[:, None] * values).sum(0) / (e.sum() + math.exp(sink - m))


def attention_kept_first(q, k, v, sink, scale, size, keep_first, store=lambda a: a):
    """q [T, H, d], k [T, G, d], v [T, G, dv]; i sees j <= i with i - j < size or j < keep_first.  `store` rounds what a cache
    would hold."""
    T, H, _ = q.shape
    G = k.shape[1]
    k, v = store(k), store(v)
    out = np.zeros((T, H, v.shape[2]))
    for i in range(T):
        js = [j for j in range(i + 1) if i - j < size or j < keep_first]
        for h in range(H):
            g = h // (H // G)
            out[i, h] = sink_softmax_sum([q[i, h] @ k[j, g] * scale for j in js], v[js, g], sink[h])
    return out


def attention_pooled_blocks(q, k, v, sink, scale, size, pool, store=lambda a: a):
    """i sees the tokens j with 0 <= i - j < size and one mean key / value per block of `pool` positions that ends at or before
    i - size; everything in one softmax with the sink."""
    T, H, _ = q.shape
    G = k.shape[1]
    k, v = store(k), store(v)
    nb = T // pool
    bk = store(np.stack([k[b * pool:(b + 1) * pool].mean(0) for b in range(nb)])) if nb else np.zeros((0,) + k.shape[1:])
    bv = store(np.stack([v[b * pool:(b + 1) * pool].mean(0) for b in range(nb)])) if nb else np.zeros((0,) + v.shape[1:])
    out = np.zeros((T, H, v.shape[2]))
    for i in range(T):
        js = [j for j in range(i + 1) if i - j < size]
        bs = [b for b in range(nb) if b * pool + pool - 1 <= i - size]
        for h in range(H):
            g = h // (H // G)
            sc = [q[i, h] @ bk[b, g] * scale for b in bs] + [q[i, h] @ k[j, g] * scale for j in js]
            vals = np.concatenate([bv[bs, g], v[js, g]]) if bs else v[js, g]
            out[i, h] = sink_softmax_sum(sc, vals, sink[h])
    return out


def min_gru(h, w):
    """h [T, D] -> [T, D]; w: z, z_b, x, x_b, g, o.  State from zero."""
    z = sigmoid(h @ w["z"].T + w["z_b"])
    u = h @ w["x"].T + w["x_b"]
    cand = np.where(u >= 0, u + 0.5, sigmoid(u))
    gate = h @ w["g"].T
    S = np.zeros(z.shape[1])
    out = np.zeros_like(z)
    for t in range(h.shape[0]):
        S = (1.0 - z[t]) * S + z[t] * cand[t]
        out[t] = S * gate[t] * sigmoid(gate[t])
    return out @ w["o"].T


def left_mixer(h, w, m, eps, store=lambda a: a):
    """The convolved, normed, rotated attention over a window and pooled blocks.  w: q, k, v, q_conv, k_conv, v_conv, q_norm,
    k_norm, sink, o; m: the mixer's config.  -> (output, (k, v) as a cache would hold them)."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q, k, v = (short_conv(h @ w[n].T, w[n + "_conv"]) for n in ("q", "k", "v"))
    q, k = rms(q, eps) * w["q_norm"], rms(k, eps) * w["k_norm"]
    pos = np.arange(T)
    rot = m.get("rot")
    q, k = q.reshape(T, H, d), k.reshape(T, G, d)
    if rot:
        q, k = rotate_pairs(q, pos, rot["dims"], rot["base"]), rotate_pairs(k, pos, rot["dims"], rot["base"])
    v = v.reshape(T, G, dv)
    o = attention_pooled_blocks(q, k, v, w["sink"], m["scale"], m["mask"]["size"], m["mask"]["pool"], store)
    return o.reshape(T, H * dv) @ w["o"].T, (k, v)


def attention_mixer(h, w, m, eps, shared=None, store=lambda a: a):
    """Per-head normed attention with kept first tokens.  shared = (k, v) of another layer (as cached) where the mixer has none
    of its own.  -> (output, (k, v))."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms((h @ w["q"].T).reshape(T, H, d), eps) * w["q_norm"]
    if shared is None:
        k = rms((h @ w["k"].T).reshape(T, G, d), eps) * w["k_norm"]
        v = (h @ w["v"].T).reshape(T, G, dv)
    else:
        k, v = shared
    o = attention_kept_first(q, k, v, w["sink"], m["scale"], m["mask"]["size"], m["mask"].get("keep_first", 0), store)
    return o.reshape(T, H * dv) @ w["o"].T, (k, v)


def dense_ff(h, w):
    a = np.maximum(h @ w["up"].T, 0.0)
    return (a * a) @ w["down"].T


def expert(h, gate, up, down, limit):
    g = np.minimum(h @ gate.T, limit)
    u = np.clip(h @ up.T, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ down.T


def moe_ff(h, w, top, identity, limit):
    """w: router [E + identity, D], correction, experts: list of (gate, up, down)."""
    z = h @ w["router"].T
    e = np.exp(z - z.max(-1, keepdims=True))
    s = e / e.sum(-1, keepdims=True)
    choice = s + w["correction"]
    E = len(w["experts"])
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        order = sorted(range(E + identity), key=lambda i: (-choice[t, i], i))[:top]
        for i in order:
            out[t] += s[t, i] * (h[t] if i >= E else expert(h[t:t + 1], *w["experts"][i], limit)[0])
    return out


def forward(config, W, tokens, taps=None, store=lambda a: a):
    """W: name -> float64 array (the checkpoint's names).  -> logits [T, vocab]; taps (a list) receives the stream after each layer."""
    eps = config["norm"]["eps"]
    x = W["embed"][np.asarray(tokens)]
    cached = {}
    for i, L in enumerate(config["layers"]):
        p, m = f"l{i}.", L["mixer"]
        h = rms(x, eps) * W[p + "norm1"]
        if L["type"] == "parallel":
            a, b = p + "mix.left.", p + "mix.right."
            wl = {n: W[a + n] for n in ("q", "k", "v", "sink", "o")}
            wl.update({n + "_conv": W[a + n + ".conv"] for n in ("q", "k", "v")}, q_norm=W[a + "q.norm"], k_norm=W[a + "k.norm"])
            wr = {n: W[b + n] for n in ("z", "x", "g", "o")}
            wr.update(z_b=W[b + "z.b"], x_b=W[b + "x.b"])
            (left, cached[i]), right = left_mixer(h, wl, m["left"], eps, store), min_gru(h, wr)
            y = 0.5 * (rms(left, eps) * W[a + "out"] + rms(right, eps) * W[b + "out"])
        elif L["type"] == "attention":
            a = p + "mix."
            wa = {n: W[a + n] for n in ("q", "sink", "o")}
            wa["q_norm"] = W[a + "q.norm"]
            shared = None
            if m.get("kv_from") is not None:
                shared = cached[int(m["kv_from"])]
            else:
                wa.update(k=W[a + "k"], v=W[a + "v"], k_norm=W[a + "k.norm"])
            y, cached[i] = attention_mixer(h, wa, m, eps, shared, store)
        else:
            raise ValueError(L["type"])
        x = x + rms(y, eps) * W[p + "norm1b"]
        mlp = L.get("mlp")
        if mlp:
            h = rms(x, eps) * W[p + "norm2"]
            q = p + "mlp."
            if mlp["kind"] == "dense":
                y = dense_ff(h, {"up": W[q + "up"], "down": W[q + "down"]})
            else:
                r = mlp["router"]
                ws = {"router": W[q + "router"], "correction": W[q + "correction"],
                      "experts": [(W[f"{q}e{e}.gate"], W[f"{q}e{e}.up"], W[f"{q}e{e}.down"]) for e in range(r["experts"])]}
                y = moe_ff(h, ws, r["top"], r.get("identity", 0), mlp["expert"]["limit"])
            x = x + rms(y, eps) * W[p + "norm2b"]
        if taps is not None:
            taps.append(x.copy())
    return (rms(x, eps) * W["final.norm"]) @ W["head"].T


def tensor_shapes(config):
    """name -> shape of every tensor a checkpoint of this config holds."""
    D, V, out = config["width"], config["vocab"], {}
    out["embed"], out["head"], out["final.norm"] = (V, D), (V, D), ()
    for i, L in enumerate(config["layers"]):
        p, m = f"l{i}.", L["mixer"]
        for n in ("norm1", "norm1b"):
            out[p + n] = ()

        def attention(q, a, whole, own=True):
            H, G, d, dv = a["heads"], a.get("kv_heads", a["heads"]), a["dim"], a["vdim"]
            out[q + "q"], out[q + "o"], out[q + "sink"] = (H * d, D), (D, H * dv), (H,)
            out[q + "q.norm"] = (H * d,) if whole else (d,)
            if own:
                out[q + "k"], out[q + "v"], out[q + "k.norm"] = (G * d, D), (G * dv, D), (G * d,) if whole else (d,)
            if a.get("conv"):
                out[q + "q.conv"], out[q + "k.conv"], out[q + "v.conv"] = (H * d, a["conv"]), (G * d, a["conv"]), (G * dv, a["conv"])

        if L["type"] == "parallel":
            attention(p + "mix.left.", m["left"], True)
            n = m["right"]["width"]
            for k in ("z", "x", "g"):
                out[p + "mix.right." + k] = (n, D)
            out[p + "mix.right.z.b"], out[p + "mix.right.x.b"], out[p + "mix.right.o"] = (n,), (n,), (D, n)
            out[p + "mix.left.out"], out[p + "mix.right.out"] = (D,), (D,)
        else:
            attention(p + "mix.", m, False, own=m.get("kv_from") is None)
        mlp = L.get("mlp")
        if mlp:
            out[p + "norm2"], out[p + "norm2b"] = (), ()
            if mlp["kind"] == "dense":
                out[p + "mlp.up"], out[p + "mlp.down"] = (mlp["ff"], D), (D, mlp["ff"])
            else:
                r, ff = mlp["router"], mlp["expert"]["ff"]
                n = r["experts"] + r.get("identity", 0)
                out[p + "mlp.router"], out[p + "mlp.correction"] = (n, D), (n,)
                for e in range(r["experts"]):
                    out[f"{p}mlp.e{e}.gate"], out[f"{p}mlp.e{e}.up"], out[f"{p}mlp.e{e}.down"] = (ff, D), (ff, D), (D, ff)
    return out


def random_weights(config, seed=0):
    """Random tensors (numpy float64, every value a bfloat16 number) with scales that keep every mechanism awake: gains near 1,
    sinks and corrections of the size of the scores they compete with."""
    import torch
    g = torch.Generator().manual_seed(seed)
    W = {}
    for name, shape in tensor_shapes(config).items():
        last = name.rsplit(".", 1)[-1]
        if shape == () or last in ("norm", "out"):
            t = 1.0 + 0.3 * torch.randn(shape, generator=g)
        elif last == "sink":
            t = torch.randn(shape, generator=g)
        elif last == "correction":
            t = 0.1 * torch.randn(shape, generator=g)
        elif last == "b":
            t = 0.5 * torch.randn(shape, generator=g)
        elif last == "conv":
            t = torch.randn(shape, generator=g) / math.sqrt(shape[1])
        elif name in ("embed",):
            t = torch.randn(shape, generator=g)
        else:
            t = torch.randn(shape, generator=g) / math.sqrt(shape[-1])
        W[name] = t.bfloat16().double().numpy()
    return W
