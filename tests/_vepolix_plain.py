"""Plain, slow float64 statement of the Vepolix design: one function per mechanism, written from its equations, sharing no code
with qserve_amd.  Whole sequences only: no cache, no state hand-over, no batching - every token of a sequence is computed in
one go from the first, which is what the engine's cuts, batches and reused pages and slots must reproduce.

Notation: h [T, D] the input of a sublayer, W["name"] the checkpoint tensors (float64 here), `p` a tensor-name prefix.
"""
import math

import torch

F64 = torch.float64


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(z):
    return z * torch.sigmoid(z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def sinusoid(T, width):
    """Position p as a vector of sine / cosine pairs: pair i holds (sin, cos) of the angle p f_i, f_i = 10000^(-2i / width)."""
    out = torch.zeros(T, width, dtype=F64)
    for i in range((width + 1) // 2):
        a = torch.arange(T, dtype=F64) * (10000.0 ** (-2.0 * i / width))
        out[:, 2 * i] = torch.sin(a)
        if 2 * i + 1 < width:
            out[:, 2 * i + 1] = torch.cos(a)
    return out


def distance_bucket(n, rows, far):
    """Row of the bias table for the distance n >= 0: one row per distance below rows / 2, then rows spaced evenly in the
    logarithm of the distance up to `far`, the last row for everything beyond."""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


# ---- mixers ---------------------------------------------------------------------------------------------------------------

def chunked_attention(h, W, p, m, eps, v_first=None):
    """Softmax attention inside chunks of mask.size positions with a learned bias per (distance bucket, head); queries and
    keys are RMS-normed over all heads at once.  v_first [T, G, vdim] (or None): the values this layer's are blended with.
    -> (output [T, D], the values this layer used, before any blend - what a first layer hands on)."""
    T = h.size(0)
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    chunk = m["mask"]["size"] if m.get("mask") else None
    q = (rms(h @ W[p + "q"].T, eps) * W[p + "q.norm"]).view(T, H, d)
    k = (rms(h @ W[p + "k"].T, eps) * W[p + "k.norm"]).view(T, G, d)
    v = (h @ W[p + "v"].T).view(T, G, dv)
    own = v
    if v_first is not None:
        lam = W[p + "vmix"]
        v = (1.0 - lam) * v + lam * v_first
    rel = W[p + "rel"]
    B = rel.size(0)
    out = torch.zeros(T, H, dv, dtype=F64)
    for i in range(T):
        lo = (i // chunk) * chunk if chunk else 0
        js = list(range(lo, i + 1))
        rows = torch.tensor([distance_bucket(i - j, B, m["bias_max"]) for j in js])
        for hh in range(H):
            g = hh // (H // G)
            s = (k[lo:i + 1, g] @ q[i, hh]) * m["scale"] + rel[rows, hh]
            out[i, hh] = torch.softmax(s, dim=0) @ v[lo:i + 1, g]
    return out.reshape(T, H * dv) @ W[p + "o"].T, own


def mlstm(h, W, p, m, eps):
    """Matrix memory with exponential gates kept in range by a running maximum that starts at 0."""
    T = h.size(0)
    H, d, dv, cap = m["heads"], m["dim"], m["vdim"], float(m["gate_cap"])
    q = (h @ W[p + "q"].T).view(T, H, d) * d ** -0.5
    k = (h @ W[p + "k"].T).view(T, H, d)
    v = (h @ W[p + "v"].T).view(T, H, dv)
    li = cap * torch.tanh((h @ W[p + "i"].T + W[p + "i.b"]) / cap)                                   # [T, H]
    lf = torch.nn.functional.logsigmoid(cap * torch.tanh((h @ W[p + "f"].T + W[p + "f.b"]) / cap))
    out = torch.zeros(T, H, dv, dtype=F64)
    for hh in range(H):
        S, n, mx = torch.zeros(d, dv, dtype=F64), torch.zeros(d, dtype=F64), 0.0
        for t in range(T):
            new = max(float(lf[t, hh]) + mx, float(li[t, hh]))
            a, b = math.exp(float(lf[t, hh]) + mx - new), math.exp(float(li[t, hh]) - new)
            S = a * S + b * torch.outer(k[t, hh], v[t, hh])
            n = a * n + b * k[t, hh]
            mx = new
            out[t, hh] = (S.T @ q[t, hh]) / (max(abs(float(n @ q[t, hh])), math.exp(-mx)) + 1e-6)
    o = rms(out, eps).reshape(T, H * dv) * W[p + "norm"]
    return (o * torch.sigmoid(h @ W[p + "g"].T)) @ W[p + "o"].T


# ---- feed-forwards --------------------------------------------------------------------------------------------------------

def gated_unit(h, W, p, act):
    return (act(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def route(h, W, p, r):
    """-> (indices [T, top], weights [T, top]).  Choice by sigmoid score + correction inside the kept groups (group score =
    sum of its two largest choice scores); weights = the plain sigmoid scores times router.scale."""
    s = torch.sigmoid(h @ W[p + "router"].T)
    choice = s + W[p + "correction"]
    T, E = s.shape
    groups = r.get("groups") or {}
    G = int(groups.get("count", 1))
    keep = int(groups.get("keep", G))
    per = E // G
    idx, wt = [], []
    for t in range(T):
        c = choice[t].clone()
        score = [sum(sorted(c[g * per:(g + 1) * per].tolist(), reverse=True)[:2]) for g in range(G)]
        kept = sorted(range(G), key=lambda g: (-score[g], g))[:keep]
        for g in range(G):
            if g not in kept:
                c[g * per:(g + 1) * per] = -math.inf
        top = sorted(range(E), key=lambda e: (-float(c[e]), e))[:r["top"]]
        idx.append(top)
        wt.append([float(s[t, e]) * r["scale"] for e in top])
    return torch.tensor(idx), torch.tensor(wt, dtype=F64)


def moe(h, W, p, mlp):
    idx, wt = route(h, W, p, mlp["router"])
    y = torch.zeros_like(h)
    for t in range(h.size(0)):
        for e, w in zip(idx[t].tolist(), wt[t].tolist()):
            y[t] += w * gated_unit(h[t:t + 1], W, f"{p}e{e}.", silu)[0]
    if mlp.get("shared"):
        y = y + gated_unit(h, W, p + "shared.", silu)
    return y


def feed_forward(h, W, p, mlp):
    if mlp["kind"] == "dense":
        return gated_unit(h, W, p, gelu_tanh)
    return moe(h, W, p, mlp)


# ---- the model --------------------------------------------------------------------------------------------------------------

def forward(cfg, W, tokens):
    """-> (logits [T, vocab], the residual stream after every layer [layers, T, width])."""
    eps, D = cfg["norm"]["eps"], cfg["width"]
    T = len(tokens)
    x = W["embed"][torch.tensor(tokens)] * cfg["embedding"]["scale"] + sinusoid(T, D)
    v_first, taps = None, []
    for i, L in enumerate(cfg["layers"]):
        h = rms(x, eps) * W[f"l{i}.norm1"]
        if L["type"] == "attention":
            mix = L["mixer"].get("v_mix")
            y, own = chunked_attention(h, W, f"l{i}.mix.", L["mixer"], eps, v_first if mix else None)
            if mix and v_first is None:
                v_first = own
        elif L["type"] == "mlstm":
            y = mlstm(h, W, f"l{i}.mix.", L["mixer"], eps)
        else:
            raise ValueError(L["type"])
        if L.get("mlp"):
            y = y + feed_forward(h, W, f"l{i}.mlp.", L["mlp"])
        x = x + y
        taps.append(x)
    return (rms(x, eps) * W["final.norm"]) @ W["head"].T, torch.stack(taps)


def tensor_shapes(cfg):
    D, V = cfg["width"], cfg["vocab"]
    out = {"embed": (V, D), "head": (V, D), "final.norm": (D,)}
    for i, L in enumerate(cfg["layers"]):
        m, p = L["mixer"], f"l{i}.mix."
        out[f"l{i}.norm1"] = (D,)
        if L["type"] == "attention":
            H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            out.update({p + "q": (H * d, D), p + "k": (G * d, D), p + "v": (G * dv, D), p + "q.norm": (H * d,), p + "k.norm": (G * d,),
                        p + "rel": (m["rel_rows"], H), p + "vmix": (), p + "o": (D, H * dv)})
        else:
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            out.update({p + "q": (H * d, D), p + "k": (H * d, D), p + "v": (H * dv, D), p + "g": (H * dv, D), p + "o": (D, H * dv),
                        p + "norm": (H * dv,), p + "i": (H, D), p + "i.b": (H,), p + "f": (H, D), p + "f.b": (H,)})
        mlp, q = L.get("mlp"), f"l{i}.mlp."
        if not mlp:
            continue
        if mlp["kind"] == "dense":
            out.update({q + "gate": (mlp["ff"], D), q + "up": (mlp["ff"], D), q + "down": (D, mlp["ff"])})
        else:
            E, ff = mlp["router"]["experts"], mlp["expert"]["ff"]
            for e in range(E):
                out.update({f"{q}e{e}.gate": (ff, D), f"{q}e{e}.up": (ff, D), f"{q}e{e}.down": (D, ff)})
            out.update({q + "router": (E, D), q + "correction": (E,)})
            if mlp.get("shared"):
                sf = mlp["shared"]["ff"]
                out.update({q + "shared.gate": (sf, D), q + "shared.up": (sf, D), q + "shared.down": (D, sf)})
    return out


def random_weights(cfg, seed=0):
    """float64 tensors for every name of the configuration.  (`rel_rows` of an attention mixer is this module's own key: the
    number of rows of its bias table - a checkpoint gives it by the tensor's shape.)  Spreads are chosen so that every
    mechanism matters: norm weights around 1, biases and corrections of visible size, gates that open and close."""
    g = torch.Generator().manual_seed(seed)
    W = {}
    for name, shape in tensor_shapes(cfg).items():
        last = name.split(".")[-1]
        r = torch.randn(shape, generator=g, dtype=F64)
        if name.endswith("norm") or name.endswith("norm1"):
            W[name] = 1.0 + 0.2 * r
        elif last == "rel":
            W[name] = 1.5 * r
        elif last == "vmix":
            W[name] = torch.tensor(0.35, dtype=F64) + 0.1 * r
        elif last == "correction":
            W[name] = 0.3 * r
        elif last == "b":
            W[name] = r + (2.0 if name.endswith("f.b") else 0.0)
        elif name in ("embed",):
            W[name] = 0.5 * r
        else:
            W[name] = r / math.sqrt(shape[-1])
    return W
