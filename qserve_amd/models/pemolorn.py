"""Pemolorn: a decoder-only model whose sublayers sit between two RMS norms, x <- x + norm_b(sublayer(norm_a(x))), each norm with
ONE learned gain for all coordinates; the residual stream is float.

config.json: {architecture, width, vocab, norm: {eps}, layers: [{type, mixer: {...}, mlp: {...} | null}]}.
* Mixers: `attention` = qserve_amd.layers.softmax_attention.SinkWindowAttention with per-head query / key norms, no positions,
  a window that keeps the sequence's first tokens and a sink in the softmax; with `kv_from: j` the layer has queries only and
  reads layer j's cache.  `parallel` = the same attention class with a short convolution on q, k, v, norms over the whole
  projection, rotated pairs, and pooled blocks behind the window, beside qserve_amd.layers.recurrent.MinGRU, joined by
  ParallelMixer.
* Feed-forward: dense relu^2 units (ReluSquaredFeedForward) or IdentityExpertMoE (qserve_amd.layers.moe).
* Output: the norm `final.norm`, then the `head` matrix.
Tensor names: embed, head, final.norm, l<i>.norm1 / norm1b / norm2 / norm2b, l<i>.mix.{q, k, v, o, q.norm, k.norm, sink} or
l<i>.mix.left.{q, k, v, o, q.norm, k.norm, q.conv, k.conv, v.conv, sink, out} + l<i>.mix.right.{z, z.b, x, x.b, g, o, out},
l<i>.mlp.{up, down} or l<i>.mlp.{router, correction, e<k>.{gate, up, down}}.
"""
from ..layers.moe import IdentityExpertMoE, ReluSquaredFeedForward
from ..layers.ops import linear
from ..layers.recurrent import MinGRU, ParallelMixer
from ..layers.rotary import RotaryTable
from ..layers.softmax_attention import SinkWindowAttention
from ..serving.registry import register_model


@register_model("Pemolorn")
class Pemolorn:
    def __init__(self, ops, width, vocab, eps, embed, head, final_norm, layers, rotaries):
        self.ops, self.width, self.vocab, self.eps = ops, width, vocab, eps
        self.embed, self.head, self.layers, self.rotaries = embed, head, layers, rotaries
        self.final_norm = final_norm.expand(width).contiguous()          # (the row-norm kernel takes a gain per coordinate)
        self.cache_rows, self.state_specs, self.slices = [], [], []
        for L in layers:
            m = L["mixer"]
            p0, s0 = len(self.cache_rows), len(self.state_specs)
            self.cache_rows += m.cache_rows
            self.state_specs += m.state_specs
            self.slices.append((p0, len(self.cache_rows), s0, len(self.state_specs)))
        for i, L in enumerate(layers):                        # a layer without keys and values of its own reads its source's pools
            if L["kv_from"] is not None:
                self.slices[i] = self.slices[L["kv_from"]][:2] + self.slices[i][2:]

    def reserve_positions(self, n):
        for r in self.rotaries:
            r.reserve(n)

    def graph_signature(self):
        return tuple(r.table.data_ptr() for r in self.rotaries)

    @classmethod
    def from_config(cls, config, weights, ops, device, dtype, page=64):
        D, V, eps = int(config["width"]), int(config["vocab"]), float(config["norm"]["eps"])

        def w(name):
            if name not in weights:
                raise KeyError(f"checkpoint has no tensor {name!r}")
            return weights[name].to(device=device, dtype=dtype).contiguous()

        def gain(name):
            g = w(name).reshape(-1)
            if g.numel() != 1:
                raise ValueError(f"{name}: a norm of this design has one gain, not {g.numel()}")
            return g

        tables = {}

        def table(rot):
            t = RotaryTable(int(rot["dims"]), float(rot["base"]), rot.get("scaling"), device)
            return tables.setdefault(t.key(), t)

        def attention(m, p, **kw):
            names = [("q", "q"), ("o", "o"), ("q_norm", "q.norm"), ("sink", "sink")]
            if not kw.get("shared_kv"):
                names += [("k", "k"), ("v", "v"), ("k_norm", "k.norm")]
            if kw.get("taps"):
                names += [("q_conv", "q.conv"), ("k_conv", "k.conv"), ("v_conv", "v.conv")]
            mask = m["mask"]
            return SinkWindowAttention(
                ops, heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])), dim=int(m["dim"]), vdim=int(m["vdim"]),
                scale=float(m["scale"]), eps=eps, window=int(mask["size"]), weights={k: w(p + n) for k, n in names},
                rotary=table(m["rot"]) if m.get("rot") else None, keep_first=int(mask.get("keep_first", 0)),
                pool_block=int(mask["pool"]) if mask.get("pool") else None, page=page, **kw)

        layers = []
        for i, spec in enumerate(config["layers"]):
            kind, m, p = spec["type"], spec["mixer"], f"l{i}.mix."
            src = None
            if kind == "attention":
                if m.get("kv_from") is not None:
                    src = int(m["kv_from"])
                    if not 0 <= src < i or layers[src]["kv_from"] is not None:
                        raise ValueError(f"layer {i}: keys and values from layer {src}, which has none of its own before this layer")
                    other = config["layers"][src]["mixer"]
                    other = other.get("left", other)                # (a parallel layer's cache is its attention's)
                    if any(int(other[k]) != int(m[k]) for k in ("kv_heads", "dim", "vdim")):
                        raise ValueError(f"layer {i}: layer {src}'s keys and values have other sizes")
                mixer = attention(m, p, norm="head", shared_kv=src is not None)
            elif kind == "parallel":
                a, b = m["left"], m["right"]
                left = attention(a, p + "left.", norm="all", taps=int(a["conv"]) if a.get("conv") else None)
                q = p + "right."
                wr = {k: w(q + k) for k in ("z", "x", "g", "o")}
                wr.update(z_b=w(q + "z.b"), x_b=w(q + "x.b"))
                mixer = ParallelMixer(ops, left, MinGRU(ops, width=int(b["width"]), weights=wr), w(p + "left.out"), w(p + "right.out"), eps)
            else:
                raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
            L = {"mixer": mixer, "kv_from": src, "norm1": gain(f"l{i}.norm1"), "norm1b": gain(f"l{i}.norm1b"), "ff": None}
            mlp, q = spec.get("mlp"), f"l{i}.mlp."
            if mlp:
                if mlp["kind"] == "dense":
                    L["ff"] = ReluSquaredFeedForward(ops, up=w(q + "up"), down=w(q + "down"))
                    ff, want = L["ff"].w_up.size(0), int(mlp["ff"])
                elif mlp["kind"] == "moe":
                    r = mlp["router"]
                    E = int(r["experts"])
                    L["ff"] = IdentityExpertMoE(
                        ops, router=w(q + "router"), correction=w(q + "correction"), gate=[w(f"{q}e{e}.gate") for e in range(E)],
                        up=[w(f"{q}e{e}.up") for e in range(E)], down=[w(f"{q}e{e}.down") for e in range(E)], top_k=int(r["top"]),
                        identity=int(r.get("identity", 0)), limit=float(mlp["expert"]["limit"]))
                    ff, want = L["ff"].down.size(2), int(mlp["expert"]["ff"])
                else:
                    raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
                if ff != want:
                    raise ValueError(f"layer {i}: feed-forward tensors do not have ff = {want}")
                L["norm2"], L["norm2b"] = gain(f"l{i}.norm2"), gain(f"l{i}.norm2b")
            layers.append(L)
        embed, head = w("embed"), w("head")
        if embed.shape != (V, D) or head.shape != (V, D):
            raise ValueError("embed / head do not have the shape [vocab, width] of the config")
        return cls(ops, D, V, eps, embed, head, gain("final.norm"), layers, list(tables.values()))

    def forward(self, batch, pools, states=(), tap=None):
        """-> the float residual stream [T, width] after the last layer; tap(i, x) is called after every layer (tests)."""
        ops, n = self.ops, len(self.layers)
        x, _ = ops.embed(batch.tokens, self.embed)
        h = ops.add_normed_rms_norm(x, None, None, self.layers[0]["norm1"], self.eps) if n else None
        for i, L in enumerate(self.layers):
            p0, p1, s0, s1 = self.slices[i]
            y = L["mixer"](h, batch, pools[p0:p1], states[s0:s1])
            nxt = self.layers[i + 1]["norm1"] if i + 1 < n else None
            # each pass adds a normed sublayer output to the stream and norms the stream for the sublayer that follows
            if L["ff"] is not None:
                h = ops.add_normed_rms_norm(x, y, L["norm1b"], L["norm2"], self.eps)
                h = ops.add_normed_rms_norm(x, L["ff"](h), L["norm2b"], nxt, self.eps)
            else:
                h = ops.add_normed_rms_norm(x, y, L["norm1b"], nxt, self.eps)
            if tap is not None:
                tap(i, x)
        return x

    def logits(self, x, rows):
        return linear(self.ops.rms_norm_rows(x, rows, self.final_norm, self.eps), self.head).float()
