"""Vepolix: a decoder-only model of parallel layers - one RMS norm feeds a mixer and a feed-forward, and both outputs join the
float residual stream together, x <- x + (mixer(h) + ff(h)) with h = rms_norm(x) * w.

config.json: {architecture, width, vocab, embedding: {scale}, norm: {eps}, layers: [{type, mixer: {...}, mlp: {...} | null}]}.
* Input: embed[token] * embedding.scale + the position as sine / cosine pairs (pair i: sin and cos of p f_i, f_i = 10000^(-2i / width)).
* Mixers: `attention` = qserve_amd.layers.softmax_attention.NormedChunkAttention (queries / keys normed over all heads, a bias
  per distance bucket and head, chunks of mask.size positions, values blended with the first v_mix layer's where v_mix is set);
  `mlstm` = qserve_amd.layers.recurrent.MatrixLSTM.
* Feed-forward: dense gated units with the tanh form of gelu, or qserve_amd.layers.moe.CorrectedSigmoidMoE (silu experts, a
  shared expert).  Output: rms_norm(x) * final.norm, then the `head` matrix.
Tensor names: embed, head, final.norm, l<i>.norm1, l<i>.mix.{q, k, v, o, q.norm, k.norm, rel, vmix} or l<i>.mix.{q, k, v, g, o,
norm, i, i.b, f, f.b}, l<i>.mlp.{gate, up, down} or l<i>.mlp.{router, correction, e<k>.{gate, up, down}, shared.{gate, up, down}}.
"""
import torch

from ..layers.moe import CorrectedSigmoidMoE, GatedFeedForward
from ..layers.ops import linear
from ..layers.recurrent import MatrixLSTM
from ..layers.softmax_attention import NormedChunkAttention
from ..serving.registry import register_model


def sinusoid_frequencies(width, base=10000.0):
    """float [(width + 1) // 2]: base^(-2i / width), made in float64 and rounded once."""
    return torch.tensor([base ** (-2.0 * i / width) for i in range((width + 1) // 2)], dtype=torch.float64).to(torch.float32)


@register_model("Vepolix")
class Vepolix:
    def __init__(self, ops, width, vocab, eps, scale, embed, freq, head, final_norm, layers):
        self.ops, self.width, self.vocab, self.eps, self.scale = ops, width, vocab, eps, scale
        self.embed, self.freq, self.head, self.final_norm, self.layers = embed, freq, head, final_norm, layers
        self.cache_rows, self.state_specs, self.slices = [], [], []
        for L in layers:
            m = L["mixer"]
            p0, s0 = len(self.cache_rows), len(self.state_specs)
            self.cache_rows += m.cache_rows
            self.state_specs += m.state_specs
            self.slices.append((p0, len(self.cache_rows), s0, len(self.state_specs)))

    @classmethod
    def from_config(cls, config, weights, ops, device, dtype, page=64):
        D, V, eps = int(config["width"]), int(config["vocab"]), float(config["norm"]["eps"])

        def w(name):
            if name not in weights:
                raise KeyError(f"checkpoint has no tensor {name!r}")
            return weights[name].to(device=device, dtype=dtype).contiguous()

        def unit(prefix, ff, act):
            u = GatedFeedForward(ops, gate=w(prefix + "gate"), up=w(prefix + "up"), down=w(prefix + "down"), act=act)
            if u.w_down.shape != (D, int(ff)):
                raise ValueError(f"{prefix}: feed-forward tensors do not have ff = {ff}")
            return u

        layers, published = [], False
        for i, spec in enumerate(config["layers"]):
            kind, m, p = spec["type"], spec["mixer"], f"l{i}.mix."
            if kind == "attention":
                wm = {k: w(p + n) for k, n in (("q", "q"), ("k", "k"), ("v", "v"), ("o", "o"), ("q_norm", "q.norm"), ("k_norm", "k.norm"))}
                wm["rel"] = w(p + "rel") if (p + "rel") in weights else None
                blend = bool(m.get("v_mix"))
                mixer = NormedChunkAttention(
                    ops, heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])), dim=int(m["dim"]), vdim=int(m["vdim"]),
                    scale=float(m["scale"]), eps=eps, weights=wm, chunk=int(m["mask"]["size"]) if m.get("mask") else None,
                    bias_far=m.get("bias_max"), publish=blend and not published,
                    mix=float(weights[p + "vmix"].float()) if blend and published else None, page=page)
                published = published or blend
            elif kind == "mlstm":
                wm = {k: w(p + k) for k in ("q", "k", "v", "g", "o", "norm", "i", "f")}
                wm.update(i_b=w(p + "i.b"), f_b=w(p + "f.b"))
                mixer = MatrixLSTM(ops, heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]), gate_cap=float(m["gate_cap"]),
                                   eps=eps, weights=wm)
            else:
                raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
            L = {"mixer": mixer, "norm1": w(f"l{i}.norm1"), "ff": None}
            mlp, q = spec.get("mlp"), f"l{i}.mlp."
            if mlp:
                if mlp["kind"] == "dense":
                    L["ff"] = unit(q, mlp["ff"], "gelu_tanh")
                elif mlp["kind"] == "moe":
                    r = mlp["router"]
                    E, g = int(r["experts"]), r.get("groups") or {}
                    L["ff"] = CorrectedSigmoidMoE(
                        ops, router=w(q + "router"), correction=w(q + "correction"), gate=[w(f"{q}e{e}.gate") for e in range(E)],
                        up=[w(f"{q}e{e}.up") for e in range(E)], down=[w(f"{q}e{e}.down") for e in range(E)], top_k=int(r["top"]),
                        groups=int(g.get("count", 1)), keep=int(g.get("keep", g.get("count", 1))), scale=float(r.get("scale", 1.0)),
                        shared=unit(q + "shared.", mlp["shared"]["ff"], "silu") if mlp.get("shared") else None)
                    if L["ff"].down.size(2) != int(mlp["expert"]["ff"]):
                        raise ValueError(f"layer {i}: expert tensors do not have ff = {mlp['expert']['ff']}")
                else:
                    raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
            layers.append(L)
        embed, head = w("embed"), w("head")
        if embed.shape != (V, D) or head.shape != (V, D):
            raise ValueError("embed / head do not have the shape [vocab, width] of the config")
        return cls(ops, D, V, eps, float(config["embedding"]["scale"]), embed, sinusoid_frequencies(D).to(device), head,
                   w("final.norm"), layers)

    def forward(self, batch, pools, states=(), tap=None):
        """-> the float residual stream [T, width] after the last layer; tap(i, x) is called after every layer (tests)."""
        ops, n = self.ops, len(self.layers)
        x = ops.embed_sinusoid(batch.tokens, batch.pos, self.embed, self.freq, self.scale)
        h = ops.add_rms_norm(x, [], self.layers[0]["norm1"], self.eps) if n else None
        carry = {}                                              # what one layer of this step hands to later ones
        for i, L in enumerate(self.layers):
            p0, p1, s0, s1 = self.slices[i]
            ys = [L["mixer"](h, batch, pools[p0:p1], states[s0:s1], carry)]
            if L["ff"] is not None:
                f = L["ff"](h)
                ys += f if isinstance(f, list) else [f]
            # the next layer's input comes out of the pass that adds this layer's outputs to the stream
            h = ops.add_rms_norm(x, ys, self.layers[i + 1]["norm1"] if i + 1 < n else None, self.eps)
            if tap is not None:
                tap(i, x)
        return x

    def logits(self, x, rows):
        return linear(self.ops.rms_norm_rows(x, rows, self.final_norm, self.eps), self.head).float()
