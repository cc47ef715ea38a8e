"""Causal grouped-query softmax attention over a paged cache, with rotated keys AND rotated values.

q (H heads), k, v (G heads; query head h reads key / value head h // (H / G)) come from one product.  The first `rot_n`
dimensions of every q and k head turn with the position (halves layout, table `rope_k`); every value turns over all its
`vdim` dimensions by its own position (table `rope_v`) and is cached so; a head's output at position i is turned back by
-i, so that the sum carries the RELATIVE rotation i - j of each value.  score = q . k * scale, softmax over j <= i.

Cache: per key / value head one pool of rows [v (vdim) | k (dim)].  The attention itself is the paged row-attention kernel of
the latent layers (qserve_amd.layers.latent_attention): a query [0 (vdim) | q * scale] against such rows scores q . k, and
the softmax-weighted sum of the rows' first vdim elements is the output; one launch serves all key / value heads.

`NormedChunkAttention` is the position-free sibling on the same cache rows and kernel: queries and keys are RMS-normed over the
whole projection, positions enter through a learned bias per (distance bucket, head) and through chunks that bound what a query
sees, and the values may be blended with those an earlier layer computed for the same token.
"""
import math

import torch

from .ops import linear


class RotatedValueAttention:
    def __init__(self, ops, *, heads, kv_heads, dim, vdim, scale, rot_n, rope_k, rope_v, weights, page=64):
        """weights: q [H dim, D], k [G dim, D], v [G vdim, D], o [D, H vdim]."""
        if heads % kv_heads or vdim % 2 or rot_n % 2 or rot_n > dim:
            raise ValueError(f"attention: {heads} heads over {kv_heads}, vdim {vdim}, {rot_n} rotated of {dim}")
        self.ops, self.H, self.G, self.dim, self.vdim, self.scale, self.page = ops, heads, kv_heads, dim, vdim, float(scale), page
        self.rot_n, self.rope_k, self.rope_v = rot_n, rope_k, rope_v
        w = weights
        D = w["q"].size(1)
        for k, shp in {"q": (heads * dim, D), "k": (kv_heads * dim, D), "v": (kv_heads * vdim, D), "o": (D, heads * vdim)}.items():
            if tuple(w[k].shape) != shp:
                raise ValueError(f"attention weight {k}: shape {tuple(w[k].shape)}, expected {shp}")
        self.w_in, self.w_o = torch.cat([w["q"], w["k"], w["v"]], dim=0).contiguous(), w["o"].contiguous()
        self.cache_rows, self.state_specs = [(kv_heads, vdim + dim)], []

    def __call__(self, h, batch, pools, states):
        ops, T, H, G = self.ops, h.size(0), self.H, self.G
        pool = pools[0]                                                    # [G, rows, vdim + dim]
        n = batch.max_pos + 1
        proj = linear(h, self.w_in)
        qf = ops.attention_prep(proj, 0, H * self.dim, (H + G) * self.dim, H, G, self.dim, self.vdim, self.rot_n,
                                self.rope_k.reserve(n), self.rope_v.reserve(n), self.scale, pool, batch)
        o = ops.latent_attention(qf, pool, batch, None, self.vdim, self.page, q_first=self.vdim)      # head h reads pool h // (H / G)
        ops.rotate_heads(o, self.rope_v.table, batch.pos, -1.0)
        return linear(o.view(T, H * self.vdim), self.w_o)


def distance_bucket(n, rows, far):
    """Row of a bias table with `rows` rows for the distance n >= 0: distances below rows / 2 have a row each; from there the rows
    are spaced evenly in log(distance) up to `far`, bucket = rows / 2 + floor(log(n / half) / log(far / half) * (rows - half)), capped
    at the last row.  With integer `far` the floor is taken exactly (integer powers), not through floating-point logarithms."""
    half = rows // 2
    if n < half:
        return n
    m = rows - half
    if far <= half:
        raise ValueError(f"a bias table of {rows} rows needs its far distance above {half}, not {far}")
    if float(far).is_integer():
        far, k = int(far), 0
        while k < m and far ** (k + 1) * half ** (m - k - 1) <= n ** m:     # (far / half)^((k + 1) / m) <= n / half
            k += 1
    else:
        k = int(math.floor(math.log(n / half) / math.log(far / half) * m))
    return min(rows - 1, half + k)


def distance_bias_table(rel, far, length):
    """rel [rows, H] -> float [H, length]: entry [h, n] = rel[distance_bucket(n), h]; the kernels clamp larger distances to the
    last entry, so `length` = far + 1 covers every distance (beyond `far` the bucket is the last row)."""
    rows = rel.size(0)
    idx = torch.tensor([distance_bucket(n, rows, far) for n in range(length)], dtype=torch.long, device=rel.device)
    return rel.float()[idx].t().contiguous()


class NormedChunkAttention:
    def __init__(self, ops, *, heads, kv_heads, dim, vdim, scale, eps, weights, chunk=None, bias_far=None, mix=None, publish=False,
                 page=64):
        """weights: q [H dim, D], k [G dim, D], v [G vdim, D], q_norm [H dim], k_norm [G dim], o [D, H vdim], rel [rows, H] or None.
        chunk: position i sees j <= i with floor(j / chunk) == floor(i / chunk) (None: all j <= i).  bias_far: the distance at
        which the bias table's logarithmic rows end.  publish: this layer's own values go into the step's carry as "v_first";
        mix (a number): the cached values are (1 - mix) v + mix carry["v_first"]."""
        if heads % kv_heads:
            raise ValueError(f"attention: {heads} heads over {kv_heads}")
        self.ops, self.H, self.G, self.dim, self.vdim, self.page = ops, heads, kv_heads, dim, vdim, page
        self.scale, self.eps, self.chunk, self.mix, self.publish = float(scale), float(eps), int(chunk) if chunk else None, mix, publish
        w = weights
        D = w["q"].size(1)
        for k, shp in {"q": (heads * dim, D), "k": (kv_heads * dim, D), "v": (kv_heads * vdim, D), "q_norm": (heads * dim,),
                       "k_norm": (kv_heads * dim,), "o": (D, heads * vdim)}.items():
            if tuple(w[k].shape) != shp:
                raise ValueError(f"attention weight {k}: shape {tuple(w[k].shape)}, expected {shp}")
        self.w_in, self.w_o = torch.cat([w["q"], w["k"], w["v"]], dim=0).contiguous(), w["o"].contiguous()
        self.q_norm, self.k_norm = w["q_norm"].contiguous(), w["k_norm"].contiguous()
        self.bias = None
        if w.get("rel") is not None:
            if w["rel"].dim() != 2 or w["rel"].size(1) != heads or bias_far is None:
                raise ValueError(f"attention bias table {tuple(w['rel'].shape)} for {heads} heads, far distance {bias_far}")
            far = int(bias_far) if float(bias_far).is_integer() else float(bias_far)
            length = int(math.ceil(far)) + 1
            self.bias = distance_bias_table(w["rel"], far, min(length, self.chunk) if self.chunk else length)
        self.cache_rows, self.state_specs = [(kv_heads, vdim + dim)], []

    def __call__(self, h, batch, pools, states, carry=None):
        ops, T, H, G = self.ops, h.size(0), self.H, self.G
        pool = pools[0]                                                    # [G, rows, vdim + dim]
        proj = linear(h, self.w_in)
        o_k, o_v = H * self.dim, (H + G) * self.dim
        own = proj[:, o_v:o_v + G * self.vdim]
        v_first = None
        if self.mix is not None:
            v_first = carry["v_first"]
            if v_first.shape != own.shape:
                raise ValueError("blended values: the layers' value sizes differ")
        if self.publish:
            carry["v_first"] = own
        qf = ops.normed_attention_prep(proj, 0, o_k, o_v, H, G, self.dim, self.vdim, self.q_norm, self.k_norm, self.eps, self.scale,
                                       v_first, self.mix or 0.0, pool, batch)
        o = ops.latent_attention(qf, pool, batch, None, self.vdim, self.page, q_first=self.vdim, chunk=self.chunk, bias=self.bias)
        return linear(o.view(T, H * self.vdim), self.w_o)


class SinkWindowAttention:
    """Grouped-query attention over a sliding window whose softmax has a sink: a learned number per head joins the denominator,
    sum_j e^(s_j) + e^(sink_h), and carries no value.  score = q . k * scale.  Options, all parameters:

    * norm "head": q and k are RMS-normed per head with one weight [dim] shared by the heads; "all": over the whole projection
      with a weight as wide as it.
    * taps: a short causal convolution over time on every channel of q, k and v (weights [channels, taps], no bias, no
      activation) straight after the projection; the last taps - 1 projected rows of a sequence are its state (two copies).
    * rotary (a RotaryTable): the first rotary.dims dimensions of every q and k head turn with the position, neighbours paired.
    * keep_first: the first that many positions stay visible to every later query, at their true positions.
    * pool_block = P: beside the window's tokens a query at i sees one key and one value per block [bP, bP + P) that ends at or
      before i - window: the means of the block's cached keys and values (a second pool, ceil(page / P) rows per page, held by
      the page of the block's first position).
    * shared_kv: the layer has no keys and values of its own and reads the pools of another layer of the same head counts.
    Cache: per key / value head one pool of rows [v | k] (k after norm and rotation), as the row-attention kernels read them."""

    def __init__(self, ops, *, heads, kv_heads, dim, vdim, scale, eps, window, weights, norm="head", taps=None, rotary=None,
                 keep_first=0, pool_block=None, shared_kv=False, page=64):
        """weights: q [H dim, D], o [D, H vdim], q_norm, sink [H]; unless shared_kv: k [G dim, D], v [G vdim, D], k_norm; with
        taps: q_conv [H dim, taps], k_conv, v_conv."""
        if heads % kv_heads or norm not in ("head", "all") or not window or int(window) < 1:
            raise ValueError(f"attention: {heads} heads over {kv_heads}, norm {norm!r}, window {window}")
        if shared_kv and (taps or pool_block):
            raise ValueError("attention: a layer that reads another layer's keys and values has no convolution or pooled blocks")
        if pool_block and keep_first:
            raise ValueError("attention: pooled blocks and kept first tokens are alternatives")
        if pool_block and int(pool_block) < 1:
            raise ValueError(f"attention: pooled blocks of {pool_block} positions")
        self.ops, self.H, self.G, self.dim, self.vdim, self.page = ops, heads, kv_heads, dim, vdim, page
        self.scale, self.eps, self.window, self.keep_first = float(scale), float(eps), int(window), int(keep_first or 0)
        self.per_head, self.taps, self.rotary, self.shared_kv = norm == "head", int(taps) if taps else None, rotary, bool(shared_kv)
        self.pool_block = int(pool_block) if pool_block else None
        if rotary is not None and rotary.dims > dim:
            raise ValueError(f"attention: {rotary.dims} rotated dimensions in heads of {dim}")
        w = weights
        D = w["q"].size(1)
        expect = {"q": (heads * dim, D), "o": (D, heads * vdim), "sink": (heads,), "q_norm": (dim if self.per_head else heads * dim,)}
        if not shared_kv:
            expect.update(k=(kv_heads * dim, D), v=(kv_heads * vdim, D), k_norm=(dim if self.per_head else kv_heads * dim,))
        if self.taps:
            expect.update(q_conv=(heads * dim, self.taps), k_conv=(kv_heads * dim, self.taps), v_conv=(kv_heads * vdim, self.taps))
        for k, shp in expect.items():
            if tuple(w[k].shape) != shp:
                raise ValueError(f"attention weight {k}: shape {tuple(w[k].shape)}, expected {shp}")
        self.w_in = (w["q"] if shared_kv else torch.cat([w["q"], w["k"], w["v"]], dim=0)).contiguous()
        self.w_o, self.q_norm, self.k_norm = w["o"].contiguous(), w["q_norm"].contiguous(), None if shared_kv else w["k_norm"].contiguous()
        self.sink = w["sink"].float().contiguous()
        self.conv = torch.cat([w["q_conv"], w["k_conv"], w["v_conv"]], dim=0).float().contiguous() if self.taps else None
        self.C = (heads + kv_heads) * dim + kv_heads * vdim
        R = vdim + dim
        self.cache_rows, self.state_specs = [], []
        if not shared_kv:
            self.cache_rows.append((kv_heads, R))
            if self.pool_block:
                # (blocks longer than a page: at most one block starts in a page, one row a page)
                self.cache_rows.append((kv_heads, R, (page + self.pool_block - 1) // self.pool_block))
        if self.taps and self.taps > 1:
            from ..serving.cache import StateSpec
            self.state_specs.append(StateSpec((self.taps - 1, self.C), copies=2))

    def __call__(self, h, batch, pools, states, carry=None):
        ops, T, H, G, d, dv = self.ops, h.size(0), self.H, self.G, self.dim, self.vdim
        proj = linear(h, self.w_in)
        if self.taps and self.taps > 1:
            proj = ops.conv_silu_unit(proj, 0, self.conv, states[0], batch, 0, 1, act="none")          # float [T, C]
        elif self.taps:
            proj = proj.float() * self.conv[:, 0]
        q = proj[:, :H * d]
        k, v = (None, None) if self.shared_kv else (proj[:, H * d:(H + G) * d], proj[:, (H + G) * d:])
        rope = self.rotary.reserve(batch.max_pos + 1) if self.rotary is not None else None
        pool = pools[0]
        qf = ops.qk_norm_rope_prep(q, k, v, H, G, d, dv, self.q_norm, self.k_norm, self.per_head, self.eps, rope,
                                   self.rotary.dims if rope is not None else 0, self.scale, pool, batch)
        pooled = None
        if self.pool_block:
            pooled = pools[1]
            ops.pool_blocks(pool, pooled, batch, self.pool_block, self.page)
        o = ops.latent_attention(qf, pool, batch, self.window, dv, self.page, q_first=dv, keep_first=self.keep_first, sink=self.sink,
                                 pooled=pooled, pool_block=self.pool_block or 0)
        return linear(o.view(T, H * dv), self.w_o)
