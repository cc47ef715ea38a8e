"""Linear-recurrence mixers: a matrix state S [dim, vdim] per head and sequence, advanced token by token in float.

GatedLinearAttention   S <- diag(a) S + k v^T;  o = S^T q          a = sigmoid(z)^(1 / tau) per key channel
GatedDeltaRule         S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q   (o is read from the updated S)
                       g = exp(-exp(A_log) softplus(z + dt_bias)) per head and key channel, beta = sigmoid(.) per head,
                       q, k, v through a short causal convolution + silu, q and k made unit vectors per head

MatrixLSTM             S <- a S + b k v^T, n <- a n + b k;  o = S^T q / (max(|n . q|, exp(-m)) + 1e-6)
                       a = exp(f + m' - m), b = exp(i - m) per head from a log input gate i and a log forget gate f, both soft-
                       capped, and the running maximum m = max(f + m', i) that keeps the exponentials in range (m' = 0 at the start)

All read every projection of the layer input from ONE product; the low-rank second stages (decay, gate) are products of
their own.  State per sequence: the matrices (one copy: a run of tokens is read, advanced and written back by the workgroups
that own its columns) and, for the convolution, the last taps - 1 inputs (two copies, swapped per step).
"""
import torch

from ..serving.cache import StateSpec
from .ops import linear


def _check(w, expect, what):
    for k, shp in expect.items():
        if tuple(w[k].shape) != shp:
            raise ValueError(f"{what} weight {k}: shape {tuple(w[k].shape)}, expected {shp}")


class GatedLinearAttention:
    def __init__(self, ops, *, heads, dim, vdim, tau, eps, weights):
        """weights: q, k [H dim, D], v, g [H vdim, D], o [D, H vdim], norm [vdim], a1 [r, D], a2 [H dim, r], a2_b [H dim]."""
        self.ops, self.H, self.dim, self.vdim, self.tau, self.eps = ops, heads, dim, vdim, float(tau), float(eps)
        w = weights
        D, r = w["q"].size(1), w["a1"].size(0)
        _check(w, {"q": (heads * dim, D), "k": (heads * dim, D), "v": (heads * vdim, D), "g": (heads * vdim, D), "o": (D, heads * vdim),
                   "norm": (vdim,), "a1": (r, D), "a2": (heads * dim, r), "a2_b": (heads * dim,)}, "gated linear attention")
        self.w_in = torch.cat([w["q"], w["k"], w["v"], w["g"], w["a1"]], dim=0).contiguous()
        self.r, self.w_a2, self.b_a2, self.norm, self.w_o = r, w["a2"].contiguous(), w["a2_b"], w["norm"], w["o"].contiguous()
        self.cache_rows, self.state_specs = [], [StateSpec((heads, dim, vdim))]

    def __call__(self, h, batch, pools, states):
        ops, H, d, dv = self.ops, self.H, self.dim, self.vdim
        proj = linear(h, self.w_in)
        o_q, o_k, o_v, o_g, o_a = 0, H * d, 2 * H * d, 2 * H * d + H * dv, 2 * H * d + 2 * H * dv
        z = linear(proj[:, o_a:o_a + self.r], self.w_a2)
        a = ops.decay(z, self.b_a2, None, self.tau, H, d)
        o = ops.recurrent_scan(proj[:, o_q:o_k], proj[:, o_k:o_v], proj[:, o_v:o_g], a, None, states[0], batch, H, H, d, dv,
                               d ** -0.5)
        return linear(ops.head_rms_gate(o, self.norm, proj[:, o_g:o_a], "silu", self.eps), self.w_o)


class GatedDeltaRule:
    def __init__(self, ops, *, heads, kv_heads, dim, vdim, taps, eps, weights):
        """weights: q, k [G dim, D], v [H vdim, D], q_conv, k_conv [G dim, taps], v_conv [H vdim, taps], b [H, D], A_log [H],
        norm [vdim], a1 [r, D], a2 [H dim, r], dt_bias [H dim], g1 [r', D], g2 [H vdim, r'], o [D, H vdim]."""
        if heads % kv_heads or taps < 1:
            raise ValueError(f"gated delta rule: {heads} heads over {kv_heads}, {taps} taps")
        self.ops, self.H, self.G, self.dim, self.vdim, self.taps, self.eps = ops, heads, kv_heads, dim, vdim, int(taps), float(eps)
        w = weights
        D, r, rg = w["q"].size(1), w["a1"].size(0), w["g1"].size(0)
        _check(w, {"q": (kv_heads * dim, D), "k": (kv_heads * dim, D), "v": (heads * vdim, D), "q_conv": (kv_heads * dim, taps),
                   "k_conv": (kv_heads * dim, taps), "v_conv": (heads * vdim, taps), "b": (heads, D), "A_log": (heads,),
                   "norm": (vdim,), "a1": (r, D), "a2": (heads * dim, r), "dt_bias": (heads * dim,), "g1": (rg, D),
                   "g2": (heads * vdim, rg), "o": (D, heads * vdim)}, "gated delta rule")
        self.w_in = torch.cat([w["q"], w["k"], w["v"], w["b"], w["a1"], w["g1"]], dim=0).contiguous()
        self.conv = torch.cat([w["q_conv"], w["k_conv"], w["v_conv"]], dim=0).float().contiguous()
        self.r, self.rg = r, rg
        self.w_a2, self.dt_bias, self.a_log = w["a2"].contiguous(), w["dt_bias"], w["A_log"].float().contiguous()
        self.w_g2, self.norm, self.w_o = w["g2"].contiguous(), w["norm"], w["o"].contiguous()
        self.C = 2 * kv_heads * dim + heads * vdim
        self.cache_rows = []
        self.state_specs = [StateSpec((heads, dim, vdim)), StateSpec((max(self.taps - 1, 1), self.C), copies=2)]

    def __call__(self, h, batch, pools, states):
        ops, H, G, d, dv = self.ops, self.H, self.G, self.dim, self.vdim
        proj = linear(h, self.w_in)
        o_b = self.C
        o_a, o_g = o_b + H, o_b + H + self.r
        qkv = ops.conv_silu_unit(proj, 0, self.conv, states[1], batch, 2 * G, d)       # float [T, C]: q | k (unit) | v
        g = ops.decay(linear(proj[:, o_a:o_g], self.w_a2), self.dt_bias, self.a_log, 0.0, H, d)
        o = ops.recurrent_scan(qkv[:, :G * d], qkv[:, G * d:2 * G * d], qkv[:, 2 * G * d:], g, proj[:, o_b:o_a], states[0], batch,
                               H, G, d, dv, d ** -0.5)
        gate = linear(proj[:, o_g:o_g + self.rg], self.w_g2)
        return linear(ops.head_rms_gate(o, self.norm, gate, "sigmoid", self.eps), self.w_o)


class ParallelMixer:
    """Two mixers side by side on the same input; result = half the sum of their outputs, each RMS-normed over the model width
    with its own weight."""

    def __init__(self, ops, left, right, w_left, w_right, eps):
        self.ops, self.left, self.right, self.w_left, self.w_right, self.eps = ops, left, right, w_left, w_right, float(eps)
        self.cache_rows = list(left.cache_rows) + list(right.cache_rows)
        self.state_specs = list(left.state_specs) + list(right.state_specs)
        self._np, self._ns = len(left.cache_rows), len(left.state_specs)

    def __call__(self, h, batch, pools, states):
        a = self.left(h, batch, pools[:self._np], states[:self._ns])
        b = self.right(h, batch, pools[self._np:], states[self._ns:])
        return self.ops.rms_pair_mean(a, self.w_left, b, self.w_right, self.eps)


class MatrixLSTM:
    """Matrix memory with exponential gates (mLSTM).  The normaliser n rides along as one more column of the state: the values
    are extended by a column of ones, so S' = [S | n] [dim, vdim + pad] obeys the same recurrence and q reads S^T q and n . q
    in one go.  State per sequence: S' and the running maximum m per head."""

    def __init__(self, ops, *, heads, dim, vdim, gate_cap, eps, weights):
        """weights: q, k [H dim, D], v, g [H vdim, D], o [D, H vdim], norm [H vdim], i, f [H, D], i_b, f_b [H]."""
        self.ops, self.H, self.dim, self.vdim, self.cap, self.eps = ops, heads, dim, vdim, float(gate_cap), float(eps)
        w = weights
        D = w["q"].size(1)
        _check(w, {"q": (heads * dim, D), "k": (heads * dim, D), "v": (heads * vdim, D), "g": (heads * vdim, D), "o": (D, heads * vdim),
                   "norm": (heads * vdim,), "i": (heads, D), "f": (heads, D), "i_b": (heads,), "f_b": (heads,)}, "matrix LSTM")
        if self.cap <= 0.0:
            raise ValueError(f"matrix LSTM: gate cap {gate_cap}")
        self.w_in = torch.cat([w["q"], w["k"], w["v"], w["g"], w["i"], w["f"]], dim=0).contiguous()
        self.b_i, self.b_f = w["i_b"].float().contiguous(), w["f_b"].float().contiguous()
        self.norm, self.w_o = w["norm"].contiguous(), w["o"].contiguous()
        self.cols = vdim + (4 if vdim % 4 == 0 else 1)             # (a multiple of four keeps the kernels' 16-byte accesses)
        self.cache_rows, self.state_specs = [], [StateSpec((heads, dim, self.cols)), StateSpec((heads,))]

    def __call__(self, h, batch, pools, states, carry=None):
        ops, H, d, dv = self.ops, self.H, self.dim, self.vdim
        proj = linear(h, self.w_in)
        o_k, o_v, o_g, o_i = H * d, 2 * H * d, 2 * H * d + H * dv, 2 * H * d + 2 * H * dv
        a, b, m = ops.max_gates(proj, o_i, o_i + H, self.b_i, self.b_f, self.cap, states[1], batch, H)
        o = ops.recurrent_scan(proj[:, :o_k], proj[:, o_k:o_v], proj[:, o_v:o_g], a, None, states[0], batch, H, H, d, self.cols,
                               d ** -0.5, kscale=b, v_cols=dv)
        return linear(ops.head_rms_gate(o, self.norm, proj[:, o_g:o_i], "sigmoid", self.eps, vdim=dv, den_m=m), self.w_o)


class MinGRU:
    """A gated recurrence whose gates read only the current token (minGRU): element by element S <- (1 - z) S + z c with the
    gate z = sigmoid(W_z h + b_z) and the candidate c = u + 1/2 where u = W_x h + b_x >= 0, sigmoid(u) below; the output is
    W_o (S * silu(W_g h)).  State per sequence: S, float [width], from zero."""

    def __init__(self, ops, *, width, weights):
        """weights: z, x, g [width, D], z_b, x_b [width], o [D, width]."""
        self.ops, self.width = ops, int(width)
        w = weights
        D = w["z"].size(1)
        _check(w, {"z": (width, D), "x": (width, D), "g": (width, D), "z_b": (width,), "x_b": (width,), "o": (D, width)}, "minGRU")
        self.w_in = torch.cat([w["z"], w["x"], w["g"]], dim=0).contiguous()
        self.b_z, self.b_x, self.w_o = w["z_b"].contiguous(), w["x_b"].contiguous(), w["o"].contiguous()
        self.cache_rows, self.state_specs = [], [StateSpec((self.width,))]

    def __call__(self, h, batch, pools, states, carry=None):
        n = self.width
        proj = linear(h, self.w_in)
        return linear(self.ops.min_gru_scan(proj, 0, n, 2 * n, self.b_z, self.b_x, states[0], batch, n), self.w_o)
