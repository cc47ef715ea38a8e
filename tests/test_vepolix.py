"""The Vepolix model and its mechanisms through the serving engine against the plain float64 oracle (tests/_vepolix_plain.py).

Every test runs with the unfused tensor-op backend on the CPU (host logic: pages, state rows, runs, the layers' composition)
and, marked `gpu`, with the HIP kernels.  Configurations and weights are made here: small, random, sizes unlike each other so
that a mixed-up dimension shows; where random weights would hide a fault (one key among hundreds, a chunk's edge, a state
that is lost, a stale slot) the weights or inputs are made so that it shows.
"""
import json
import math
import os
import subprocess
import sys

import pytest
import torch

import _vepolix_plain as P
from qserve_amd.layers.moe import CorrectedSigmoidMoE, GatedFeedForward
from qserve_amd.layers.ops import make_ops
from qserve_amd.layers.softmax_attention import NormedChunkAttention, distance_bias_table, distance_bucket
from qserve_amd.models.vepolix import Vepolix
from qserve_amd.serving import Engine, SamplingParams
from qserve_amd.serving.cache import CacheFull, PagedCache
from qserve_amd.serving.engine import StepBatch

BACKENDS = [pytest.param("unfused", id="unfused-cpu"), pytest.param("hip", marks=pytest.mark.gpu, id="hip")]
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(params=BACKENDS)
def backend(request):
    if request.param == "hip" and not torch.cuda.is_available():
        pytest.skip("no GPU")
    return request.param


def device_of(backend):
    return "cuda:0" if backend == "hip" else "cpu"


def att(heads=4, kv_heads=2, dim=12, vdim=8, chunk=20, rows=10, far=40, scale=None, v_mix=False, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "bias_max": far, "rel_rows": rows, "v_mix": v_mix,
         "scale": scale if scale is not None else 1.0 / math.sqrt(dim)}
    if chunk:
        m["mask"] = {"size": chunk}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def lstm(heads=3, dim=8, vdim=12, cap=10.0, mlp=None):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}, "mlp": mlp}


def dense(ff=28):
    return {"kind": "dense", "ff": ff}


def moe(experts=6, top=2, ff=9, groups=3, keep=2, scale=1.7, shared=11):
    m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "scale": scale,
                                                         "groups": {"count": groups, "keep": keep}}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def make_config(layers, width=40, vocab=53, eps=1e-5, scale=3.0):
    return {"architecture": "Vepolix", "width": width, "vocab": vocab, "embedding": {"scale": scale}, "norm": {"eps": eps},
            "layers": layers}


def standard_config():
    return make_config([att(v_mix=True, mlp=dense()), lstm(mlp=moe()), att(heads=2, kv_heads=2, dim=6, vdim=8, chunk=33, rows=8, far=30),
                        att(heads=6, kv_heads=2, dim=5, vdim=8, chunk=7, rows=6, far=5, v_mix=True, mlp=moe(experts=4, top=3, groups=1, keep=1, shared=None)),
                        lstm(heads=2, dim=5, vdim=7, cap=4.0, mlp=dense(13)), att(v_mix=True, chunk=None, rows=12, far=70)])


def f32(W):
    return {k: (v.float() if v.is_floating_point() else v) for k, v in W.items()}


def build_engine(cfg, W, backend, dtype="float32", max_tokens=1024, max_seqs=4, **kw):
    return Engine(Vepolix, cfg, W, dtype=dtype, device=device_of(backend), max_tokens=max_tokens, max_seqs=max_seqs,
                  backend=backend, **kw)


def tokens_for(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


def run_schedule(eng, seqs, steps):
    """seqs: {name: tokens}; steps: [[(name, count), ...]] -> {name: logits [len, vocab]}; a sequence is closed after its last token."""
    at, slots, got = {k: 0 for k in seqs}, {}, {k: [] for k in seqs}
    for step in steps:
        items, want, n = [], [], 0
        for name, count in step:
            if name not in slots:
                slots[name] = eng.open_sequence()
            items.append((slots[name], seqs[name][at[name]:at[name] + count]))
            want += range(n, n + count)
            n += count
        logits = eng.execute(items, want).double().cpu()
        n = 0
        for name, count in step:
            got[name].append(logits[n:n + count])
            n += count
            at[name] += count
            if at[name] == len(seqs[name]):
                eng.close_sequence(slots.pop(name))
    return {k: torch.cat(v) for k, v in got.items() if v}


def assert_close(got, ref, tol, what=""):
    err = (got - ref).abs().max().item()
    scale = max(1.0, ref.abs().max().item())
    assert err <= tol * scale, f"{what}: max error {err:.3e} (allowed {tol * scale:.3e})"


F32_TOL = 2e-4      # float32 runs of a whole model against float64 (a fault shows at 1e-2 and above)


# ---- mechanisms alone ---------------------------------------------------------------------------------------------------------

def test_distance_buckets_and_the_bias_table():
    for rows, far in ((10, 40), (32, 128), (8, 16), (6, 5), (16, 32), (12, 70), (4, 1000), (16, 72)):
        half = rows // 2
        got = [distance_bucket(n, rows, far) for n in range(far + 50)]
        assert got[:half] == list(range(half)) and got[half] == half and max(got) == rows - 1 and got[far] == rows - 1
        assert all(b >= a for a, b in zip(got, got[1:]))
        for n in range(far + 50):
            ref = P.distance_bucket(n, rows, far)
            if got[n] != ref:           # only where the logarithm lands on an integer and floating point falls short of it
                x = math.log(n / half) / math.log(far / half) * (rows - half)
                assert abs(x - round(x)) < 1e-9 and got[n] == half + round(x), (rows, far, n)
    # (16, 32): the distance 16 = 8 * 4^(4 / 8) sits exactly on a row's edge and belongs to the upper row; (16, 72): 24 = 8 * 9^(4 / 8)
    assert distance_bucket(16, 16, 32) == 8 + 4 and distance_bucket(15, 16, 32) == 8 + 3
    assert distance_bucket(24, 16, 72) == 8 + 4 and distance_bucket(23, 16, 72) == 8 + 3
    rel = torch.arange(10 * 3, dtype=torch.float32).view(10, 3)
    t = distance_bias_table(rel, 40, 41)
    assert t.shape == (3, 41) and t[1, 3] == rel[3, 1] and t[2, 40] == rel[9, 2] and t[0, 7] == rel[P.distance_bucket(7, 10, 40), 0]


def test_sinusoid_embedding_and_rms_norms(backend):
    from qserve_amd.models.vepolix import sinusoid_frequencies
    dev = device_of(backend)
    ops = make_ops(backend, torch.float32, dev)
    g = torch.Generator().manual_seed(0)
    for D, V in ((7, 5), (40, 11), (300, 3)):
        table = torch.randn(V, D, generator=g)
        pos = torch.tensor([0, 1, 2, 63, 64, 500, 1499, 3], dtype=torch.int32)
        tok = torch.randint(0, V, (pos.numel(),), generator=g, dtype=torch.int32)
        x = ops.embed_sinusoid(tok.to(dev), pos.to(dev), table.to(dev), sinusoid_frequencies(D).to(dev), 2.5)
        ref = table[tok.long()].double() * 2.5 + P.sinusoid(1500, D)[pos.long()]
        assert_close(x.double().cpu(), ref, 2e-4, f"embedding, width {D}")          # (float angles: 1499 * 6e-8 relative)
        assert_close(x[:3].double().cpu(), ref[:3], 2e-6, "embedding, first positions")
        a, b, c, w = (torch.randn(pos.numel(), D, generator=g) for _ in range(3)), None, None, torch.randn(D, generator=g)
        a, b, c = a
        for ys in ([], [a], [a, b], [a, b, c]):
            xd = x.clone()
            h = ops.add_rms_norm(xd, [y.to(dev) for y in ys], w.to(dev), 1e-3)
            want = x.double().cpu() + sum(y.double() for y in ys) if ys else x.double().cpu()
            assert_close(xd.double().cpu(), want, 2e-6, "residual sum")
            assert_close(h.double().cpu(), P.rms(want, 1e-3) * w.double(), 2e-6, "norm of the sum")
            assert ops.add_rms_norm(xd, [y.to(dev) for y in ys], None, 1e-3) is None
        rows = torch.tensor([7, 0, 4], dtype=torch.int32)
        out = ops.rms_norm_rows(x, rows.to(dev), w.to(dev), 1e-5)
        assert_close(out.double().cpu(), P.rms(x.double().cpu()[rows.long()], 1e-5) * w.double(), 2e-6, "norm of chosen rows")


def _one_layer_engine(layer, backend, width=24, seed=3, max_tokens=256, max_seqs=3, dtype="float32"):
    cfg = make_config([layer], width=width)
    W = P.random_weights(cfg, seed=seed)
    Wd = f32(W) if dtype == "float32" else {k: v.bfloat16() for k, v in W.items()}
    return cfg, W, build_engine(cfg, Wd, backend, dtype=dtype, max_tokens=max_tokens, max_seqs=max_seqs)


def _plain_mixer(layer, h, W, cfg, v_first=None):
    if layer["type"] == "attention":
        return P.chunked_attention(h, W, "l0.mix.", layer["mixer"], cfg["norm"]["eps"], v_first)[0]
    return P.mlstm(h, W, "l0.mix.", layer["mixer"], cfg["norm"]["eps"])


def _mixer_alone(backend, layer, T, splits, seed=3, width=24, tol=2e-5, dtype="float32"):
    """One mixer through its layer object, the engine's cache and state, the tokens cut at `splits`, against the oracle."""
    cfg, W, eng = _one_layer_engine(layer, backend, width=width, seed=seed, dtype=dtype, max_tokens=max(256, T + 64))
    if dtype != "float32":
        W = {k: v.bfloat16().double() for k, v in W.items()}
    dev, st = eng.device, torch.float32 if dtype == "float32" else torch.bfloat16
    mixer = eng.model.layers[0]["mixer"]
    p0, p1, s0, s1 = eng.model.slices[0]
    g = torch.Generator().manual_seed(seed + 100)
    h = torch.randn(T, width, generator=g).bfloat16().float()
    ref = _plain_mixer(layer, h.double(), W, cfg)
    eng.open_sequence()                                                    # (not slot 0)
    slot = eng.open_sequence()
    for s in eng.cache.states:
        s.fill_(5.0)                                                       # stale state: a new sequence must not read it
    outs, lo = [], 0
    for hi in list(splits) + [T]:
        b = eng.layout([(slot, [0] * (hi - lo))])
        outs.append(mixer(h[lo:hi].to(st).to(dev), b, eng.cache.pools[p0:p1], eng.cache.states[s0:s1], {}).double().cpu())
        lo = hi
    assert_close(torch.cat(outs), ref, tol, f"{layer['type']} cut at {splits}")


def test_chunked_attention_alone(backend):
    _mixer_alone(backend, att(), 70, [])
    _mixer_alone(backend, att(), 70, [1, 3, 19, 20, 21, 40, 69])                         # cuts at and around the chunks' edges
    _mixer_alone(backend, att(heads=6, kv_heads=1, dim=5, vdim=3, chunk=64, rows=4, far=9), 150, [63, 64, 65, 129])   # chunk = page
    _mixer_alone(backend, att(heads=2, kv_heads=2, dim=16, vdim=24, chunk=70, rows=16, far=64), 160, [2, 69, 71, 139, 141])
    _mixer_alone(backend, att(heads=3, kv_heads=3, dim=4, vdim=4, chunk=1, rows=2, far=3), 9, [4])          # every token alone
    _mixer_alone(backend, att(chunk=None, rows=12, far=30), 100, [50, 99])                # no chunks: every earlier key, distances beyond `far`


@pytest.mark.gpu
def test_chunked_attention_on_the_matrix_cores():
    """bfloat16 storage with sizes the matrix-core kernel takes (prompt tiles, key splits over workgroups for single tokens)."""
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    for layer, T, splits in ((att(heads=4, kv_heads=2, dim=16, vdim=8, chunk=96, rows=10, far=60), 300, [95, 96, 97, 200, 298, 299]),
                             (att(heads=8, kv_heads=4, dim=40, vdim=24, chunk=200, rows=20, far=150), 420, [399, 400, 401, 419]),
                             (att(heads=5, kv_heads=1, dim=8, vdim=16, chunk=None, rows=8, far=500), 700, [650] + list(range(690, 700)))):
        _mixer_alone("hip", layer, T, splits, dtype="bfloat16", tol=2e-2, width=32)


def test_matrix_lstm_alone(backend):
    _mixer_alone(backend, lstm(), 40, [])
    _mixer_alone(backend, lstm(), 40, [1, 3, 17, 18, 39])
    _mixer_alone(backend, lstm(heads=1, dim=40, vdim=70, cap=30.0), 21, [2, 4])            # a column split over several lanes, two column blocks
    _mixer_alone(backend, lstm(heads=5, dim=3, vdim=2, cap=1.0), 9, [8])
    _mixer_alone(backend, lstm(heads=2, dim=16, vdim=16, cap=6.0), 200, [15, 31, 48, 81, 145, 146])   # gate scans of 64 and the staging of 16 at their edges


def test_exponential_gates_stay_in_range(backend):
    """Input gates far above the forget gates' reach and back: exp(i) alone would overflow a float; with the running maximum the
    state keeps its scale, and the maximum starts at 0 (a first input gate below 0 is weighed against exp(0))."""
    dev = device_of(backend)
    ops = make_ops(backend, torch.float32, dev)
    H, T, cap = 2, 150, 120.0
    g = torch.Generator().manual_seed(4)
    zi = torch.randn(T, H, generator=g) * 3.0
    zi[0] = -4.0
    zi[40:45] = 300.0
    zi[46:] -= 30.0
    zf = torch.randn(T, H, generator=g) * 2.0 + 1.0
    proj = torch.cat([zi, zf], dim=1).contiguous()
    bi, bf = torch.tensor([0.5, -0.5]), torch.tensor([1.0, 2.0])
    li = cap * torch.tanh((zi.double() + bi.double()) / cap)
    lf = torch.nn.functional.logsigmoid(cap * torch.tanh((zf.double() + bf.double()) / cap))
    m_ref, a_ref, b_ref, prev = [], [], [], torch.zeros(H, dtype=torch.float64)
    for t in range(T):
        m = torch.maximum(lf[t] + prev, li[t])
        a_ref.append(torch.exp(lf[t] + prev - m)), b_ref.append(torch.exp(li[t] - m)), m_ref.append(m)
        prev = m
    assert float(m_ref[0].min()) > -3.0 and float(torch.stack(m_ref).max()) > 100.0
    from qserve_amd.serving.cache import StateSpec
    cache = PagedCache([], 4, 3, torch.float32, dev, states=[StateSpec((H,))])
    cache.states[0].fill_(55.0)
    slot, lo = 2, 0
    a, b, m = [], [], []
    for hi in (1, 64, 65, 129, T):
        n = hi - lo
        batch = StepBatch(tokens=None, seq=None, pos=torch.arange(lo, hi, dtype=torch.int32, device=dev), slot=None, block_table=None,
                          max_pos=hi - 1, n_tokens=n, items=[(slot, 0, n)])
        out = ops.max_gates(proj[lo:hi].contiguous().to(dev), 0, H, bi.to(dev), bf.to(dev), cap, cache.states[0], batch, H)
        a.append(out[0].cpu()), b.append(out[1].cpu()), m.append(out[2].cpu())
        lo = hi
    assert_close(torch.cat(m).double(), torch.stack(m_ref), 1e-6, "running maximum")
    assert_close(torch.cat(a).double(), torch.stack(a_ref), 1e-4, "decay")
    assert_close(torch.cat(b).double(), torch.stack(b_ref), 1e-4, "input scale")
    assert float(cache.states[0][0].min()) == 55.0 and abs(float(cache.states[0][slot, 0]) - float(m_ref[-1][0])) < 1e-4


def _router_case(g, E, D, T, spread=1.0):
    return torch.randn(T, D, generator=g), {"p.router": torch.randn(E, D, generator=g).double() * 0.6,
                                            "p.correction": torch.randn(E, generator=g).double() * spread}


def test_corrected_router_alone(backend):
    dev = device_of(backend)
    ops = make_ops(backend, torch.float32, dev)
    g = torch.Generator().manual_seed(11)
    for E, groups, keep, top, D, T, spread in ((6, 3, 2, 2, 40, 33, 0.3), (12, 4, 3, 5, 24, 50, 0.3), (8, 1, 1, 8, 16, 5, 1.0),
                                               (9, 9, 4, 4, 20, 30, 0.5), (10, 2, 1, 5, 72, 20, 3.0), (64, 8, 3, 6, 32, 40, 0.2)):
        h, W = _router_case(g, E, D, T, spread)
        r = {"top": top, "scale": 1.9, "groups": {"count": groups, "keep": keep}}
        idx, wt = ops.moe_route(h.to(dev), W["p.router"].float().to(dev), top, groups, keep, score="sigmoid",
                                correction=W["p.correction"].float().to(dev), group_top=2, scale=1.9)
        ridx, rwt = P.route(h.double(), W, "p.", r)
        order = idx.cpu().long().argsort(dim=1), ridx.argsort(dim=1)
        assert torch.equal(idx.cpu().long().gather(1, order[0]), ridx.gather(1, order[1])), f"experts chosen, E={E}"
        assert_close(wt.cpu().double().gather(1, order[0]), rwt.gather(1, order[1]), 2e-6, "weights: plain scores times the scale")


def test_the_correction_moves_the_choice_not_the_weights(backend):
    dev = device_of(backend)
    ops = make_ops(backend, torch.float32, dev)
    h = torch.zeros(1, 8)
    h[0, 0] = 1.0
    Wr = torch.zeros(6, 8)
    Wr[:, 0] = torch.tensor([2.0, 1.0, -1.0, 0.0, 3.0, -3.0])                 # sigmoid: .88 .73 .27 .5 .95 .05
    none = torch.zeros(6)
    idx, wt = ops.moe_route(h.to(dev), Wr.to(dev), 2, 1, 1, score="sigmoid", correction=none.to(dev), group_top=2, scale=1.0)
    assert sorted(idx[0].tolist()) == [0, 4]
    corr = torch.tensor([0.0, 0.0, 5.0, 0.0, -5.0, 0.0])
    idx, wt = ops.moe_route(h.to(dev), Wr.to(dev), 2, 1, 1, score="sigmoid", correction=corr.to(dev), group_top=2, scale=3.0)
    assert sorted(idx[0].tolist()) == [0, 2]
    w = dict(zip(idx[0].tolist(), wt[0].tolist()))
    assert abs(w[2] - 3.0 / (1.0 + math.e)) < 1e-6 and abs(w[0] - 3.0 / (1.0 + math.exp(-2.0))) < 1e-6
    # groups of two: (0, 1) sums 1.61, (2, 3) 0.77, (4, 5) 1.0 - by its largest member alone the last group would be second
    idx, _ = ops.moe_route(h.to(dev), Wr.to(dev), 2, 3, 1, score="sigmoid", correction=none.to(dev), group_top=2, scale=1.0)
    assert sorted(idx[0].tolist()) == [0, 1]
    far = torch.tensor([-9.0, -9.0, 0.0, 0.0, -9.5, 0.0])                    # group scores -16.4, .77, -8.5: groups 1 and 2 are kept
    idx, _ = ops.moe_route(h.to(dev), Wr.to(dev), 3, 3, 2, score="sigmoid", correction=far.to(dev), group_top=2, scale=1.0)
    assert sorted(idx[0].tolist()) == [2, 3, 5]
    # all corrected scores negative: an expert outside the kept groups is not chosen although its score is the largest of all that
    # are left (a mask of zeros instead of minus infinity would choose it)
    neg = torch.tensor([-3.0, -9.0, -2.0, -2.0, -2.0, -2.0])                 # groups: -10.4, -3.2, -3.0; kept: 2 and 1
    Wr2 = torch.zeros(6, 8)
    idx, _ = ops.moe_route(h.to(dev), Wr2.to(dev), 4, 3, 2, score="sigmoid", correction=neg.to(dev), group_top=2, scale=1.0)
    assert sorted(idx[0].tolist()) == [2, 3, 4, 5]


def test_feed_forwards_alone(backend):
    dev = device_of(backend)
    ops = make_ops(backend, torch.float32, dev)
    g = torch.Generator().manual_seed(2)
    h = torch.randn(9, 24, generator=g) * 2
    W = {k: torch.randn(s, generator=g).double() / 4 for k, s in (("p.gate", (14, 24)), ("p.up", (14, 24)), ("p.down", (24, 14)))}
    for act, fn in (("gelu_tanh", P.gelu_tanh), ("silu", P.silu)):
        layer = GatedFeedForward(ops, gate=W["p.gate"].float().to(dev), up=W["p.up"].float().to(dev), down=W["p.down"].float().to(dev), act=act)
        assert_close(layer(h.to(dev)).double().cpu(), P.gated_unit(h.double(), W, "p.", fn), 1e-5, act)
    z = torch.linspace(-6, 6, 41, dtype=torch.float64)
    assert_close(P.gelu_tanh(z), torch.nn.functional.gelu(z, approximate="tanh"), 1e-12)
    for E, groups, keep, top, ff, D, T, shared in ((6, 3, 2, 2, 9, 40, 33, 11), (12, 4, 3, 2, 24, 72, 33, 0), (4, 1, 1, 4, 10, 36, 2, 5),
                                                   (8, 4, 2, 2, 16, 64, 90, 32)):
        hh, W = _router_case(g, E, D, T, 0.3)
        names = [f"e{e}." for e in range(E)] + (["shared."] if shared else [])
        for n in names:
            f = shared if n == "shared." else ff
            W[f"p.{n}gate"], W[f"p.{n}up"] = (torch.randn(f, D, generator=g).double() / math.sqrt(D) for _ in range(2))
            W[f"p.{n}down"] = torch.randn(D, f, generator=g).double() / math.sqrt(f)
        mlp = {"router": {"top": top, "scale": 1.3, "groups": {"count": groups, "keep": keep}}, "shared": {"ff": shared} if shared else None}
        sh = GatedFeedForward(ops, **{k: W[f"p.shared.{k}"].float().to(dev) for k in ("gate", "up", "down")}) if shared else None
        layer = CorrectedSigmoidMoE(ops, router=W["p.router"].float().to(dev), correction=W["p.correction"].float().to(dev),
                                    gate=[W[f"p.e{e}.gate"].float().to(dev) for e in range(E)], up=[W[f"p.e{e}.up"].float().to(dev) for e in range(E)],
                                    down=[W[f"p.e{e}.down"].float().to(dev) for e in range(E)], top_k=top, groups=groups, keep=keep, scale=1.3, shared=sh)
        ys = layer(hh.to(dev))
        assert len(ys) == (2 if shared else 1)
        assert_close(sum(y.double().cpu() for y in ys), P.moe(hh.double(), W, "p.", mlp), 1e-5, f"experts E={E}")


# ---- faults that random weights would hide ---------------------------------------------------------------------------------------

def _selector_attention(backend, L, spike, dtype, nq, chunk, bias_at=None):
    """Attention alone with selector weights: the layer input IS [q | k | v], the norms leave directions alone.  All keys are
    small but the one at `spike`; the queries point there.  -> (layer output of the last nq positions, oracle, h)."""
    H, G, d, dv = 2, 1, 8, 8
    m = {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "scale": 6.0, "bias_max": 20, "mask": {"size": chunk}}
    D = H * d + d + dv
    eye = torch.eye(D, dtype=torch.float64)
    rel = torch.zeros(6, H, dtype=torch.float64)
    if bias_at is not None:
        rel[bias_at] = 14.0
    W = {"p.q": eye[:16], "p.k": eye[16:24], "p.v": eye[24:32], "p.o": eye[:, :16].contiguous(), "p.q.norm": torch.ones(16, dtype=torch.float64),
         "p.k.norm": torch.ones(8, dtype=torch.float64), "p.rel": rel}
    g = torch.Generator().manual_seed((spike or 0) * 7 + L)
    h = (torch.randn(L, D, generator=g) * 0.05).bfloat16().double()
    h[:, 24:32] = torch.randn(L, dv, generator=g).bfloat16().double()
    if spike is not None:
        h[spike, 16 + 7] = 4.0                                               # a key eight times the others (after the norm: ~2.8 against ~0.3)
    if bias_at is not None:
        h[:, :24] = 0.0                                                      # every key the same, off the queries' direction: the bias alone decides
        h[:, 16] = 3.0
    h[:, 7] = 2.0
    h[:, 8 + 7] = 2.0
    ref = P.chunked_attention(h, W, "p.", m, 1e-5)[0]
    dev = device_of(backend)
    ops = make_ops(backend, dtype, dev)
    page, npages = 64, (L + 63) // 64
    cache = PagedCache([(G, dv + d)], npages + 3, 2, dtype, dev, page=page)
    cache.free_pages = torch.randperm(npages + 3, generator=g).tolist()     # pages out of order, not the first ones
    cache.admit()
    slot = cache.admit()
    layer = NormedChunkAttention(ops, heads=H, kv_heads=G, dim=d, vdim=dv, scale=6.0, eps=1e-5, chunk=chunk, bias_far=20,
                                 weights={k[2:].replace(".", "_"): v.to(dtype).to(dev) for k, v in W.items()})
    out = None
    for lo, hi in ((0, L - nq), (L - nq, L)):
        rows = cache.extend(slot, hi - lo)
        b = StepBatch(tokens=None, seq=torch.full((hi - lo,), slot, dtype=torch.int32, device=dev),
                      pos=torch.arange(lo, hi, dtype=torch.int32, device=dev), slot=torch.tensor(rows, dtype=torch.int64, device=dev),
                      block_table=cache.block_table(), max_pos=hi - 1, n_tokens=hi - lo, items=[(slot, 0, hi - lo)])
        out = layer(h[lo:hi].to(dtype).to(dev), b, cache.pools, [], {})
    return out.double().cpu(), ref[L - nq:], h


STORAGE = [pytest.param(torch.float32, 2e-5, id="float32"), pytest.param(torch.bfloat16, 3e-2, id="bfloat16")]


@pytest.mark.parametrize("dtype,tol", STORAGE)
@pytest.mark.parametrize("nq", [1, 3], ids=["decoded", "prompt"])
def test_keys_at_chunk_edges_and_page_borders_stand_out(backend, nq, dtype, tol):
    """Chunks of 200 positions, a sequence of 330: the last queries see [200, 330).  A loud key just inside (200, 201) carries the
    output; just outside (199, 198) or far back (0, 64) it must not be heard at all."""
    L, chunk = 330, 200
    for spike in (0, 64, 198, 199, 200, 201, 255, 256, 257, L - 4, L - 1):
        out, ref, h = _selector_attention(backend, L, spike, dtype, nq, chunk)
        if 200 <= spike < L - 3:
            assert (ref[-1, :8] - h[spike, 24:32]).abs().max() < 0.15, f"the key at {spike} should carry the output"
        if spike < 200:
            assert (ref[-1, :8] - h[spike, 24:32]).abs().max() > 0.3, f"the key at {spike} lies outside the chunk"
        assert_close(out, ref, tol, f"spike at {spike}")
    # the same at a chunk's edge that is no page's edge and with the queries in the chunk's first positions
    for L2, spike in ((203, 199), (203, 200), (201, 199), (201, 200), (400, 399), (401, 399), (401, 400)):
        out, ref, _ = _selector_attention(backend, L2, spike, dtype, 1, chunk)
        assert_close(out, ref, tol, f"length {L2}, spike at {spike}")


@pytest.mark.parametrize("dtype,tol", STORAGE)
def test_the_distance_bias_picks_its_bucket(backend, dtype, tol):
    """Quiet keys, one loud row of the bias table: the output is the value at that distance (rows 0 - 2: the distance itself; row 3:
    distances 3 - 5 of a 6-row table that ends at 20; row 5: everything from 11 on)."""
    L = 90
    for row, dists in ((0, [0]), (2, [2]), (3, [3, 4, 5]), (5, list(range(11, 90)))):
        out, ref, h = _selector_attention(backend, L, None, dtype, 2, 500, bias_at=row)
        want = h[[L - 1 - d_ for d_ in dists], 24:32].mean(0)
        assert (ref[-1, :8] - want).abs().max() < 0.2, f"bias row {row}"
        assert_close(out, ref, tol, f"bias row {row}")


def test_a_far_write_stays_in_the_matrix_memory(backend):
    """Forget gates at their cap and one early token with a large input gate and value: hundreds of tokens later the read-out is
    still that token's.  Cut into steps, so a state that is dropped, zeroed or taken from another slot shows."""
    layer = lstm(heads=2, dim=8, vdim=6, cap=13.0)
    cfg = make_config([layer], width=24)
    W = P.random_weights(cfg, seed=5)
    p = "l0.mix."
    W[p + "f.b"] = torch.full_like(W[p + "f.b"], 40.0)                       # logsigmoid(13 tanh(40 / 13)) = -2e-6 a token
    W[p + "f"] *= 0.0
    W[p + "i"] *= 0.0
    W[p + "i"][:, 0] = 8.0                                                   # the input gate follows input channel 0 alone
    W[p + "i.b"] = torch.zeros_like(W[p + "i.b"])
    eng = build_engine(cfg, f32(W), backend, max_tokens=512, max_seqs=3)
    mixer = eng.model.layers[0]["mixer"]
    T = 300
    g = torch.Generator().manual_seed(1)
    h = (torch.randn(T, 24, generator=g) * 0.3).bfloat16().float()
    h[:, 0], h[3, 0] = -1.0, 1.0                                             # exp(-8) for every token but the fourth, exp(8) for it
    h[3, 1:] *= 4.0
    Wd = {k: v.double() for k, v in W.items()}
    ref = P.mlstm(h.double(), Wd, p, layer["mixer"], 1e-5)
    quiet = h.clone()
    quiet[3] = h[4]
    without = P.mlstm(quiet.double(), Wd, p, layer["mixer"], 1e-5)
    assert (ref[-1] - without[-1]).abs().max() > 0.05 * ref[-1].abs().max()      # the far token still decides the last output
    eng.open_sequence()                                                       # the test's sequence does not sit in slot 0
    slot = eng.open_sequence()
    for s in eng.cache.states:
        s.fill_(7.0)                                                          # stale state everywhere: a new sequence must not read it
    outs, lo = [], 0
    for hi in (2, 5, 64, 65, 200, 299, 300):
        b = eng.layout([(slot, [0] * (hi - lo))])
        outs.append(mixer(h[lo:hi].to(eng.device), b, [], eng.cache.states, {}).double().cpu())
        lo = hi
    # (float states against float64: where the read-out nearly cancels, rounding shows at a few 1e-4; a lost state at 5e-2 and above)
    assert_close(torch.cat(outs), ref, 1e-3, "matrix memory: far write")


def test_blended_values_come_from_the_first_blending_layer(backend):
    """Three attention layers, the middle one outside the blend: the third takes the FIRST layer's own values (not the second's, not
    blended ones), and what it caches are the blended values - decoded tokens read them back."""
    cfg = make_config([att(v_mix=True), att(v_mix=False), att(v_mix=True)], width=24)
    W = P.random_weights(cfg, seed=8)
    W["l2.mix.vmix"] = torch.tensor(0.8, dtype=torch.float64)
    W["l0.mix.vmix"] = torch.tensor(0.9, dtype=torch.float64)               # (the first layer's own number is not used)
    toks = tokens_for(cfg, 50, 3)
    ref, _ = P.forward(cfg, W, toks)
    other = dict(W)
    other["l2.mix.vmix"] = torch.tensor(0.0, dtype=torch.float64)
    assert (P.forward(cfg, other, toks)[0] - ref).abs().max() > 1e-2        # the blend matters
    other = dict(W)
    other["l0.mix.vmix"] = torch.tensor(0.1, dtype=torch.float64)
    assert (P.forward(cfg, other, toks)[0] - ref).abs().max() == 0.0
    eng = build_engine(cfg, f32(W), backend)
    got = run_schedule(eng, {"s": toks}, [[("s", 30)], [("s", 15)]] + [[("s", 1)]] * 5)
    assert_close(got["s"], ref, F32_TOL, "blend over three layers")


# ---- whole model through the engine --------------------------------------------------------------------------------------------

@pytest.fixture(scope="module")
def std():
    cfg = standard_config()
    W = P.random_weights(cfg, seed=1)
    seqs = {"a": tokens_for(cfg, 150, 1), "b": tokens_for(cfg, 37, 2), "c": tokens_for(cfg, 1, 3), "d": tokens_for(cfg, 81, 4)}
    out = {k: P.forward(cfg, W, v) for k, v in seqs.items()}
    return cfg, W, seqs, {k: v[0] for k, v in out.items()}, {k: v[1] for k, v in out.items()}


def test_layers_one_by_one(backend, std):
    cfg, W, seqs, _, layers = std
    eng = build_engine(cfg, f32(W), backend)
    slot = eng.open_sequence()
    b = eng.layout([(slot, seqs["b"])])
    seen = []
    eng.model.forward(b, eng.cache.pools, states=eng.cache.states, tap=lambda i, x: seen.append(x.double().cpu().clone()))
    assert len(seen) == len(cfg["layers"])
    for i, x in enumerate(seen):
        assert_close(x, layers["b"][i], F32_TOL, f"residual stream after layer {i}")


def test_whole_prompts(backend, std):
    cfg, W, seqs, ref, _ = std
    eng = build_engine(cfg, f32(W), backend)
    for k in seqs:
        got = run_schedule(eng, seqs, [[(k, len(seqs[k]))]])
        assert_close(got[k], ref[k], F32_TOL, f"whole prompt {k}")


def test_prefill_then_token_by_token(backend, std):
    cfg, W, seqs, ref, _ = std
    eng = build_engine(cfg, f32(W), backend)
    for k, first in (("a", 60), ("b", 1), ("d", 64)):
        n = len(seqs[k])
        got = run_schedule(eng, seqs, [[(k, first)]] + [[(k, 1)]] * (n - first))
        assert_close(got[k], ref[k], F32_TOL, f"{k}: {first} tokens, then one by one")


def test_portions_of_several_sizes(backend, std):
    cfg, W, seqs, ref, _ = std
    eng = build_engine(cfg, f32(W), backend)
    for sizes in ([2] * 75, [64, 64, 22], [63, 2, 2, 61, 22], [3, 1, 1, 2, 5, 7, 45, 64, 1, 19, 2], [149, 1], [20, 13, 7, 26, 33, 51]):
        assert sum(sizes) == 150
        got = run_schedule(eng, seqs, [[("a", s)] for s in sizes])
        assert_close(got["a"], ref["a"], F32_TOL, f"portions {sizes[:6]}...")


def test_unequal_batches_match_each_alone(backend, std):
    cfg, W, seqs, ref, _ = std
    eng = build_engine(cfg, f32(W), backend)
    steps = [[("a", 29), ("b", 2), ("c", 1)],
             [("a", 64), ("b", 1), ("d", 17)],
             [("b", 30), ("d", 1), ("a", 2)],
             [("d", 63), ("a", 1), ("b", 1)]]
    steps += [[("a", 1), ("b", 1)]] * 3 + [[("a", 1)]] * 51
    got = run_schedule(eng, seqs, steps)
    for k in seqs:
        assert_close(got[k], ref[k], F32_TOL, f"mixed batch, sequence {k}")


def test_a_sequence_left_out_of_steps_goes_on_later(backend, std):
    cfg, W, seqs, ref, _ = std
    eng = build_engine(cfg, f32(W), backend)
    steps = [[("b", 10), ("d", 3)], [("d", 2)], [("d", 1)], [("b", 1), ("d", 1)], [("d", 70)], [("b", 26), ("d", 4)]]
    got = run_schedule(eng, seqs, steps)
    for k in ("b", "d"):
        assert_close(got[k], ref[k], F32_TOL, f"sequence {k}")


def test_pages_slots_and_states_are_used_again(backend, std):
    cfg, W, seqs, ref, _ = std
    eng = build_engine(cfg, f32(W), backend, max_tokens=256, max_seqs=2)          # 4 pages, 2 slots: a (3 pages) + one more
    assert eng.cache.num_pages == 4
    seen_pages = []
    for rnd in range(3):
        order = [("a", "b"), ("d", "b"), ("b", "a")][rnd]
        steps = [[(order[0], 30), (order[1], 5)], [(order[0], len(seqs[order[0]]) - 30), (order[1], len(seqs[order[1]]) - 5)]]
        got = run_schedule(eng, seqs, steps)
        for k in order:
            assert_close(got[k], ref[k], F32_TOL, f"round {rnd}, sequence {k}")
        assert len(eng.cache.free_pages) == 4 and len(eng.cache.free_slots) == 2
        seen_pages.append(tuple(eng.cache.free_pages))
        assert all(float(s.abs().max()) > 0 for s in eng.cache.states)            # the slots' states are left as they were: stale
    assert len(set(seen_pages)) > 1
    s0, s1 = eng.open_sequence(), eng.open_sequence()
    with pytest.raises(CacheFull):
        eng.open_sequence()
    eng.close_sequence(s0)
    eng.close_sequence(s1)


def test_first_tokens_and_single_token_sequences(backend, std):
    cfg, W, seqs, ref, _ = std
    eng = build_engine(cfg, f32(W), backend)
    got = run_schedule(eng, seqs, [[("c", 1)]])
    assert_close(got["c"], ref["c"], F32_TOL)
    got = run_schedule(eng, seqs, [[("b", 1)], [("b", 1)], [("b", 2)], [("b", 33)]])
    assert_close(got["b"][:4], ref["b"][:4], F32_TOL, "first tokens")


def test_long_decoding(backend):
    cfg = make_config([lstm(mlp=dense(12)), att(chunk=50, mlp=None, v_mix=True), lstm(heads=2, dim=4, vdim=4, mlp=moe(experts=4, top=1, groups=2, keep=1))],
                      width=32, vocab=29)
    W = P.random_weights(cfg, seed=9)
    toks = tokens_for(cfg, 210, 5)
    ref, _ = P.forward(cfg, W, toks)
    eng = build_engine(cfg, f32(W), backend, max_tokens=256, max_seqs=1)
    got = run_schedule(eng, {"s": toks}, [[("s", 3)]] + [[("s", 1)]] * 207)      # decoded tokens pass four chunk edges and three page borders
    assert_close(got["s"], ref, F32_TOL, "207 decoded tokens")


@pytest.mark.parametrize("variant", range(4))
def test_other_sizes(backend, variant):
    layers, kw = [
        ([lstm(heads=1, dim=2, vdim=2, cap=1.0, mlp=moe(experts=2, top=2, ff=1, groups=1, keep=1, shared=1))], dict(width=8, vocab=5, eps=1e-3)),
        ([att(heads=6, kv_heads=3, dim=16, vdim=24, chunk=31, rows=20, far=100, v_mix=True, mlp=moe(experts=9, top=5, ff=33, groups=3, keep=3)),
          lstm(heads=4, dim=32, vdim=16, mlp=dense(100)), att(heads=3, kv_heads=3, dim=8, vdim=24, chunk=64, v_mix=True, mlp=None)],
         dict(width=96, vocab=200, scale=0.5)),
        ([att(heads=2, kv_heads=2, dim=6, vdim=64, chunk=10, rows=2, far=2, mlp=None), lstm(heads=1, dim=70, vdim=5, cap=50.0)],
         dict(width=41, vocab=33, eps=1e-6)),
        ([lstm(mlp=dense(8)), lstm(mlp=moe(experts=8, top=3, groups=4, keep=2, scale=0.5)), att(heads=1, kv_heads=1, v_mix=True, mlp=None)],
         dict(width=48, vocab=61, scale=1.0)),
    ][variant]
    cfg = make_config(layers, **kw)
    W = P.random_weights(cfg, seed=20 + variant)
    toks = tokens_for(cfg, 75, variant)
    ref, _ = P.forward(cfg, W, toks)
    eng = build_engine(cfg, f32(W), backend)
    got = run_schedule(eng, {"s": toks}, [[("s", 40)], [("s", 30)]] + [[("s", 1)]] * 5)
    assert_close(got["s"], ref, F32_TOL, f"sizes variant {variant}")


def test_bfloat16_storage_stays_near_the_oracle(backend, std):
    cfg, W, seqs, ref, _ = std
    Wb = {k: v.bfloat16() for k, v in W.items()}
    exact = {k: P.forward(cfg, {n: v.double() for n, v in Wb.items()}, seqs[k])[0] for k in ("a", "b")}
    eng = build_engine(cfg, Wb, backend, dtype="bfloat16")
    got = run_schedule(eng, seqs, [[("a", 70), ("b", 37)], [("a", 80)]])
    for k in ("a", "b"):
        d = got[k] - exact[k]
        rel = (d - d.mean(-1, keepdim=True)).pow(2).mean().sqrt() / exact[k].std()
        assert rel < 0.1, f"bfloat16 run of {k}: relative error {rel:.3f}"
    got2 = run_schedule(eng, seqs, [[("a", 3)], [("a", 147)]])                      # cut differently: the same up to rounding
    rel = (got2["a"] - got["a"]).pow(2).mean().sqrt() / exact["a"].std()
    assert rel < 0.1


# ---- generation through the engine's own entry point and scheduler ---------------------------------------------------------------

def oracle_greedy(cfg, W, prompt, n):
    toks, margins = list(prompt), []
    for _ in range(n):
        lg = P.forward(cfg, W, toks)[0][-1]
        top2 = lg.topk(2).values
        margins.append(float(top2[0] - top2[1]))
        toks.append(int(lg.argmax()))
    return toks[len(prompt):], margins


def test_greedy_generation_through_the_scheduler(backend, std):
    cfg, W, _, _, _ = std
    prompts = [tokens_for(cfg, n, 40 + n) for n in (5, 70, 1, 33, 12, 64)]
    eng = build_engine(cfg, f32(W), backend, max_tokens=512, max_seqs=3, max_batch_tokens=48, prefill_chunk=20)
    outs = eng.generate(prompts, SamplingParams(max_new=6))
    assert not eng.has_work() and len(eng.cache.free_pages) == eng.cache.num_pages and len(eng.cache.free_slots) == 3
    for p, o in zip(prompts, outs):
        ref, margins = oracle_greedy(cfg, W, p, 6)
        for i, (a, b) in enumerate(zip(o, ref)):
            if a != b:
                assert margins[i] < 1e-3, f"prompt of {len(p)}: token {i} is {a}, oracle {b} (margin {margins[i]:.2e})"
                break
        else:
            assert len(o) == 6


def _save_model(tmp_path, cfg, W):
    from safetensors.torch import save_file
    cfg = json.loads(json.dumps(cfg))
    for L in cfg["layers"]:
        L["mixer"].pop("rel_rows", None)                                     # (this file's own key: a checkpoint gives it by the shape)
    with open(tmp_path / "config.json", "w") as f:
        json.dump(cfg, f)
    save_file({k: v.bfloat16().contiguous() for k, v in W.items()}, str(tmp_path / "model.safetensors"))


def test_registry_and_checkpoint_directory(tmp_path, backend, std):
    from qserve_amd.serving import registry
    assert registry.architectures()["Vepolix"] == "paged"
    cfg, W, seqs, _, _ = std
    _save_model(tmp_path, cfg, W)
    ref = P.forward(cfg, {k: v.bfloat16().double() for k, v in W.items()}, seqs["b"])[0]
    eng = Engine.from_pretrained(str(tmp_path), dtype="float32", device=device_of(backend), max_tokens=128, backend=backend)
    got = run_schedule(eng, seqs, [[("b", 37)]])
    assert_close(got["b"], ref, F32_TOL)
    bad = dict(cfg, layers=[dict(cfg["layers"][0], type="unknown")])
    with pytest.raises(ValueError):
        Vepolix.from_config(bad, f32(W), make_ops("unfused", torch.float32, "cpu"), "cpu", torch.float32)
    with pytest.raises(KeyError):
        Vepolix.from_config(cfg, {k: v for k, v in f32(W).items() if k != "l1.mix.f.b"}, make_ops("unfused", torch.float32, "cpu"), "cpu", torch.float32)


# ---- GPU only ---------------------------------------------------------------------------------------------------------------------

@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_replay_command(tmp_path, dtype, std):
    """bin/trace_run on a checkpoint directory: portions, single tokens, a mixed batch, a sequence ended and its slot used again."""
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    cfg, W, seqs, _, _ = std
    _save_model(tmp_path, cfg, W)
    Wb = {k: v.bfloat16().double() for k, v in W.items()}
    ref = {k: P.forward(cfg, Wb, seqs[k])[0] for k in ("a", "b", "d")}
    a, b, d = seqs["a"], seqs["b"], seqs["d"]
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:100], "want": [0, 99]}, {"id": "b", "tokens": b[:36], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "b", "tokens": b[36:], "want": [0]}, {"id": "a", "tokens": a[100:149], "want": [48]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": a[149:], "want": []}], "end": ["a"]},
             {"step": 3, "entries": [{"id": "d", "tokens": d, "want": [0, 80]}], "end": ["d"]}]
    out = tmp_path / "out"
    r = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", str(tmp_path), "--dtype", dtype, "--out", str(out),
                        "--max-tokens", "256", "--max-seqs", "2"], input="".join(json.dumps(s) + "\n" for s in steps), text=True,
                       capture_output=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [x for x in r.stdout.split("\n") if x.startswith("done")] == [f"done {i}" for i in range(4)]
    assert not (out / "2.f32").exists()
    import numpy as np
    V = cfg["vocab"]
    want = {0: torch.stack([ref["a"][0], ref["a"][99]]), 1: torch.stack([ref["b"][36], ref["a"][148]]), 3: torch.stack([ref["d"][0], ref["d"][80]])}
    for i, w in want.items():
        got = torch.from_numpy(np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, V)).double()
        if dtype == "float32":
            assert_close(got, w, F32_TOL, f"step {i}")
        else:
            dlt = got - w
            assert (dlt - dlt.mean(-1, keepdim=True)).pow(2).mean().sqrt() / w.std() < 0.1, f"step {i}"


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_steps_from_a_graph_match_eager_steps(dtype, std):
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    cfg, W, seqs, ref, _ = std
    Wd = f32(W) if dtype == "float32" else {k: v.bfloat16() for k, v in W.items()}
    tol = 2e-5 if dtype == "float32" else 3e-2
    engines = [build_engine(cfg, Wd, "hip", dtype=dtype, decode_graphs=g) for g in (False, True)]
    steps = [[("a", 100), ("b", 20)]] + [[("a", 1), ("b", 1)]] * 6 + [[("d", 30)]] + [[("a", 1), ("b", 1), ("d", 1)]] * 5 + \
            [[("b", 6), ("a", 1)]] + [[("a", 1), ("d", 1)]] * 8
    got = [run_schedule(e, seqs, steps) for e in engines]
    assert any(v is not False for v in engines[1]._graphs.values()), "no step was captured"
    for k in got[0]:
        assert_close(got[1][k], got[0][k], tol, f"graph against eager, sequence {k}")
        if dtype == "float32":
            assert_close(got[1][k], ref[k][:got[0][k].shape[0]], F32_TOL, f"graph against the oracle, sequence {k}")


@pytest.mark.gpu
@pytest.mark.parametrize("runs,heads,dim,vdim,cols", [(32, 4, 64, 128, 132), (8, 16, 64, 128, 132), (8, 32, 64, 128, 132), (3, 2, 64, 128, 132),
                                                      (32, 4, 32, 64, 68), (20, 8, 64, 128, 128)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
def test_scan_forms_at_launch_sizes_that_fill_the_chip(runs, heads, dim, vdim, cols, dtype):
    """The scan kernel picks its form (rows per lane, waves per SIMD, staging depth) from the number of workgroups a launch has;
    small models never reach the forms for full chips.  Runs of unequal lengths, some continuing a sequence, with one decay per
    head, a key scale and the column of ones, against the unfused statement of the same recurrence."""
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    dev = "cuda:0"
    g = torch.Generator().manual_seed(runs * 100 + heads)
    lens = [int(n) for n in torch.randint(1, 41, (runs,), generator=g)]
    lens[0], lens[-1] = 40, 17
    T = sum(lens)
    items, pos, at = [], [], 0
    for s, n in enumerate(lens):
        items.append((s, at, n))
        first = 0 if s % 3 else 5                                            # every third run continues a sequence
        pos += range(first, first + n)
        at += n
    pos = torch.tensor(pos, dtype=torch.int32, device=dev)
    batch = StepBatch(tokens=None, seq=None, pos=pos, slot=None, block_table=None, max_pos=int(pos.max()), n_tokens=T, items=items)
    proj = (torch.randn(T, 2 * heads * dim + heads * vdim, generator=g) * 0.5).to(dtype).to(dev)
    q, k, v = proj[:, :heads * dim], proj[:, heads * dim:2 * heads * dim], proj[:, 2 * heads * dim:]
    decay = (torch.rand(T, heads, generator=g) * 0.3 + 0.7).to(dev)
    ks = torch.rand(T, heads, generator=g).to(dev)
    state = torch.randn(runs, heads, dim, cols, generator=g).to(dev)
    kw = dict(kscale=ks, v_cols=vdim) if cols > vdim else {}
    outs = []
    for name in ("hip", "unfused"):
        st = state.clone()
        o = make_ops(name, dtype, dev).recurrent_scan(q, k, v, decay, None, st, batch, heads, heads, dim, cols, dim ** -0.5, **kw)
        outs.append((o.double().cpu(), st.double().cpu()))
    assert_close(outs[0][0], outs[1][0], 2e-5, "read-outs")
    assert_close(outs[0][1], outs[1][1], 2e-5, "states")
