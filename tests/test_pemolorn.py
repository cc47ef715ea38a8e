"""The Pemolorn model and its mechanisms through the serving engine against the plain float64 statement (tests/_pemolorn_plain.py).

Every test runs with the unfused tensor-op backend on the CPU (host logic: pages, block rows, state rows, runs, the layers'
composition) and, marked `gpu`, with the HIP kernels.  Configurations and weights are made here: small, random, sizes unlike each
other so that a mixed-up dimension shows; where random weights would hide a fault (one kept key among hundreds, a window's edge, a
block that is seen one token early, a sink that is left out, a state that is lost) the weights or inputs are made so that it shows.
"""
import json
import math
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import _pemolorn_plain as P
from qserve_amd.layers.moe import IdentityExpertMoE, ReluSquaredFeedForward
from qserve_amd.layers.ops import make_ops
from qserve_amd.layers.recurrent import MinGRU
from qserve_amd.layers.rotary import RotaryTable
from qserve_amd.layers.softmax_attention import SinkWindowAttention
from qserve_amd.models.pemolorn import Pemolorn
from qserve_amd.serving import Engine, SamplingParams
from qserve_amd.serving.cache import CacheFull, PagedCache, StateSpec
from qserve_amd.serving.engine import StepBatch

BACKENDS = [pytest.param("unfused", id="unfused-cpu"), pytest.param("hip", marks=pytest.mark.gpu, id="hip")]
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
STORAGE = [pytest.param(torch.float32, 2e-5, id="float32"), pytest.param(torch.bfloat16, 3e-2, id="bfloat16")]


@pytest.fixture(params=BACKENDS)
def backend(request):
    if request.param == "hip" and not torch.cuda.is_available():
        pytest.skip("no GPU")
    return request.param


def device_of(backend):
    return "cuda:0" if backend == "hip" else "cpu"


def att(heads=4, kv_heads=2, dim=12, vdim=8, size=24, keep=5, scale=None, kv_from=None, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": size, "keep_first": keep},
         "scale": scale if scale is not None else 1.0 / math.sqrt(dim)}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m, "mlp": mlp}


def par(heads=6, kv_heads=3, dim=8, vdim=10, size=17, pool=5, conv=3, rot=4, base=1000.0, width=28, scale=None, mlp=None):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv, "mask": {"size": size, "pool": pool},
            "rot": {"dims": rot, "base": base}, "scale": scale if scale is not None else 1.0 / math.sqrt(dim)}
    return {"type": "parallel", "mixer": {"left": left, "right": {"width": width}}, "mlp": mlp}


def dense(ff=28):
    return {"kind": "dense", "ff": ff}


def moe(experts=5, identity=2, top=3, ff=9, limit=0.8):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "identity": identity, "top": top}}


def make_config(layers, width=40, vocab=53, eps=1e-5):
    return {"architecture": "Pemolorn", "width": width, "vocab": vocab, "norm": {"eps": eps}, "layers": layers}


def standard_config():
    return make_config([par(mlp=moe()), att(mlp=dense()), att(heads=6, kv_heads=2, dim=12, vdim=8, size=70, keep=9, kv_from=1, mlp=moe(top=1)),
                        par(heads=2, kv_heads=1, dim=6, vdim=4, size=64, pool=64, conv=2, rot=6, width=40), att(size=9, keep=0, mlp=None),
                        att(size=31, keep=40, kv_from=4, mlp=moe(experts=3, identity=0, top=2, ff=12, limit=2.5))])


def t64(W):
    return {k: torch.from_numpy(np.asarray(v)) for k, v in W.items()}


def f32(W):
    return {k: v.float() for k, v in t64(W).items()}


def build_engine(cfg, W, backend, dtype="float32", max_tokens=1024, max_seqs=4, **kw):
    return Engine(Pemolorn, cfg, W, dtype=dtype, device=device_of(backend), max_tokens=max_tokens, max_seqs=max_seqs,
                  backend=backend, **kw)


def tokens_for(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


def plain_logits(cfg, W, toks, taps=None):
    return torch.from_numpy(P.forward(cfg, W, toks, taps))


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
    ref = torch.as_tensor(ref)
    err = (got - ref).abs().max().item()
    scale = max(1.0, ref.abs().max().item())
    assert err <= tol * scale, f"{what}: max error {err:.3e} (allowed {tol * scale:.3e})"


F32_TOL = 2e-4      # float32 runs of a whole model against float64 (a fault shows at 1e-2 and above)


def batch_for(cache, slot, lo, hi, dev):
    rows = cache.extend(slot, hi - lo)
    n = hi - lo
    return StepBatch(tokens=None, seq=torch.full((n,), slot, dtype=torch.int32, device=dev),
                     pos=torch.arange(lo, hi, dtype=torch.int32, device=dev), slot=torch.tensor(rows, dtype=torch.int64, device=dev),
                     block_table=cache.block_table(), max_pos=hi - 1, n_tokens=n, items=[(slot, 0, n)],
                     run_off=torch.arange(n, dtype=torch.int32, device=dev))


# ---- mechanisms alone ---------------------------------------------------------------------------------------------------------

def test_norms_around_a_sublayer(backend):
    dev = device_of(backend)
    ops = make_ops(backend, torch.float32, dev)
    g = torch.Generator().manual_seed(0)
    for D in (7, 40, 300, 1024 + 36):
        x = torch.randn(5, D, generator=g) * 3
        y = torch.randn(5, D, generator=g) * 0.01 + 2.0                     # a mean far from zero: RMS, not a variance
        for wide in (False, True):
            wp = torch.randn(D if wide else 1, generator=g)
            wn = torch.randn(D if wide else 1, generator=g)
            xd = x.clone().to(dev)
            h = ops.add_normed_rms_norm(xd, y.to(dev), wp.to(dev), wn.to(dev), 1e-2)
            want = x.double() + torch.from_numpy(P.rms(y.double().numpy(), 1e-2)) * wp.double()
            assert_close(xd.double().cpu(), want, 2e-6, f"stream + normed output, width {D}")
            assert_close(h.double().cpu(), torch.from_numpy(P.rms(want.numpy(), 1e-2)) * wn.double(), 2e-6, "norm of the new stream")
            assert ops.add_normed_rms_norm(xd, y.to(dev), wp.to(dev), None, 1e-2) is None
            x0 = x.clone().to(dev)
            h0 = ops.add_normed_rms_norm(x0, None, None, wn.to(dev), 1e-2)
            assert torch.equal(x0.cpu(), x)
            assert_close(h0.double().cpu(), torch.from_numpy(P.rms(x.double().numpy(), 1e-2)) * wn.double(), 2e-6, "norm alone")


def test_query_key_norms_and_rotated_pairs(backend):
    """Per-head norms with a shared weight and norms over the whole projection; the first `rot` dimensions of every head turn as
    neighbours, the rest pass; positions far from zero."""
    dev = device_of(backend)
    ops = make_ops(backend, torch.float32, dev)
    g = torch.Generator().manual_seed(1)
    for H, G, d, dv, rot, per_head in ((4, 2, 12, 8, 4, True), (6, 3, 8, 10, 8, False), (2, 1, 6, 4, 0, False), (3, 3, 16, 2, 6, True)):
        T, base = 6, 50.0
        pos = torch.tensor([0, 1, 63, 64, 700, 2], dtype=torch.int32)
        q, k, v = (torch.randn(T, n, generator=g) for n in (H * d, G * d, G * dv))
        qw, kw = (torch.randn(d if per_head else n * d, generator=g) for n in (H, G))
        table = RotaryTable(rot, base, None, dev, positions=701) if rot else None
        cache = PagedCache([(G, dv + d)], 12, 1, torch.float32, dev)
        slot = cache.admit()
        b = batch_for(cache, slot, 0, T, dev)
        b.pos, b.max_pos = pos.to(dev), 700
        qf = ops.qk_norm_rope_prep(q.to(dev), k.to(dev), v.to(dev), H, G, d, dv, qw.to(dev), kw.to(dev), per_head, 1e-4,
                                   table.table if rot else None, rot, 0.7, cache.pools[0], b)

        def plain(u, w, n):
            u = u.double().numpy()
            u = P.rms(u.reshape(T, n, d), 1e-4) * w.double().numpy() if per_head else (P.rms(u, 1e-4) * w.double().numpy()).reshape(T, n, d)
            return torch.from_numpy(P.rotate_pairs(u, pos.numpy(), rot, base) if rot else u)

        assert_close(qf[..., dv:].double().cpu(), plain(q, qw, H) * 0.7, 1e-5, "queries")
        assert float(qf[..., :dv].abs().max()) == 0.0
        rows = cache.pools[0][:, b.slot].transpose(0, 1).double().cpu()                        # [T, G, dv + d]
        assert_close(rows[..., dv:], plain(k, kw, G), 1e-5, "cached keys")
        assert torch.equal(rows[..., :dv].float(), v.view(T, G, dv))
        before = cache.pools[0].clone()
        ops.qk_norm_rope_prep(q.to(dev), None, None, H, G, d, dv, qw.to(dev), None, per_head, 1e-4, table.table if rot else None, rot,
                              0.7, None, b)
        assert torch.equal(before, cache.pools[0])                                             # a layer without keys writes nothing


def test_short_convolution_carries_its_last_inputs(backend):
    dev = device_of(backend)
    ops = make_ops(backend, torch.float32, dev)
    g = torch.Generator().manual_seed(2)
    for C, taps, cuts in ((10, 3, [1, 2, 3, 9]), (70, 4, [5]), (6, 2, [1, 2, 3]), (300, 5, [2, 3, 4, 30])):
        T = 33
        u = torch.randn(T, C + 3, generator=g)
        w = torch.randn(C, taps, generator=g)
        ref = P.short_conv(u[:, 2:2 + C].double().numpy(), w.double().numpy())
        cache = PagedCache([], 2, 3, torch.float32, dev, states=[StateSpec((taps - 1, C), copies=2)])
        cache.states[0].fill_(7.0)
        slot, outs, lo = 1, [], 0
        for hi in cuts + [T]:
            n = hi - lo
            rd, wr = cache.step_rows(slot)
            b = StepBatch(tokens=None, seq=None, pos=torch.arange(lo, hi, dtype=torch.int32, device=dev), slot=None, block_table=None,
                          max_pos=hi - 1, n_tokens=n, items=[(slot, 0, n)], run_off=torch.arange(n, dtype=torch.int32, device=dev),
                          state_rd=torch.full((n,), rd if lo else -1, dtype=torch.int32, device=dev),
                          state_wr=torch.tensor([-1] * (n - 1) + [wr], dtype=torch.int32, device=dev))
            outs.append(ops.conv_silu_unit(u[lo:hi].contiguous().to(dev), 2, w.to(dev), cache.states[0], b, 0, 1, act="none").cpu())
            lo = hi
        assert_close(torch.cat(outs).double(), ref, 2e-6, f"{taps} taps cut at {cuts}")


def _mixer_alone(backend, layer, T, splits, seed=3, width=24, tol=2e-5, dtype="float32"):
    """One mixer through its layer object, the engine's cache and state, the tokens cut at `splits`, against the plain statement."""
    cfg = make_config([layer], width=width)
    W = P.random_weights(cfg, seed=seed)
    Wd = f32(W) if dtype == "float32" else {k: v.bfloat16() for k, v in t64(W).items()}
    eng = build_engine(cfg, Wd, backend, dtype=dtype, max_tokens=max(256, T + 64), max_seqs=3)
    dev, st = eng.device, torch.float32 if dtype == "float32" else torch.bfloat16
    mixer = eng.model.layers[0]["mixer"]
    p0, p1, s0, s1 = eng.model.slices[0]
    g = torch.Generator().manual_seed(seed + 100)
    h = torch.randn(T, width, generator=g).bfloat16().float()
    eps, m, p = cfg["norm"]["eps"], layer["mixer"], "l0.mix."
    hd = h.double().numpy()
    if layer["type"] == "parallel":
        a, b = p + "left.", p + "right."
        wl = {n: W[a + n] for n in ("q", "k", "v", "sink", "o")}
        wl.update({n + "_conv": W[a + n + ".conv"] for n in ("q", "k", "v")}, q_norm=W[a + "q.norm"], k_norm=W[a + "k.norm"])
        wr = {n: W[b + n] for n in ("z", "x", "g", "o")}
        wr.update(z_b=W[b + "z.b"], x_b=W[b + "x.b"])
        ref = 0.5 * (P.rms(P.left_mixer(hd, wl, m["left"], eps)[0], eps) * W[a + "out"] + P.rms(P.min_gru(hd, wr), eps) * W[b + "out"])
    else:
        wa = {n: W[p + n] for n in ("q", "k", "v", "sink", "o")}
        wa.update(q_norm=W[p + "q.norm"], k_norm=W[p + "k.norm"])
        ref = P.attention_mixer(hd, wa, m, eps)[0]
    eng.open_sequence()                                                    # (not slot 0)
    slot = eng.open_sequence()
    for s in eng.cache.states:
        s.fill_(5.0)                                                       # stale state: a new sequence must not read it
    outs, lo = [], 0
    for hi in list(splits) + [T]:
        b = eng.layout([(slot, [0] * (hi - lo))])
        outs.append(mixer(h[lo:hi].to(st).to(dev), b, eng.cache.pools[p0:p1], eng.cache.states[s0:s1]).double().cpu())
        lo = hi
    assert_close(torch.cat(outs), ref, tol, f"{layer['type']} cut at {splits}")


def test_kept_first_attention_alone(backend):
    _mixer_alone(backend, att(), 70, [])
    _mixer_alone(backend, att(), 70, [1, 4, 5, 6, 23, 24, 25, 29, 30, 69])                        # cuts around the kept tokens' and the window's edges
    _mixer_alone(backend, att(heads=6, kv_heads=1, dim=5, vdim=3, size=64, keep=64), 200, [63, 64, 65, 128, 129])   # window = kept = page
    _mixer_alone(backend, att(heads=2, kv_heads=2, dim=16, vdim=24, size=1, keep=1), 20, [1, 2, 7])           # a window of the token itself
    _mixer_alone(backend, att(heads=3, kv_heads=3, dim=4, vdim=4, size=40, keep=0), 130, [39, 40, 41, 100])   # nothing kept
    _mixer_alone(backend, att(heads=4, kv_heads=4, dim=8, vdim=8, size=10, keep=70), 150, [69, 70, 71, 80, 81])  # more kept than a page holds


def test_pooled_block_attention_beside_min_gru_alone(backend):
    _mixer_alone(backend, par(), 80, [])
    _mixer_alone(backend, par(), 80, [1, 2, 3, 4, 5, 6, 16, 17, 18, 21, 22, 26, 27, 79])             # around block ends and the first block's entry
    _mixer_alone(backend, par(heads=2, kv_heads=2, dim=6, vdim=4, size=64, pool=64, conv=2, rot=6, width=9), 260, [63, 64, 127, 128, 129, 192])
    _mixer_alone(backend, par(heads=3, kv_heads=1, dim=10, vdim=6, size=1, pool=1, conv=4, rot=2, width=50), 40, [3, 4, 20])   # every earlier token is a block
    _mixer_alone(backend, par(heads=4, kv_heads=2, dim=4, vdim=12, size=30, pool=7, conv=1, rot=4, width=70), 200, [6, 7, 63, 64, 65, 69, 70, 140])
    _mixer_alone(backend, par(heads=2, kv_heads=1, dim=8, vdim=8, size=5, pool=50, conv=3, rot=8, width=12), 170, [49, 50, 54, 55, 56, 104, 105, 106])
    _mixer_alone(backend, par(heads=2, kv_heads=2, dim=4, vdim=4, size=3, pool=70, conv=2, rot=2, width=6), 300, [69, 70, 72, 73, 139, 140, 143, 280])  # blocks longer than a page


@pytest.mark.gpu
def test_attention_on_the_matrix_cores():
    """bfloat16 storage with sizes the matrix-core kernel takes: prompt tiles whose later rows lie past the first key tile, key splits
    over workgroups for single tokens, several tiles of pooled rows."""
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    for layer, T, splits in ((att(heads=4, kv_heads=2, dim=16, vdim=8, size=88, keep=24), 300, [87, 88, 89, 126, 170, 298, 299]),
                             (att(heads=8, kv_heads=4, dim=40, vdim=24, size=33, keep=70), 420, [399, 400, 401, 419]),
                             (att(heads=6, kv_heads=2, dim=8, vdim=16, size=200, keep=3), 700, [650] + list(range(690, 700))),
                             (par(heads=8, kv_heads=4, dim=16, vdim=16, size=44, pool=10, rot=8, width=48), 500, [43, 44, 53, 54, 126, 170, 498, 499]),
                             (par(heads=4, kv_heads=4, dim=32, vdim=8, size=20, pool=3, conv=2, rot=32, width=16), 400, [300] + list(range(390, 400)))):
        _mixer_alone("hip", layer, T, splits, dtype="bfloat16", tol=3e-2, width=32)


def test_min_gru_alone(backend):
    dev = device_of(backend)
    g = torch.Generator().manual_seed(5)
    for n, D, T, cuts in ((28, 24, 50, [1, 2, 9, 10, 17, 49]), (300, 16, 21, [8]), (5, 40, 9, []), (64, 8, 130, [64, 65])):
        ops = make_ops(backend, torch.float32, dev)
        w = {k: torch.randn(n, D, generator=g).double() / math.sqrt(D) * 2 for k in ("z", "x", "g")}
        w.update(z_b=torch.randn(n, generator=g).double(), x_b=torch.randn(n, generator=g).double(), o=torch.randn(D, n, generator=g).double() / math.sqrt(n))
        h = torch.randn(T, D, generator=g)
        ref = P.min_gru(h.double().numpy(), {k: v.numpy() for k, v in w.items()})
        layer = MinGRU(ops, width=n, weights={k: v.float().to(dev) for k, v in w.items()})
        cache = PagedCache([], 2, 3, torch.float32, dev, states=layer.state_specs)
        cache.states[0].fill_(9.0)
        slot, outs, lo = 2, [], 0
        for hi in cuts + [T]:
            b = StepBatch(tokens=None, seq=None, pos=torch.arange(lo, hi, dtype=torch.int32, device=dev), slot=None, block_table=None,
                          max_pos=hi - 1, n_tokens=hi - lo, items=[(slot, 0, hi - lo)])
            outs.append(layer(h[lo:hi].to(dev), b, [], cache.states).double().cpu())
            lo = hi
        assert_close(torch.cat(outs), ref, 2e-5, f"minGRU of width {n} cut at {cuts}")
        assert float(cache.states[0][0].min()) == 9.0                      # another slot's state is not touched


def test_the_candidate_has_two_branches_and_the_state_is_kept(backend):
    """u = -3, 0, 2 give the candidates sigmoid(-3), 1/2, 5/2; a gate of 1 replaces the state, a gate of 0 keeps it over hundreds of
    tokens and through steps of one token."""
    dev = device_of(backend)
    ops = make_ops(backend, torch.float32, dev)
    n, T = 3, 400
    proj = torch.zeros(T, 3 * n)
    proj[:, :n] = -40.0                                                    # gate shut ...
    proj[0, :n] = 40.0                                                     # ... but for the first token
    proj[0, n:2 * n] = torch.tensor([-3.0, 0.0, 2.0])
    proj[:, 2 * n:] = 30.0                                                 # silu(30) = 30
    zero = torch.zeros(n)
    state = torch.full((2, n), 4.0)
    state = state.to(dev)
    outs, lo = [], 0
    for hi in (1, 2, 3, 200, 399, T):
        b = StepBatch(tokens=None, seq=None, pos=torch.arange(lo, hi, dtype=torch.int32, device=dev), slot=None, block_table=None,
                      max_pos=hi - 1, n_tokens=hi - lo, items=[(1, 0, hi - lo)])
        outs.append(ops.min_gru_scan(proj[lo:hi].contiguous().to(dev), 0, n, 2 * n, zero.to(dev), zero.to(dev), state, b, n).cpu())
        lo = hi
    out = torch.cat(outs) / 30.0
    want = torch.tensor([1.0 / (1.0 + math.exp(3.0)), 0.5, 2.5])
    assert (out[0] - want).abs().max() < 1e-6 and (out[-1] - want).abs().max() < 1e-5 and (state[1].cpu() - want).abs().max() < 1e-5
    assert float(state[0].min()) == 4.0


def _router_case(g, n, D, T, spread):
    return torch.randn(T, D, generator=g), torch.randn(n, D, generator=g).double() * 0.6, torch.randn(n, generator=g).double() * spread


def test_router_with_identity_experts_alone(backend):
    dev = device_of(backend)
    g = torch.Generator().manual_seed(11)
    for E, ident, top, D, ff, T, limit in ((5, 2, 3, 40, 9, 33, 0.8), (12, 4, 2, 24, 16, 70, 1.0), (1, 1, 2, 16, 8, 5, 3.0),
                                           (9, 0, 4, 20, 5, 30, 0.5), (3, 6, 9, 72, 8, 20, 2.0), (24, 3, 2, 64, 48, 600, 1.5)):
        ops = make_ops(backend, torch.float32, dev)
        h, router, corr = _router_case(g, E + ident, D, T, 0.05)
        ex = [tuple(torch.randn(s, generator=g).double() / 3 for s in ((ff, D), (ff, D), (D, ff))) for _ in range(E)]
        ref = P.moe_ff(h.double().numpy(), {"router": router.numpy(), "correction": corr.numpy(),
                                             "experts": [tuple(t.numpy() for t in e) for e in ex]}, top, ident, limit)
        layer = IdentityExpertMoE(ops, router=router.float().to(dev), correction=corr.float().to(dev), gate=[e[0].float().to(dev) for e in ex],
                                  up=[e[1].float().to(dev) for e in ex], down=[e[2].float().to(dev) for e in ex], top_k=top,
                                  identity=ident, limit=limit)
        for lo, hi in ((0, T), (0, 1), (1, 3), (3, min(T, 12))):           # step sizes of every expert kernel form
            assert_close(layer(h[lo:hi].to(dev)).double().cpu(), ref[lo:hi], 2e-5, f"{E} experts + {ident} identity, top {top}, tokens {lo}:{hi}")


@pytest.mark.gpu
def test_expert_kernel_forms_in_bfloat16():
    """bfloat16 storage at sizes that take each form of the expert kernels (per token, expert-major, grouped on the matrix cores, vendor
    products per expert): clamped units and identity experts in all of them.  The router reads the same bfloat16 input as the plain
    statement, so the choices agree and only rounding is left."""
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    dev = "cuda:0"
    ops = make_ops("hip", torch.bfloat16, dev)
    g = torch.Generator().manual_seed(21)
    for E, ident, top, D, ff, limit in ((6, 2, 3, 64, 64, 1.25), (5, 3, 2, 40, 24, 0.75), (30, 6, 4, 128, 64, 2.0)):
        T = 700
        h = torch.randn(T, D, generator=g).bfloat16()
        router = (torch.randn(E + ident, D, generator=g) * 0.6).bfloat16()
        corr = (torch.randn(E + ident, generator=g) * 0.05).bfloat16()
        ex = [tuple((torch.randn(s_, generator=g) / 3).bfloat16() for s_ in ((ff, D), (ff, D), (D, ff))) for _ in range(E)]
        ref = torch.from_numpy(P.moe_ff(h.double().numpy(), {"router": router.double().numpy(), "correction": corr.double().numpy(),
                                                             "experts": [tuple(t.double().numpy() for t in e) for e in ex]}, top, ident, limit))
        layer = IdentityExpertMoE(ops, router=router.to(dev), correction=corr.to(dev), gate=[e[0].to(dev) for e in ex],
                                  up=[e[1].to(dev) for e in ex], down=[e[2].to(dev) for e in ex], top_k=top, identity=ident, limit=limit)
        for lo, hi in ((0, 1), (1, 3), (3, 40), (40, 340), (0, T)):
            got = layer(h[lo:hi].to(dev)).double().cpu()
            d = got - ref[lo:hi]
            bad = (d.abs().max(-1).values > 3e-2 * ref.abs().max()).nonzero().flatten().tolist()
            assert len(bad) <= (hi - lo) // 100, f"{E} + {ident} experts, tokens {lo}:{hi}: rows {bad[:5]} differ (a tipped choice is rare)"


def test_the_correction_moves_the_choice_not_the_weights_and_identity_returns_the_input(backend):
    dev = device_of(backend)
    ops = make_ops(backend, torch.float32, dev)
    D = 8
    h = torch.zeros(2, D)
    h[:, 0] = 1.0
    h[1, 3] = -2.0
    router = torch.zeros(4, D)
    router[:, 0] = torch.tensor([2.0, 1.0, 0.0, -1.0])                    # softmax: .644 .237 .087 .032
    s = torch.softmax(router[:, 0], 0)
    idx, wt = ops.moe_route(h.to(dev), router.to(dev), 2, 1, 1, correction=torch.zeros(4).to(dev))
    assert sorted(idx[0].tolist()) == [0, 1]
    corr = torch.tensor([0.0, -1.0, 0.0, 1.0])
    idx, wt = ops.moe_route(h.to(dev), router.to(dev), 2, 1, 1, correction=corr.to(dev))
    assert sorted(idx[0].tolist()) == [0, 3]
    w = dict(zip(idx[0].tolist(), wt[0].tolist()))
    assert abs(w[3] - float(s[3])) < 1e-6 and abs(w[0] - float(s[0])) < 1e-6 and abs(sum(w.values()) - 1.0) > 0.2   # plain scores, not renormalised
    # outputs 2 and 3 are identity experts; a correction makes them the only ones chosen: the layer returns (s2 + s3) h
    zero = torch.zeros(5, D)
    layer = IdentityExpertMoE(ops, router=router.to(dev), correction=torch.tensor([-5.0, -5.0, 0.0, 0.0]).to(dev), gate=[zero.to(dev)] * 2,
                              up=[zero.to(dev)] * 2, down=[zero.t().contiguous().to(dev)] * 2, top_k=2, identity=2, limit=1.0)
    y = layer(h.to(dev)).cpu()
    assert (y - float(s[2] + s[3]) * h).abs().max() < 1e-6


def test_expert_units_clamp_before_the_product(backend):
    """gate pre-activations of 5 and -5 and up pre-activations of 5, -5 with limit 1.5: g = 1.5 and -5 (only capped above), u = 1.5 and
    -1.5, unit = g sigmoid(1.702 g) (u + 1)."""
    dev = device_of(backend)
    ops = make_ops(backend, torch.float32, dev)
    D, ff = 8, 4
    h = torch.zeros(1, D)
    h[0, 0] = 1.0
    gate, up = torch.zeros(ff, D), torch.zeros(ff, D)
    gate[:, 0] = torch.tensor([5.0, -5.0, 5.0, 0.5])
    up[:, 0] = torch.tensor([5.0, 5.0, -5.0, 0.25])
    down = torch.zeros(D, ff)
    down[:ff] = torch.eye(ff)
    idx, wt = torch.zeros(1, 1, dtype=torch.int32), torch.ones(1, 1)
    from qserve_amd.layers.moe import _interleave
    y = ops.moe_experts(h.to(dev), _interleave(gate[None], up[None]).to(dev), down[None].contiguous().to(dev), idx.to(dev), wt.to(dev),
                        act="clamped_glu", limit=1.5).cpu()[0, :ff]

    def unit(g, u):
        return g / (1.0 + math.exp(-1.702 * g)) * (u + 1.0)

    want = torch.tensor([unit(1.5, 1.5), unit(-5.0, 1.5), unit(1.5, -1.5), unit(0.5, 0.25)])
    assert (y - want).abs().max() < 1e-6


def test_dense_feed_forward_alone(backend):
    dev = device_of(backend)
    ops = make_ops(backend, torch.float32, dev)
    g = torch.Generator().manual_seed(2)
    h = torch.randn(9, 24, generator=g) * 2
    up, down = torch.randn(14, 24, generator=g).double() / 4, torch.randn(24, 14, generator=g).double() / 4
    layer = ReluSquaredFeedForward(ops, up=up.float().to(dev), down=down.float().to(dev))
    assert_close(layer(h.to(dev)).double().cpu(), P.dense_ff(h.double().numpy(), {"up": up.numpy(), "down": down.numpy()}), 2e-5, "relu^2 units")


# ---- keys that stand out: kept first tokens, window edges, pooled blocks, the sink ---------------------------------------------------

def _selector(backend, L, dtype, nq, *, spike=None, keep=0, size=50, pool=None, sink=-30.0, cuts=()):
    """Attention alone with selector weights: the layer input IS [q | k | v], the norms leave directions alone.  All keys are small but
    the one at `spike`; the queries point there.  -> (layer output of the last nq positions, plain statement, h)."""
    H, G, d, dv = 2, 1, 8, 8
    D = H * d + d + dv
    eye = np.eye(D)
    W = {"q": eye[:16], "k": eye[16:24], "v": eye[24:32], "o": np.ascontiguousarray(eye[:, :16]), "sink": np.full(H, float(sink))}
    whole = pool is not None
    W.update(q_norm=np.ones(16 if whole else 8), k_norm=np.ones(8))
    g = torch.Generator().manual_seed((spike[0] if isinstance(spike, tuple) else spike or 0) * 7 + L)
    h = (torch.randn(L, D, generator=g) * 0.05).bfloat16().double()
    h[:, 24:32] = torch.randn(L, dv, generator=g).bfloat16().double()
    if spike is not None:
        lo, hi = (spike, spike + 1) if not isinstance(spike, tuple) else spike
        h[lo:hi, 16 + 7] = 4.0                                               # keys eight times the others
    h[:, 7] = 2.0
    h[:, 8 + 7] = 2.0
    h[:, 16] = 3.0                                                           # off the queries' direction: the norm leaves quiet keys quiet
    m = {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "scale": 6.0, "mask": {"size": size, "keep_first": keep, "pool": pool}}
    hn = h.numpy()
    if whole:
        one = np.zeros((1, 1))
        one[0, 0] = 1.0
        ref = P.left_mixer(hn, dict(W, q_conv=np.ones((16, 1)), k_conv=np.ones((8, 1)), v_conv=np.ones((8, 1))), m, 1e-5)[0]
    else:
        ref = P.attention_mixer(hn, W, m, 1e-5)[0]
    dev = device_of(backend)
    ops = make_ops(backend, dtype, dev)
    page, npages = 64, (L + 63) // 64
    layer = SinkWindowAttention(ops, heads=H, kv_heads=G, dim=d, vdim=dv, scale=6.0, eps=1e-5, window=size, keep_first=keep,
                                pool_block=pool, norm="all" if whole else "head",
                                weights={k: torch.from_numpy(v).to(dtype).to(dev) for k, v in W.items()})
    cache = PagedCache(layer.cache_rows, npages + 3, 2, dtype, dev, page=page)
    cache.free_pages = torch.randperm(npages + 3, generator=g).tolist()     # pages out of order, not the first ones
    cache.admit()
    slot = cache.admit()
    out, lo = None, 0
    for hi in list(cuts) + [L - nq, L]:
        if hi <= lo:
            continue
        b = batch_for(cache, slot, lo, hi, dev)
        out = layer(h[lo:hi].to(dtype).to(dev), b, cache.pools, [])
        lo = hi
    return out.double().cpu(), torch.from_numpy(ref[L - nq:]), h


@pytest.mark.parametrize("dtype,tol", STORAGE)
@pytest.mark.parametrize("nq", [1, 20], ids=["decoded", "prompt"])
def test_kept_first_tokens_and_window_edges_stand_out(backend, nq, dtype, tol):
    """A window of 50 and 18 kept tokens, a sequence of 330: the last query sees [280, 330) and [0, 18).  A loud key among the kept
    ones (0, 17) or just inside the window (280, 281) carries the output; at 18, 19, 64, 278 or 279 it must not be heard.  With 20
    queries in the step the later ones sit in rows of the attention tile whose own window starts past the first key tile."""
    L, size, keep = 330, 50, 18
    for spike in (0, 1, 17, 18, 19, 63, 64, 278, 279, 280, 281, 319, 320, L - 1):
        out, ref, h = _selector(backend, L, dtype, nq, spike=spike, keep=keep, size=size)
        seen = spike < keep or spike >= L - size
        if seen and spike < L - nq:
            assert (ref[-1, :8] - h[spike, 24:32]).abs().max() < 0.15, f"the key at {spike} should carry the output"
        if not seen:
            assert (ref[-1, :8] - h[spike, 24:32]).abs().max() > 0.3, f"the key at {spike} is neither kept nor in the window"
        assert_close(out, ref, tol, f"spike at {spike}")
    for L2, spike, cuts in ((68, 17, (30,)), (69, 18, ()), (130, 5, (64, 100)), (200, 17, (128, 150, 190)), (51, 0, ()), (52, 1, (2,))):
        out, ref, _ = _selector(backend, L2, dtype, min(nq, 7), spike=spike, keep=keep, size=size, cuts=cuts)
        assert_close(out, ref, tol, f"length {L2}, spike at {spike}")


@pytest.mark.parametrize("dtype,tol", STORAGE)
@pytest.mark.parametrize("nq", [1, 20], ids=["decoded", "prompt"])
def test_pooled_blocks_are_seen_when_they_have_left_the_window(backend, nq, dtype, tol):
    """A window of 36 and blocks of 9: a block whose 9 keys are all loud carries the output from the token at which its last position
    is 36 back, not one earlier (block 7 = positions 63 .. 71 straddles a page border); a block far back is heard; a token behind the
    window whose block is still open is not."""
    size, pool = 36, 9
    for L, block in ((108, 7), (107, 7), (108, 8), (330, 0), (330, 5), (330, 31), (330, 32), (64 + 62, 9), (64 + 61, 9)):
        lo, hi = block * pool, block * pool + pool
        out, ref, h = _selector(backend, L, dtype, nq, spike=(lo, hi), size=size, pool=pool, cuts=(hi - 3, hi) if hi < L - nq else ())
        if hi - 1 <= L - 1 - size:                                          # the block has left the last query's window: seen as one key
            assert (ref[-1, :8] - h[lo:hi, 24:32].mean(0)).abs().max() < 0.15, f"block {block} should carry the output of a sequence of {L}"
        assert_close(out, ref, tol, f"length {L}, loud block {block}")
    # length 100: the window starts at 64 and blocks 0 .. 6 are seen.  Position 63 opens block 7: behind the window, in no seen block
    for L, spike in ((100, 63), (100, 62), (101, 63), (109, 63)):
        out, ref, h = _selector(backend, L, dtype, nq, spike=spike, size=size, pool=pool)
        if (L, spike) in ((100, 63), (101, 63)):
            assert (ref[-1, :8] - h[spike, 24:32]).abs().max() > 0.3, "a token behind the window in an open block is not seen"
        assert_close(out, ref, tol, f"length {L}, spike at {spike}")


@pytest.mark.parametrize("dtype,tol", STORAGE)
def test_the_sink_takes_its_share(backend, dtype, tol):
    """Quiet keys and a sink well above every score: the output shrinks towards zero by the sink's share, for the first token of
    a sequence as for later ones; a sink far below changes nothing."""
    for sink in (-30.0, 0.0, 8.0):
        for L, nq, kw in ((1, 1, {}), (3, 3, {}), (90, 1, {"keep": 4}), (90, 9, {"keep": 4}), (150, 2, {"pool": 10, "size": 30})):
            out, ref, h = _selector(backend, L, dtype, nq, sink=sink, **kw)
            assert_close(out, ref, tol, f"sink {sink}, length {L}")
            if sink == 8.0 and L == 1:
                assert ref.abs().max() < 0.3 * h[0, 24:32].abs().max()
            if sink == -30.0 and L == 1:
                assert (ref[0, :8] - h[0, 24:32]).abs().max() < 1e-6


@pytest.mark.parametrize("R", [6, 8, 1028])
def test_pooled_rows_live_in_their_blocks_first_page(backend, R):
    """Blocks of 12 positions on pages of 64: the block [60, 72) straddles two pages and its row belongs to the first; six rows a
    page.  The rows hold the float mean of the cached rows."""
    dev = device_of(backend)
    ops = make_ops(backend, torch.float32, dev)
    G, P_, page = 2, 12, 64
    cache = PagedCache([(G, R), (G, R, 6)], 5, 2, torch.float32, dev, page=page)
    assert cache.pools[1].shape == (G, 5 * 6, R)
    cache.free_pages = [1, 4, 0, 3, 2]                                     # handed out from the end: 2, 3, 0
    slot = cache.admit()
    g = torch.Generator().manual_seed(0)
    data = torch.randn(G, 150, R, generator=g)
    lo = 0
    for hi in (5, 11, 12, 71, 72, 73, 150):
        b = batch_for(cache, slot, lo, hi, dev)
        cache.pools[0][:, b.slot] = data[:, lo:hi].to(dev)
        ops.pool_blocks(cache.pools[0], cache.pools[1], b, P_, page)
        lo = hi
    pages = cache.pages[slot]
    for blk in range(150 // P_):
        first = blk * P_
        row = pages[first // page] * 6 + (first % page) // P_
        assert_close(cache.pools[1][:, row].double().cpu(), data[:, first:first + P_].double().mean(1), 1e-6, f"block {blk}")
    used = {pages[(b * P_) // page] * 6 + ((b * P_) % page) // P_ for b in range(150 // P_)}
    rest = [r for r in range(30) if r not in used]
    assert float(cache.pools[1][:, rest].abs().max()) == 0.0               # nothing else is written (the open block 144.. neither)
    with pytest.raises(ValueError):
        PagedCache([(G, R, 65)], 5, 2, torch.float32, dev, page=page)


# ---- the whole model ---------------------------------------------------------------------------------------------------------------

@pytest.fixture(scope="module")
def std():
    cfg = standard_config()
    W = P.random_weights(cfg, seed=1)
    seqs = {"a": tokens_for(cfg, 150, 1), "b": tokens_for(cfg, 37, 2), "c": tokens_for(cfg, 1, 3), "d": tokens_for(cfg, 81, 4)}
    ref, layers = {}, {}
    for k, v in seqs.items():
        taps = []
        ref[k] = plain_logits(cfg, W, v, taps)
        layers[k] = [torch.from_numpy(t) for t in taps]
    return cfg, W, seqs, ref, layers


def test_layers_one_by_one(backend, std):
    cfg, W, seqs, _, layers = std
    eng = build_engine(cfg, f32(W), backend)
    slot = eng.open_sequence()
    b = eng.layout([(slot, seqs["d"])])
    seen = []
    eng.model.forward(b, eng.cache.pools, states=eng.cache.states, tap=lambda i, x: seen.append(x.double().cpu().clone()))
    assert len(seen) == len(cfg["layers"])
    for i, x in enumerate(seen):
        assert_close(x, layers["d"][i], F32_TOL, f"residual stream after layer {i}")


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
        assert all(float(p.abs().max()) > 0 for p in eng.cache.pools)             # and so are the pages and the block rows
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
    cfg = make_config([par(size=20, pool=6, mlp=dense(12)), att(size=50, keep=3, mlp=None), att(size=8, keep=70, kv_from=1, mlp=moe(experts=4, identity=1, top=1))],
                      width=32, vocab=29)
    W = P.random_weights(cfg, seed=9)
    toks = tokens_for(cfg, 210, 5)
    ref = plain_logits(cfg, W, toks)
    eng = build_engine(cfg, f32(W), backend, max_tokens=256, max_seqs=1)
    got = run_schedule(eng, {"s": toks}, [[("s", 3)]] + [[("s", 1)]] * 207)      # decoded tokens pass window edges, block ends and three page borders
    assert_close(got["s"], ref, F32_TOL, "207 decoded tokens")


@pytest.mark.parametrize("variant", range(4))
def test_other_sizes(backend, variant):
    layers, kw = [
        ([par(heads=1, kv_heads=1, dim=2, vdim=2, size=1, pool=1, conv=1, rot=2, width=1, mlp=moe(experts=1, identity=1, top=2, ff=1))],
         dict(width=8, vocab=5, eps=1e-3)),
        ([att(heads=6, kv_heads=3, dim=16, vdim=24, size=31, keep=31, mlp=moe(experts=9, identity=3, top=5, ff=33, limit=0.2)),
          par(heads=4, kv_heads=4, dim=32, vdim=16, size=64, pool=32, conv=4, rot=32, width=96, mlp=dense(100)),
          att(heads=3, kv_heads=3, dim=16, vdim=24, size=64, keep=1, kv_from=0, mlp=None)], dict(width=96, vocab=200)),
        ([att(heads=2, kv_heads=2, dim=6, vdim=64, size=10, keep=2, mlp=None), par(heads=7, kv_heads=1, dim=70, vdim=5, size=3, pool=2, conv=2, rot=10, width=13)],
         dict(width=41, vocab=33, eps=1e-6)),
        ([par(mlp=dense(8)), par(size=12, pool=12, mlp=moe(experts=8, identity=8, top=3)), att(heads=1, kv_heads=1, mlp=None), att(heads=5, kv_heads=1, kv_from=2),
          att(heads=3, kv_heads=3, dim=8, vdim=10, size=200, keep=0, kv_from=0)],
         dict(width=48, vocab=61)),
    ][variant]
    cfg = make_config(layers, **kw)
    W = P.random_weights(cfg, seed=20 + variant)
    toks = tokens_for(cfg, 75, variant)
    ref = plain_logits(cfg, W, toks)
    eng = build_engine(cfg, f32(W), backend)
    got = run_schedule(eng, {"s": toks}, [[("s", 40)], [("s", 30)]] + [[("s", 1)]] * 5)
    assert_close(got["s"], ref, F32_TOL, f"sizes variant {variant}")


def test_bfloat16_storage_stays_near_the_plain_statement(backend, std):
    cfg, W, seqs, ref, _ = std
    Wb = {k: v.bfloat16() for k, v in t64(W).items()}
    eng = build_engine(cfg, Wb, backend, dtype="bfloat16")
    got = run_schedule(eng, seqs, [[("a", 70), ("b", 37)], [("a", 80)]])
    for k in ("a", "b"):
        d = got[k] - ref[k]
        rel = (d - d.mean(-1, keepdim=True)).pow(2).mean().sqrt() / ref[k].std()
        assert rel < 0.1, f"bfloat16 run of {k}: relative error {rel:.3f}"
    got2 = run_schedule(eng, seqs, [[("a", 3)], [("a", 147)]])                      # cut differently: the same up to rounding
    rel = (got2["a"] - got["a"]).pow(2).mean().sqrt() / ref["a"].std()
    assert rel < 0.1


def test_a_layer_without_keys_reads_its_source_layers_pools(backend, std):
    cfg, W, _, _, _ = std
    eng = build_engine(cfg, f32(W), backend)
    m = eng.model
    assert m.slices[2][:2] == m.slices[1][:2] and m.slices[5][:2] == m.slices[4][:2]
    assert m.layers[2]["mixer"].cache_rows == [] and len(eng.cache.pools) == 2 + 1 + 2 + 1      # two pools per pooled layer, one per owner
    bad = json.loads(json.dumps(cfg))
    bad["layers"][2]["mixer"]["kv_from"] = 3                                                    # a later layer
    with pytest.raises(ValueError):
        Pemolorn.from_config(bad, f32(W), make_ops("unfused", torch.float32, "cpu"), "cpu", torch.float32)


# ---- generation through the engine's own entry point and scheduler ---------------------------------------------------------------

def plain_greedy(cfg, W, prompt, n):
    toks, margins = list(prompt), []
    for _ in range(n):
        lg = plain_logits(cfg, W, toks)[-1]
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
        ref, margins = plain_greedy(cfg, W, p, 6)
        for i, (a, b) in enumerate(zip(o, ref)):
            if a != b:
                assert margins[i] < 1e-3, f"prompt of {len(p)}: token {i} is {a}, plain statement {b} (margin {margins[i]:.2e})"
                break
        else:
            assert len(o) == 6


def _save_model(tmp_path, cfg, W):
    from safetensors.torch import save_file
    with open(tmp_path / "config.json", "w") as f:
        json.dump(cfg, f)
    save_file({k: v.bfloat16().contiguous() for k, v in t64(W).items()}, str(tmp_path / "model.safetensors"))


def test_registry_and_checkpoint_directory(tmp_path, backend, std):
    from qserve_amd.serving import registry
    assert registry.architectures()["Pemolorn"] == "paged"
    cfg, W, seqs, ref, _ = std
    _save_model(tmp_path, cfg, W)
    eng = Engine.from_pretrained(str(tmp_path), dtype="float32", device=device_of(backend), max_tokens=128, backend=backend)
    got = run_schedule(eng, seqs, [[("b", 37)]])
    assert_close(got["b"], ref["b"], F32_TOL)
    bad = dict(cfg, layers=[dict(cfg["layers"][0], type="unknown")])
    with pytest.raises(ValueError):
        Pemolorn.from_config(bad, f32(W), make_ops("unfused", torch.float32, "cpu"), "cpu", torch.float32)
    with pytest.raises(KeyError):
        Pemolorn.from_config(cfg, {k: v for k, v in f32(W).items() if k != "l0.mix.right.z.b"}, make_ops("unfused", torch.float32, "cpu"),
                             "cpu", torch.float32)


# ---- GPU only ---------------------------------------------------------------------------------------------------------------------

@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_replay_command(tmp_path, dtype, std):
    """bin/trace_run on a checkpoint directory: portions, single tokens, a mixed batch, a sequence ended and its slot used again."""
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    cfg, W, seqs, ref, _ = std
    _save_model(tmp_path, cfg, W)
    out = tmp_path / "out"
    a, b, d = seqs["a"], seqs["b"], seqs["d"]
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:70], "want": [0, 69]}, {"id": "b", "tokens": b[:2], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "b", "tokens": b[2:], "want": [34]}, {"id": "a", "tokens": a[70:71], "want": [0]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": a[71:], "want": [78]}, {"id": "d", "tokens": d, "want": [80]}], "end": ["a", "d"]},
             {"step": 3, "entries": [{"id": "e", "tokens": b, "want": [36]}], "end": ["e"]}]
    r = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", str(tmp_path), "--dtype", dtype, "--out", str(out),
                        "--max-tokens", "320"], input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True,
                       timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [ln for ln in r.stdout.split("\n") if ln.startswith("done")] == [f"done {i}" for i in range(4)]
    V = cfg["vocab"]
    want = {0: [ref["a"][0], ref["a"][69]], 1: [ref["b"][36], ref["a"][70]], 2: [ref["a"][149], ref["d"][80]], 3: [ref["b"][36]]}
    for i, rows in want.items():
        got = torch.from_numpy(np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, V).astype(np.float64))
        assert got.shape[0] == len(rows)
        for g_, r_ in zip(got, rows):
            if dtype == "float32":
                assert_close(g_, r_, F32_TOL, f"step {i}")
            else:
                assert ((g_ - r_).pow(2).mean().sqrt() / r_.std()) < 0.1


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_steps_from_a_graph_match_eager_steps(dtype, std):
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    cfg, W, seqs, _, _ = std
    Wd = f32(W) if dtype == "float32" else {k: v.bfloat16() for k, v in t64(W).items()}
    outs = []
    for graphs in (False, True):
        eng = build_engine(cfg, Wd, "hip", dtype=dtype, max_tokens=512, max_seqs=2, decode_graphs=graphs)
        steps = [[("a", 100), ("b", 30)]] + [[("a", 1), ("b", 1)]] * 7 + [[("a", 1)]] * 43
        outs.append(run_schedule(eng, seqs, steps))
        if graphs:
            assert any(g for g in eng._graphs.values()), "no decode step was replayed from a graph"
    for k in ("a", "b"):
        assert_close(outs[1][k], outs[0][k], 1e-5 if dtype == "float32" else 2e-2, f"graph replay, sequence {k}")
