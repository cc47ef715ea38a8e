"""Throughput of a served design at layer sizes of real models, beside the closest existing model at equal size.

    python bench.py --design vekalorn [--design-sizes w2048,w4096] [--steps K] [--warmup W]     beside the W4A8KV4 Llama engine
    python bench.py --design mumelix  [--design-sizes w2048,w4096] [--steps K] [--warmup W]     beside Vekalorn
    python bench.py --design vepolix  [--design-sizes w2048,w4096] [--steps K] [--warmup W]     beside Mumelix
    python bench.py --design pemolorn [--design-sizes w2048,w4096] [--steps K] [--warmup W]     beside Mumelix

Per size (random weights, 4 layers, vocabulary 32000): prompt phase = 8 prompts x 1024 tokens in one step through
Engine.execute; decoding = 64 sequences at context 1024, one token each per step.  Beside them the Llama-style W4A8KV4
engine (qserve_amd.decode.DecodeEngine) with the same width, head count and ACTIVE feed-forward width, same batch and
context.  Per kernel class the achieved fraction of its roofline (HBM bytes for decoding, dense bf16 / fp16 matrix-core
peak for the prompt phase) is printed for both, from HIP events around every launch of one step.
One JSON line per size on standard output.
"""
import json
import math
import time

import torch

BF16_PEAK_TFLOPS = 2500.0
HBM_PEAK_GBS = 8000.0

SIZES = {
    "w2048": dict(width=2048, heads=16, dim=128, rot_dim=64, vdim=128, kv_rank=512, q_rank=768, window=1024,
                  experts=16, groups=4, keep=2, top=4, ff=1408),
    "w2048r256": dict(width=2048, heads=16, dim=128, rot_dim=64, vdim=128, kv_rank=256, q_rank=768, window=1024,
                      experts=16, groups=4, keep=2, top=4, ff=1408),
    "w4096": dict(width=4096, heads=32, dim=128, rot_dim=64, vdim=128, kv_rank=512, q_rank=1536, window=1024,
                  experts=32, groups=8, keep=4, top=4, ff=2752),
}
LAYERS, VOCAB = 4, 32000


def vekalorn_config(s):
    rot = {"base": 10000.0, "dims": s["rot_dim"], "scaling": {"factor": 8.0, "original": 4096, "fast": 32.0, "slow": 1.0}}
    mlp = {"kind": "moe", "expert": {"ff": s["ff"]},
           "router": {"experts": s["experts"], "top": s["top"], "groups": {"count": s["groups"], "keep": s["keep"]}}}
    common = {k: s[k] for k in ("heads", "dim", "vdim", "kv_rank", "q_rank")}
    a2 = {"type": "latent_attention_2", "mlp": mlp,
          "mixer": dict(common, rot_dim=s["rot_dim"], rot=rot, scale=1.0 / math.sqrt(s["dim"] + s["rot_dim"]))}
    a1 = {"type": "latent_attention", "mlp": mlp,
          "mixer": dict(common, mask={"size": s["window"]}, scale=1.0 / math.sqrt(s["dim"]))}
    return {"architecture": "Vekalorn", "width": s["width"], "vocab": VOCAB, "norm": {"eps": 1e-5},
            "layers": [a2, a1, a1, a2][:LAYERS]}


def random_weights(cfg, dev, seed=0):
    g = torch.Generator(device=dev).manual_seed(seed)
    D, V = cfg["width"], cfg["vocab"]

    def mat(o, i, s=1.0):
        return (torch.randn((o, i), device=dev, generator=g) * (s / math.sqrt(i))).bfloat16()

    def vec(n):
        return (1.0 + 0.1 * torch.randn((n,), device=dev, generator=g)).bfloat16()

    W = {"embed": torch.randn((V, D), device=dev, generator=g).bfloat16(), "head": mat(V, D), "final.norm": vec(D)}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        H, d, dv, r, qr = m["heads"], m["dim"], m["vdim"], m["kv_rank"], m["q_rank"]
        dr = m.get("rot_dim", 0)
        W[p + "norm1"], W[p + "norm2"] = vec(D), vec(D)
        W[p + "mix.dq"], W[p + "mix.dq.norm"], W[p + "mix.uq"] = mat(qr, D), vec(qr), mat(H * (d + dr), qr)
        W[p + "mix.dkv"], W[p + "mix.dkv.norm"] = mat(r + dr, D), vec(r)
        W[p + "mix.uk"], W[p + "mix.uv"], W[p + "mix.o"] = mat(H * d, r), mat(H * dv, r), mat(D, H * dv)
        if L["type"] == "latent_attention_2":
            W[p + "mix.g"] = mat(H * dv, D)
        E, ff = L["mlp"]["router"]["experts"], L["mlp"]["expert"]["ff"]
        for e in range(E):
            W[f"{p}mlp.e{e}.up"], W[f"{p}mlp.e{e}.down"] = mat(ff, D), mat(D, ff)
        W[p + "mlp.router"] = mat(E, D, 3.0)
    return W


class OpTimer:
    """HIP events around every call of the ops object's methods and of the vendor products (one step at a time)."""
    NAMES = ("embed", "add_layer_norm", "layer_norm_rows", "latent_prep", "latent_query", "latent_attention", "sigmoid_gate",
             "moe_route", "moe_experts", "embed_streams", "hc_read", "hc_write", "dyt_sum_rows", "rms_pair_mean", "glu",
             "attention_prep", "rotate_heads", "decay", "conv_silu_unit", "recurrent_scan", "head_rms_gate", "embed_sinusoid",
             "add_rms_norm", "rms_norm_rows", "normed_attention_prep", "max_gates", "add_normed_rms_norm", "qk_norm_rope_prep", "pool_blocks",
             "min_gru_scan", "relu_sq")

    def __init__(self, ops):
        self.ops, self.events, self.calls, self.on = ops, [], [], False
        for n in self.NAMES:
            setattr(ops, n, self._wrap(n, getattr(ops, n)))
        from ..layers import ops as ops_module                # the vendor products, as the layers call them
        for mod in self._linear_users():
            mod.linear = self._wrap("linear", ops_module.linear)

    @staticmethod
    def _linear_users():
        import importlib
        return [importlib.import_module("qserve_amd." + m) for m in
                ("layers.latent_attention", "layers.moe", "layers.recurrent", "layers.softmax_attention", "models.vekalorn",
                 "models.mumelix", "models.vepolix", "models.pemolorn")]

    def _wrap(self, name, fn):
        def timed(*a, **k):
            if not self.on:
                return fn(*a, **k)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            r = fn(*a, **k)
            e1.record()
            self.events.append((name, e0, e1))
            self.calls.append((name, fn, a, k))
            return r
        return timed

    def replay(self, name, reps=20):
        """The launches of `name` recorded in the last step(), each repeated back to back on the same arguments: ms per launch
        without the host's share (what the kernel itself takes), summed over the step's launches."""
        total = 0.0
        for n, fn, a, k in self.calls:
            if n != name:
                continue
            fn(*a, **k)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(reps):
                fn(*a, **k)
            e1.record()
            torch.cuda.synchronize()
            total += e0.elapsed_time(e1) / reps
        return total

    def step(self, fn):
        """Run fn() with timing on -> ({op: ms summed over its launches}, total ms between first and last event)."""
        self.events, self.calls, self.on = [], [], True
        t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0.record()
        fn()
        t1.record()
        self.on = False
        torch.cuda.synchronize()
        out = {}
        for n, e0, e1 in self.events:
            out[n] = out.get(n, 0.0) + e0.elapsed_time(e1)
        return out, t0.elapsed_time(t1)


def timed(fn, steps, warmup):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps * 1e3


def bench_vekalorn(name, s, dev, steps, warmup):
    from ..models.vekalorn import Vekalorn
    from .engine import Engine
    cfg = vekalorn_config(s)
    NB, L, BP = 64, 1024, 8
    eng = Engine(Vekalorn, cfg, random_weights(cfg, dev), dtype="bfloat16", device=dev, max_tokens=NB * (L + 384), max_seqs=NB)
    timer = OpTimer(eng.ops)
    g = torch.Generator().manual_seed(1)
    prompts = [torch.randint(0, VOCAB, (L,), generator=g).tolist() for _ in range(NB)]
    slots = [eng.open_sequence() for _ in range(NB)]
    # prompt phase: 8 steps of 8 prompts (fills the cache for decoding); step 0 warms up, the others are timed
    pre_ms, ops_pre = [], None
    for i in range(0, NB, BP):
        items = [(slots[j], prompts[j]) for j in range(i, i + BP)]
        want = [k * L + L - 1 for k in range(BP)]
        if i == BP:                                          # one step with events around every launch
            ops_pre, _ = timer.step(lambda: eng.execute(items, want))
            att_pre_ms = timer.replay("latent_attention", 5)
            continue
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        eng.execute(items, want)
        torch.cuda.synchronize()
        if i > 0:
            pre_ms.append((time.perf_counter() - t0) * 1e3)
    pre = sorted(pre_ms)[len(pre_ms) // 2]
    # decoding
    nxt = [[int(torch.randint(0, VOCAB, (1,), generator=g))] for _ in range(NB)]
    want = list(range(NB))

    def decode():
        eng.execute([(slots[j], nxt[j]) for j in range(NB)], want)

    res = {}
    forms = {"per_token": dict(moe_token_slots=10 ** 9, moe_sorted_above=10 ** 9),
             "expert_major": dict(moe_token_slots=0, moe_expert_major_slots=10 ** 9),
             "expert_sorted_vendor_products": dict(moe_token_slots=10 ** 9, moe_expert_major_slots=0, moe_sorted_above=0)}
    for label, knobs in forms.items():
        for k, v in knobs.items():
            setattr(eng.ops, k, v)
        res[label] = timed(decode, max(4, steps // 4), 2)
        for k in knobs:
            delattr(eng.ops, k)
    dec_eager = timed(decode, steps, warmup)
    ops_dec, dec_events_ms = timer.step(decode)
    att_dec_ms = timer.replay("latent_attention", 20)
    moe_dec_ms = timer.replay("moe_experts", 20)
    eng.decode_graphs = True                                 # the same steps replayed from a hipGraph
    dec = timed(decode, steps, warmup)
    graph_ok = any(v is not False for v in eng._graphs.values()) and bool(eng._graphs)
    ctx = eng.cache.length[slots[0]]
    # rooflines
    m1 = cfg["layers"][1]["mixer"]
    H, rank = m1["heads"], m1["kv_rank"]
    rows = {"latent_attention_2": rank + s["rot_dim"], "latent_attention": rank}
    kinds = [x["type"] for x in cfg["layers"]]
    T = BP * L
    flops = sum(sum(min(p + 1, s["window"]) if k == "latent_attention" else p + 1 for p in range(L)) * BP * H * (rows[k] + rank) * 2.0
                for k in kinds)
    att_pre = flops / (att_pre_ms * 1e-3) / 1e12
    by = sum(NB * (min(ctx, s["window"]) if k == "latent_attention" else ctx) * rows[k] * 2.0 for k in kinds)
    att_dec = by / (att_dec_ms * 1e-3) / 1e9
    moe_flops = LAYERS * T * s["top"] * 2 * 2.0 * s["ff"] * s["width"]
    moe_pre = moe_flops / (ops_pre["moe_experts"] * 1e-3) / 1e12
    moe_bytes = LAYERS * min(s["experts"], NB * s["top"]) * 2 * s["ff"] * s["width"] * 2.0
    moe_dec = moe_bytes / (moe_dec_ms * 1e-3) / 1e9
    out = dict(model=f"Vekalorn-{name}", prefill_tokens_per_s=T / pre * 1e3, prefill_ms=pre, decode_tokens_per_s=NB / dec * 1e3,
               decode_ms=dec, decode_from_hipgraph=graph_ok, decode_ms_eager=dec_eager, decode_ms_eager_by_expert_form=res,
               decode_ms_gpu_events=dec_events_ms, decode_experts_kernels_ms=moe_dec_ms, context=ctx,
               prefill_ops_ms=ops_pre, decode_ops_ms=ops_dec, prefill_attention_kernels_ms=att_pre_ms,
               decode_attention_kernels_ms=att_dec_ms,
               roofline=dict(prefill_attention_tflops=att_pre, prefill_attention_frac_bf16_peak=att_pre / BF16_PEAK_TFLOPS,
                             decode_attention_gbs=att_dec, decode_attention_frac_hbm=att_dec / HBM_PEAK_GBS,
                             prefill_experts_tflops=moe_pre, prefill_experts_frac_bf16_peak=moe_pre / BF16_PEAK_TFLOPS,
                             decode_experts_gbs=moe_dec, decode_experts_frac_hbm=moe_dec / HBM_PEAK_GBS))
    for sl in slots:
        eng.close_sequence(sl)
    del eng
    torch.cuda.empty_cache()
    return out


def bench_llama(name, s, dev, steps, warmup, helpers):
    """The closest existing model at equal size: same width and heads (head dimension 128), feed-forward width = the active
    expert width, W4A8 per-channel weights, KV4 cache."""
    from .. import decode as D
    cfg = dict(name=f"llama-w4a8-{name}", hidden=s["width"], heads=s["heads"], kv_heads=s["heads"], inter=s["top"] * s["ff"],
               layers=LAYERS, vocab=VOCAB, rope_theta=1e4, eps=1e-5)
    NB, L, BP = 64, 1024, 8
    pe = D.DecodeEngine(cfg, batch=BP, prompt_len=L, max_new=8, device=dev)
    pre = timed(lambda: pe.prefill(L), 3, 1)
    del pe
    torch.cuda.empty_cache()
    eng = D.DecodeEngine(cfg, batch=NB, prompt_len=L, max_new=64, device=dev)
    eng.prefill_cache(L)
    eager = timed(eng.step, steps, warmup)
    eng.lengths.fill_(L + 1)
    eng.capture()
    dec = timed(eng.run, steps, warmup)
    eng.lengths.fill_(L + 1)
    ns = type("A", (), {})()
    kern = helpers.kernel_bench(eng, ns, torch, [L + 1]) + helpers.prefill_attention_bench(torch, dev, cfg, BP, L)
    keep = [{k: v for k, v in r.items() if k in ("kernel", "us", "gbs", "tops", "tflops", "frac_of_hbm_peak", "frac_of_fp16_mfma_peak")}
            for r in kern]
    gemm = [r for r in kern if r.get("family") == "w4a8_gemm"]
    return dict(model=cfg["name"], prefill_tokens_per_s=BP * L / pre * 1e3, prefill_ms=pre, decode_tokens_per_s=NB / dec * 1e3,
                decode_ms=dec, decode_ms_eager=eager, kernels=keep,
                roofline=dict(decode_gemm_frac_hbm=sum(r["bytes"] for r in gemm) / sum(r["us"] for r in gemm) / 1e3 / HBM_PEAK_GBS))


# ---- Mumelix ----------------------------------------------------------------------------------------------------------------
FP32_VALU_PEAK_TFLOPS = 157.0
MUMELIX = {
    "w2048": dict(g_heads=16, g_dim=64, g_vdim=128, a_heads=16, a_kv=4, a_dim=128, a_vdim=128, rot=64, d_heads=16, d_kv=4,
                  d_dim=64, d_vdim=128, taps=4, low=64, streams=2),
    "w4096": dict(g_heads=32, g_dim=64, g_vdim=128, a_heads=32, a_kv=8, a_dim=128, a_vdim=128, rot=64, d_heads=32, d_kv=8,
                  d_dim=64, d_vdim=128, taps=4, low=128, streams=2),
}


def mumelix_config(s, m):
    mlp = {"kind": "moe", "expert": {"ff": s["ff"]}, "router": {"experts": s["experts"], "top": s["top"]}}
    g = {"type": "gla", "mlp": mlp, "mixer": {"heads": m["g_heads"], "dim": m["g_dim"], "vdim": m["g_vdim"], "tau": 8.0}}
    rot = {"base": 500000.0, "dims": m["rot"], "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}}
    p = {"type": "parallel", "mlp": mlp,
         "mixer": {"left": {"heads": m["a_heads"], "kv_heads": m["a_kv"], "dim": m["a_dim"], "vdim": m["a_vdim"], "rot": rot,
                            "scale": 1.0 / math.sqrt(m["a_dim"])},
                   "right": {"heads": m["d_heads"], "kv_heads": m["d_kv"], "dim": m["d_dim"], "vdim": m["d_vdim"], "conv": m["taps"]}}}
    return {"architecture": "Mumelix", "width": s["width"], "vocab": VOCAB, "streams": m["streams"], "embedding": {"scale": 1.0},
            "norm": {"eps": 1e-5}, "layers": [g, p, g, p][:LAYERS]}


def mumelix_weights(cfg, m, dev, seed=0):
    g = torch.Generator(device=dev).manual_seed(seed)
    D, V, S, r = cfg["width"], cfg["vocab"], cfg["streams"], m["low"]

    def mat(o, i, s=1.0):
        return (torch.randn((o, i), device=dev, generator=g) * (s / math.sqrt(i))).bfloat16()

    def vec(n, mean=1.0, s=0.1):
        return (mean + s * torch.randn((n,), device=dev, generator=g)).bfloat16()

    W = {"embed": torch.randn((V, D), device=dev, generator=g).bfloat16(), "head": mat(V, D)}

    def norm(name):
        W[name], W[name + ".b"], W[name + ".alpha"] = vec(D), vec(D, 0.0), torch.tensor(0.7).bfloat16()

    norm("final.norm")
    for i, L in enumerate(cfg["layers"]):
        p, x = f"l{i}.", L["mixer"]
        norm(p + "norm1"), norm(p + "norm2")
        W[p + "shift"] = vec(D, 0.5, 0.2)
        for q in (1, 2):
            W[p + f"hc{q}.in"], W[p + f"hc{q}.out"] = vec(S, 1.0 / S), vec(S, 1.0)
            W[p + f"hc{q}.mix"] = (torch.eye(S, device=dev) * 0.9 + 0.05).bfloat16()
        if L["type"] == "gla":
            H, d, dv = x["heads"], x["dim"], x["vdim"]
            W.update({p + "mix.q": mat(H * d, D), p + "mix.k": mat(H * d, D), p + "mix.v": mat(H * dv, D), p + "mix.g": mat(H * dv, D),
                      p + "mix.o": mat(D, H * dv), p + "mix.norm": vec(dv), p + "mix.a1": mat(r, D), p + "mix.a2": mat(H * d, r),
                      p + "mix.a2.b": vec(H * d, 3.0, 1.0)})
        else:
            a, b = x["left"], x["right"]
            q = p + "mix.left."
            W.update({q + "q": mat(a["heads"] * a["dim"], D), q + "k": mat(a["kv_heads"] * a["dim"], D),
                      q + "v": mat(a["kv_heads"] * a["vdim"], D), q + "o": mat(D, a["heads"] * a["vdim"]), q + "out": vec(D)})
            q = p + "mix.right."
            H, G, d, dv, taps = b["heads"], b["kv_heads"], b["dim"], b["vdim"], b["conv"]
            W.update({q + "q": mat(G * d, D), q + "k": mat(G * d, D), q + "v": mat(H * dv, D), q + "q.conv": mat(G * d, taps),
                      q + "k.conv": mat(G * d, taps), q + "v.conv": mat(H * dv, taps), q + "b": mat(H, D), q + "A_log": vec(H, -1.0, 0.5),
                      q + "norm": vec(dv), q + "a1": mat(r, D), q + "a2": mat(H * d, r), q + "dt_bias": vec(H * d, -1.0, 1.0),
                      q + "g1": mat(r, D), q + "g2": mat(H * dv, r), q + "o": mat(D, H * dv), q + "out": vec(D)})
        E, ff = L["mlp"]["router"]["experts"], L["mlp"]["expert"]["ff"]
        for e in range(E):
            W[f"{p}mlp.e{e}.gate"], W[f"{p}mlp.e{e}.up"], W[f"{p}mlp.e{e}.down"] = mat(ff, D), mat(ff, D), mat(D, ff)
        W[p + "mlp.router"], W[p + "mlp.router.b"] = mat(E, D, 3.0), vec(E, 0.0, 0.5)
    return W


def bench_mumelix(name, s, dev, steps, warmup):
    from ..models.mumelix import Mumelix
    from .engine import Engine
    m = MUMELIX[name]
    cfg = mumelix_config(s, m)
    NB, L, BP = 64, 1024, 8
    eng = Engine(Mumelix, cfg, mumelix_weights(cfg, m, dev), dtype="bfloat16", device=dev, max_tokens=NB * (L + 384), max_seqs=NB)
    timer = OpTimer(eng.ops)
    g = torch.Generator().manual_seed(1)
    prompts = [torch.randint(0, VOCAB, (L,), generator=g).tolist() for _ in range(NB)]
    slots = [eng.open_sequence() for _ in range(NB)]
    pre_ms, ops_pre, rep_pre = [], None, {}
    for i in range(0, NB, BP):
        items = [(slots[j], prompts[j]) for j in range(i, i + BP)]
        want = [k * L + L - 1 for k in range(BP)]
        if i == BP:                                          # one step with events around every launch
            ops_pre, _ = timer.step(lambda: eng.execute(items, want))
            rep_pre = {k: timer.replay(k, 3) for k in ("latent_attention", "hc_read", "hc_write")}
            continue
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        eng.execute(items, want)
        torch.cuda.synchronize()
        if i > 0:
            pre_ms.append((time.perf_counter() - t0) * 1e3)
    pre = sorted(pre_ms)[len(pre_ms) // 2]
    nxt = [[int(torch.randint(0, VOCAB, (1,), generator=g))] for _ in range(NB)]
    want = list(range(NB))

    def decode():
        eng.execute([(slots[j], nxt[j]) for j in range(NB)], want)

    dec_eager = timed(decode, steps, warmup)
    ops_dec, dec_events_ms = timer.step(decode)
    rep_dec = {k: timer.replay(k, 20) for k in ("latent_attention", "moe_experts", "hc_read", "hc_write")}
    eng.decode_graphs = True
    dec = timed(decode, steps, warmup)
    graph_ok = any(v is not False for v in eng._graphs.values()) and bool(eng._graphs)
    ctx = eng.cache.length[slots[0]]
    T, D, S = BP * L, s["width"], m["streams"]
    n_att = sum(1 for x in cfg["layers"] if x["type"] == "parallel")
    n_gla = LAYERS - n_att
    R = m["a_dim"] + m["a_vdim"]
    # attention: useful work = q.k over dim and p.v over vdim (the kernel also multiplies the query's zero half)
    att_flops = n_att * BP * sum(p + 1 for p in range(L)) * m["a_heads"] * (m["a_dim"] + m["a_vdim"]) * 2.0
    att_pre = att_flops / (rep_pre["latent_attention"] * 1e-3) / 1e12
    att_bytes = n_att * NB * ctx * m["a_kv"] * R * 2.0
    att_dec = att_bytes / (rep_dec["latent_attention"] * 1e-3) / 1e9
    # recurrences: 5 (gated linear attention) / 7 (delta rule) float operations per state element and token; decoding moves the state twice
    el = n_gla * m["g_heads"] * m["g_dim"] * m["g_vdim"], n_att * m["d_heads"] * m["d_dim"] * m["d_vdim"]
    scan_pre = T * (5.0 * el[0] + 7.0 * el[1]) / (ops_pre["recurrent_scan"] * 1e-3) / 1e12
    scan_dec = NB * (el[0] + el[1]) * 4.0 * 2 / (ops_dec["recurrent_scan"] * 1e-3) / 1e9
    moe_flops = LAYERS * T * s["top"] * 3 * 2.0 * s["ff"] * D
    moe_pre = moe_flops / (ops_pre["moe_experts"] * 1e-3) / 1e12
    moe_bytes = LAYERS * min(s["experts"], NB * s["top"]) * 3 * s["ff"] * D * 2.0
    moe_dec = moe_bytes / (rep_dec["moe_experts"] * 1e-3) / 1e9
    # stream kernels: read S streams per sublayer, rewrite S streams (read + write) per sublayer, float
    hc_bytes = LAYERS * 2 * (S * D * 4.0 + D * 2.0) + LAYERS * 2 * (2 * S * D * 4.0 + D * 2.0)
    hc_pre = T * hc_bytes / ((rep_pre["hc_read"] + rep_pre["hc_write"]) * 1e-3) / 1e9
    out = dict(model=f"Mumelix-{name}", sizes=m, prefill_tokens_per_s=T / pre * 1e3, prefill_ms=pre, decode_tokens_per_s=NB / dec * 1e3,
               decode_ms=dec, decode_from_hipgraph=graph_ok, decode_ms_eager=dec_eager, decode_ms_gpu_events=dec_events_ms, context=ctx,
               prefill_ops_ms=ops_pre, decode_ops_ms=ops_dec, prefill_kernels_ms=rep_pre, decode_kernels_ms=rep_dec,
               roofline=dict(prefill_attention_tflops=att_pre, prefill_attention_frac_bf16_peak=att_pre / BF16_PEAK_TFLOPS,
                             decode_attention_gbs=att_dec, decode_attention_frac_hbm=att_dec / HBM_PEAK_GBS,
                             prefill_experts_tflops=moe_pre, prefill_experts_frac_bf16_peak=moe_pre / BF16_PEAK_TFLOPS,
                             decode_experts_gbs=moe_dec, decode_experts_frac_hbm=moe_dec / HBM_PEAK_GBS,
                             prefill_recurrence_tflops=scan_pre, prefill_recurrence_frac_fp32_valu_peak=scan_pre / FP32_VALU_PEAK_TFLOPS,
                             decode_recurrence_gbs=scan_dec, decode_recurrence_frac_hbm=scan_dec / HBM_PEAK_GBS,
                             prefill_stream_kernels_gbs=hc_pre, prefill_stream_kernels_frac_hbm=hc_pre / HBM_PEAK_GBS))
    for sl in slots:
        eng.close_sequence(sl)
    del eng
    torch.cuda.empty_cache()
    return out


# ---- Vepolix ----------------------------------------------------------------------------------------------------------------
def vepolix_config(s, m):
    """Mumelix's sizes in Vepolix's layers: attention with the same heads and cache rows (chunks longer than the workload's
    contexts, so both attend over the same keys), a matrix memory of the gated-linear-attention state's size, the same experts
    (plus a shared one) on the recurrent layers and a dense unit of the active expert width on the attention layers."""
    a = {"type": "attention", "mlp": {"kind": "dense", "ff": s["top"] * s["ff"]},
         "mixer": {"heads": m["a_heads"], "kv_heads": m["a_kv"], "dim": m["a_dim"], "vdim": m["a_vdim"], "mask": {"size": 2048},
                   "bias_max": 1024, "scale": 1.0 / math.sqrt(m["a_dim"]), "v_mix": True}}
    r = {"type": "mlstm", "mixer": {"heads": m["g_heads"], "dim": m["g_dim"], "vdim": m["g_vdim"], "gate_cap": 20.0},
         "mlp": {"kind": "moe", "expert": {"ff": s["ff"]}, "shared": {"ff": s["ff"]},
                 "router": {"experts": s["experts"], "top": s["top"], "scale": 2.0, "groups": {"count": s["groups"], "keep": s["keep"]}}}}
    return {"architecture": "Vepolix", "width": s["width"], "vocab": VOCAB, "embedding": {"scale": 1.0}, "norm": {"eps": 1e-5},
            "layers": [a, r, a, r][:LAYERS]}


def vepolix_weights(cfg, dev, seed=0, bias_rows=32):
    g = torch.Generator(device=dev).manual_seed(seed)
    D, V = cfg["width"], cfg["vocab"]

    def mat(o, i, s=1.0):
        return (torch.randn((o, i), device=dev, generator=g) * (s / math.sqrt(i))).bfloat16()

    def vec(n, mean=1.0, s=0.1):
        return (mean + s * torch.randn((n,), device=dev, generator=g)).bfloat16()

    def unit(p, ff):
        W[p + "gate"], W[p + "up"], W[p + "down"] = mat(ff, D), mat(ff, D), mat(D, ff)

    W = {"embed": torch.randn((V, D), device=dev, generator=g).bfloat16(), "head": mat(V, D), "final.norm": vec(D)}
    for i, L in enumerate(cfg["layers"]):
        p, x = f"l{i}.", L["mixer"]
        W[p + "norm1"] = vec(D)
        q = p + "mix."
        if L["type"] == "attention":
            H, G, d, dv = x["heads"], x["kv_heads"], x["dim"], x["vdim"]
            W.update({q + "q": mat(H * d, D), q + "k": mat(G * d, D), q + "v": mat(G * dv, D), q + "o": mat(D, H * dv), q + "q.norm": vec(H * d),
                      q + "k.norm": vec(G * d), q + "rel": vec(bias_rows * H, 0.0, 1.0).view(bias_rows, H), q + "vmix": torch.tensor(0.3).bfloat16()})
        else:
            H, d, dv = x["heads"], x["dim"], x["vdim"]
            W.update({q + "q": mat(H * d, D), q + "k": mat(H * d, D), q + "v": mat(H * dv, D), q + "g": mat(H * dv, D), q + "o": mat(D, H * dv),
                      q + "norm": vec(H * dv), q + "i": mat(H, D), q + "i.b": vec(H, 0.0, 1.0), q + "f": mat(H, D), q + "f.b": vec(H, 3.0, 1.0)})
        mlp, q = L["mlp"], p + "mlp."
        if mlp["kind"] == "dense":
            unit(q, mlp["ff"])
        else:
            for e in range(mlp["router"]["experts"]):
                unit(f"{q}e{e}.", mlp["expert"]["ff"])
            unit(q + "shared.", mlp["shared"]["ff"])
            W[q + "router"], W[q + "correction"] = mat(mlp["router"]["experts"], D, 3.0), vec(mlp["router"]["experts"], 0.0, 0.1)
    return W


def bench_vepolix(name, s, dev, steps, warmup):
    from ..models.vepolix import Vepolix
    from .engine import Engine
    m = MUMELIX[name]
    cfg = vepolix_config(s, m)
    NB, L, BP = 64, 1024, 8
    eng = Engine(Vepolix, cfg, vepolix_weights(cfg, dev), dtype="bfloat16", device=dev, max_tokens=NB * (L + 384), max_seqs=NB)
    timer = OpTimer(eng.ops)
    g = torch.Generator().manual_seed(1)
    prompts = [torch.randint(0, VOCAB, (L,), generator=g).tolist() for _ in range(NB)]
    slots = [eng.open_sequence() for _ in range(NB)]
    small = ("latent_attention", "add_rms_norm", "normed_attention_prep", "max_gates", "head_rms_gate", "recurrent_scan")
    pre_ms, ops_pre, rep_pre = [], None, {}
    for i in range(0, NB, BP):
        items = [(slots[j], prompts[j]) for j in range(i, i + BP)]
        want = [k * L + L - 1 for k in range(BP)]
        if i == BP:                                          # one step with events around every launch
            ops_pre, _ = timer.step(lambda: eng.execute(items, want))
            rep_pre = {k: timer.replay(k, 3) for k in small if k != "recurrent_scan" and k != "max_gates"}   # (these two advance state)
            continue
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        eng.execute(items, want)
        torch.cuda.synchronize()
        if i > 0:
            pre_ms.append((time.perf_counter() - t0) * 1e3)
    pre = sorted(pre_ms)[len(pre_ms) // 2]
    nxt = [[int(torch.randint(0, VOCAB, (1,), generator=g))] for _ in range(NB)]
    want = list(range(NB))

    def decode():
        eng.execute([(slots[j], nxt[j]) for j in range(NB)], want)

    dec_eager = timed(decode, steps, warmup)
    ops_dec, dec_events_ms = timer.step(decode)
    rep_dec = {k: timer.replay(k, 20) for k in ("latent_attention", "moe_experts", "add_rms_norm", "normed_attention_prep", "head_rms_gate")}
    eng.decode_graphs = True
    dec = timed(decode, steps, warmup)
    graph_ok = any(v is not False for v in eng._graphs.values()) and bool(eng._graphs)
    ctx = eng.cache.length[slots[0]]
    T, D = BP * L, s["width"]
    n_att = sum(1 for x in cfg["layers"] if x["type"] == "attention")
    n_rec = LAYERS - n_att
    R = m["a_dim"] + m["a_vdim"]
    att_flops = n_att * BP * sum(p + 1 for p in range(L)) * m["a_heads"] * (m["a_dim"] + m["a_vdim"]) * 2.0
    att_pre = att_flops / (rep_pre["latent_attention"] * 1e-3) / 1e12
    att_bytes = n_att * NB * ctx * m["a_kv"] * R * 2.0
    att_dec = att_bytes / (rep_dec["latent_attention"] * 1e-3) / 1e9
    # recurrence: 5 float operations per state element and token (decay, k v, add; q S, add); decoding moves the state twice
    el = n_rec * m["g_heads"] * m["g_dim"] * m["g_vdim"]
    scan_pre = T * 5.0 * el / (ops_pre["recurrent_scan"] * 1e-3) / 1e12
    scan_dec = NB * el * 4.0 * 2 / (ops_dec["recurrent_scan"] * 1e-3) / 1e9
    moe_flops = n_rec * T * s["top"] * 3 * 2.0 * s["ff"] * D
    moe_pre = moe_flops / (ops_pre["moe_experts"] * 1e-3) / 1e12
    moe_bytes = n_rec * min(s["experts"], NB * s["top"]) * 3 * s["ff"] * D * 2.0
    moe_dec = moe_bytes / (rep_dec["moe_experts"] * 1e-3) / 1e9
    # residual kernel: reads and writes the float stream, reads the sublayers' outputs (2 on attention layers, 3 on the others),
    # writes the next input; the first call only norms, the last only adds
    res_bytes = T * (LAYERS * (8.0 * D + 2.0 * D) + (2 * n_att + 3 * n_rec) * 2.0 * D)
    res_pre = res_bytes / (rep_pre["add_rms_norm"] * 1e-3) / 1e9
    out = dict(model=f"Vepolix-{name}", sizes=m, prefill_tokens_per_s=T / pre * 1e3, prefill_ms=pre, decode_tokens_per_s=NB / dec * 1e3,
               decode_ms=dec, decode_from_hipgraph=graph_ok, decode_ms_eager=dec_eager, decode_ms_gpu_events=dec_events_ms, context=ctx,
               prefill_ops_ms=ops_pre, decode_ops_ms=ops_dec, prefill_kernels_ms=rep_pre, decode_kernels_ms=rep_dec,
               roofline=dict(prefill_attention_tflops=att_pre, prefill_attention_frac_bf16_peak=att_pre / BF16_PEAK_TFLOPS,
                             decode_attention_gbs=att_dec, decode_attention_frac_hbm=att_dec / HBM_PEAK_GBS,
                             prefill_experts_tflops=moe_pre, prefill_experts_frac_bf16_peak=moe_pre / BF16_PEAK_TFLOPS,
                             decode_experts_gbs=moe_dec, decode_experts_frac_hbm=moe_dec / HBM_PEAK_GBS,
                             prefill_recurrence_tflops=scan_pre, prefill_recurrence_frac_fp32_valu_peak=scan_pre / FP32_VALU_PEAK_TFLOPS,
                             decode_recurrence_gbs=scan_dec, decode_recurrence_frac_hbm=scan_dec / HBM_PEAK_GBS,
                             prefill_residual_kernel_gbs=res_pre, prefill_residual_kernel_frac_hbm=res_pre / HBM_PEAK_GBS))
    for sl in slots:
        eng.close_sequence(sl)
    del eng
    torch.cuda.empty_cache()
    return out


# ---- Pemolorn ---------------------------------------------------------------------------------------------------------------
PEMOLORN_WINDOW, PEMOLORN_POOL, PEMOLORN_KEEP = 512, 64, 64


def pemolorn_config(s, m):
    """Mumelix's sizes in Pemolorn's layers: the attention heads and cache rows of its parallel layers, a minGRU as wide as the model
    beside them, the same experts (plus four identity experts).  Layers: parallel (window 512 + pooled blocks of 64, dense unit of the
    active expert width), attention (window over the whole context, 64 kept tokens), parallel, attention on the second layer's cache."""
    att = {"heads": m["a_heads"], "kv_heads": m["a_kv"], "dim": m["a_dim"], "vdim": m["a_vdim"], "scale": 1.0 / math.sqrt(m["a_dim"])}
    moe = {"kind": "moe", "expert": {"ff": s["ff"], "limit": 7.0}, "router": {"experts": s["experts"], "identity": 4, "top": s["top"]}}
    left = dict(att, conv=m["taps"], mask={"size": PEMOLORN_WINDOW, "pool": PEMOLORN_POOL}, rot={"base": 500000.0, "dims": m["rot"]})
    p = {"type": "parallel", "mixer": {"left": left, "right": {"width": s["width"]}}}
    a = {"type": "attention", "mixer": dict(att, mask={"size": 2048, "keep_first": PEMOLORN_KEEP}), "mlp": moe}
    shared = {"type": "attention", "mixer": dict(a["mixer"], kv_from=1), "mlp": moe}
    return {"architecture": "Pemolorn", "width": s["width"], "vocab": VOCAB, "norm": {"eps": 1e-5},
            "layers": [dict(p, mlp={"kind": "dense", "ff": s["top"] * s["ff"]}), a, dict(p, mlp=moe), shared][:LAYERS]}


def pemolorn_weights(cfg, dev, seed=0):
    g = torch.Generator(device=dev).manual_seed(seed)
    D, V = cfg["width"], cfg["vocab"]

    def mat(o, i, s=1.0):
        return (torch.randn((o, i), device=dev, generator=g) * (s / math.sqrt(i))).bfloat16()

    def vec(n, mean=1.0, s=0.1):
        return (mean + s * torch.randn((n,), device=dev, generator=g)).bfloat16()

    def one(mean=1.0):
        return vec(1, mean).reshape(())

    W = {"embed": torch.randn((V, D), device=dev, generator=g).bfloat16(), "head": mat(V, D), "final.norm": one()}
    for i, L in enumerate(cfg["layers"]):
        p, x = f"l{i}.", L["mixer"]
        for n in ("norm1", "norm1b", "norm2", "norm2b"):
            W[p + n] = one()

        def attention(q, a, whole, own=True):
            H, G, d, dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            W.update({q + "q": mat(H * d, D), q + "o": mat(D, H * dv), q + "sink": vec(H, 0.0, 1.0), q + "q.norm": vec(H * d if whole else d)})
            if own:
                W.update({q + "k": mat(G * d, D), q + "v": mat(G * dv, D), q + "k.norm": vec(G * d if whole else d)})
            if a.get("conv"):
                W.update({q + "q.conv": mat(H * d, a["conv"]), q + "k.conv": mat(G * d, a["conv"]), q + "v.conv": mat(G * dv, a["conv"])})

        if L["type"] == "parallel":
            attention(p + "mix.left.", x["left"], True)
            n, q = x["right"]["width"], p + "mix.right."
            W.update({q + "z": mat(n, D), q + "x": mat(n, D), q + "g": mat(n, D), q + "o": mat(D, n), q + "z.b": vec(n, 0.0, 1.0),
                      q + "x.b": vec(n, 0.0, 1.0), p + "mix.left.out": vec(D), p + "mix.right.out": vec(D)})
        else:
            attention(p + "mix.", x, False, own=x.get("kv_from") is None)
        mlp, q = L["mlp"], p + "mlp."
        if mlp["kind"] == "dense":
            W[q + "up"], W[q + "down"] = mat(mlp["ff"], D), mat(D, mlp["ff"])
        else:
            r = mlp["router"]
            for e in range(r["experts"]):
                W[f"{q}e{e}.gate"], W[f"{q}e{e}.up"], W[f"{q}e{e}.down"] = mat(mlp["expert"]["ff"], D), mat(mlp["expert"]["ff"], D), mat(D, mlp["expert"]["ff"])
            n = r["experts"] + r["identity"]
            W[q + "router"], W[q + "correction"] = mat(n, D, 3.0), vec(n, 0.0, 0.02)
    return W


def bench_pemolorn(name, s, dev, steps, warmup):
    from ..models.pemolorn import Pemolorn
    from .engine import Engine
    m = MUMELIX[name]
    cfg = pemolorn_config(s, m)
    NB, L, BP = 64, 1024, 8
    eng = Engine(Pemolorn, cfg, pemolorn_weights(cfg, dev), dtype="bfloat16", device=dev, max_tokens=NB * (L + 384), max_seqs=NB)
    timer = OpTimer(eng.ops)
    g = torch.Generator().manual_seed(1)
    prompts = [torch.randint(0, VOCAB, (L,), generator=g).tolist() for _ in range(NB)]
    slots = [eng.open_sequence() for _ in range(NB)]
    stateless = ("latent_attention", "add_normed_rms_norm", "qk_norm_rope_prep", "pool_blocks", "rms_pair_mean")
    pre_ms, ops_pre, rep_pre = [], None, {}
    for i in range(0, NB, BP):
        items = [(slots[j], prompts[j]) for j in range(i, i + BP)]
        want = [k * L + L - 1 for k in range(BP)]
        if i == BP:                                          # one step with events around every launch
            ops_pre, _ = timer.step(lambda: eng.execute(items, want))
            rep_pre = {k: timer.replay(k, 3) for k in stateless}      # (the scan and the convolution advance state: timed in the step)
            continue
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        eng.execute(items, want)
        torch.cuda.synchronize()
        if i > 0:
            pre_ms.append((time.perf_counter() - t0) * 1e3)
    pre = sorted(pre_ms)[len(pre_ms) // 2]
    nxt = [[int(torch.randint(0, VOCAB, (1,), generator=g))] for _ in range(NB)]
    want = list(range(NB))

    def decode():
        eng.execute([(slots[j], nxt[j]) for j in range(NB)], want)

    dec_eager = timed(decode, steps, warmup)
    ops_dec, dec_events_ms = timer.step(decode)
    rep_dec = {k: timer.replay(k, 20) for k in ("latent_attention", "moe_experts", "add_normed_rms_norm", "qk_norm_rope_prep")}
    eng.decode_graphs = True
    dec = timed(decode, steps, warmup)
    graph_ok = any(v is not False for v in eng._graphs.values()) and bool(eng._graphs)
    ctx = eng.cache.length[slots[0]]
    T, D = BP * L, s["width"]
    kinds = [x["type"] for x in cfg["layers"]]
    n_par, n_att = kinds.count("parallel"), kinds.count("attention")
    n_moe = sum(1 for x in cfg["layers"] if x["mlp"]["kind"] == "moe")
    R = m["a_dim"] + m["a_vdim"]
    W_, P_ = PEMOLORN_WINDOW, PEMOLORN_POOL

    def seen(p, kind):                                       # keys a query at position p scores
        return p + 1 if kind == "attention" else min(p + 1, W_) + max(0, p - W_ + 1) // P_

    # attention: useful work = q.k over dim and p.v over vdim for every visible key (the kernel also multiplies the query's zero half)
    att_flops = sum(BP * sum(seen(p, k) for p in range(L)) for k in kinds) * m["a_heads"] * R * 2.0
    att_pre = att_flops / (rep_pre["latent_attention"] * 1e-3) / 1e12
    att_bytes = sum(NB * seen(ctx - 1, k) for k in kinds) * m["a_kv"] * R * 2.0
    att_dec = att_bytes / (rep_dec["latent_attention"] * 1e-3) / 1e9
    # the element-wise recurrence moves three pre-activations in and one value out per token and channel (bfloat16)
    scan_bytes = n_par * D * 4 * 2.0
    scan_pre = T * scan_bytes / (ops_pre["min_gru_scan"] * 1e-3) / 1e9
    scan_dec = NB * (scan_bytes + n_par * D * 8.0) / (ops_dec["min_gru_scan"] * 1e-3) / 1e9      # (+ the float state in and out)
    active = s["top"] * s["experts"] / (s["experts"] + 4.0)  # chosen router outputs that are experts with weights, on average
    moe_flops = n_moe * T * active * 3 * 2.0 * s["ff"] * D
    moe_pre = moe_flops / (ops_pre["moe_experts"] * 1e-3) / 1e12
    moe_bytes = n_moe * min(s["experts"], NB * s["top"]) * 3 * s["ff"] * D * 2.0
    moe_dec = moe_bytes / (rep_dec["moe_experts"] * 1e-3) / 1e9
    # residual kernel: per sublayer the float stream in and out, the sublayer's output in, the next input out; the first call only norms
    res_bytes = T * (2 * LAYERS * (8.0 * D + 4.0 * D) + 4.0 * D + 2.0 * D)
    res_pre = res_bytes / (rep_pre["add_normed_rms_norm"] * 1e-3) / 1e9
    out = dict(model=f"Pemolorn-{name}", sizes=m, prefill_tokens_per_s=T / pre * 1e3, prefill_ms=pre, decode_tokens_per_s=NB / dec * 1e3,
               decode_ms=dec, decode_from_hipgraph=graph_ok, decode_ms_eager=dec_eager, decode_ms_gpu_events=dec_events_ms, context=ctx,
               prefill_ops_ms=ops_pre, decode_ops_ms=ops_dec, prefill_kernels_ms=rep_pre, decode_kernels_ms=rep_dec,
               roofline=dict(prefill_attention_tflops=att_pre, prefill_attention_frac_bf16_peak=att_pre / BF16_PEAK_TFLOPS,
                             decode_attention_gbs=att_dec, decode_attention_frac_hbm=att_dec / HBM_PEAK_GBS,
                             prefill_experts_tflops=moe_pre, prefill_experts_frac_bf16_peak=moe_pre / BF16_PEAK_TFLOPS,
                             decode_experts_gbs=moe_dec, decode_experts_frac_hbm=moe_dec / HBM_PEAK_GBS,
                             prefill_recurrence_gbs=scan_pre, prefill_recurrence_frac_hbm=scan_pre / HBM_PEAK_GBS,
                             decode_recurrence_gbs=scan_dec, decode_recurrence_frac_hbm=scan_dec / HBM_PEAK_GBS,
                             prefill_residual_kernel_gbs=res_pre, prefill_residual_kernel_frac_hbm=res_pre / HBM_PEAK_GBS))
    for sl in slots:
        eng.close_sequence(sl)
    del eng
    torch.cuda.empty_cache()
    return out


def main(args, helpers):
    dev = "cuda:0"
    torch.cuda.set_device(0)
    from .. import build
    import os
    if not os.path.exists(build.LIB):
        build.build(verbose=False)
    steps, warmup = min(args.steps, 32), min(args.warmup, 8)
    for name in args.design_sizes.split(","):
        if args.design in ("mumelix", "vepolix", "pemolorn") and name not in MUMELIX:      # (sizes that differ in a Vekalorn-only constant)
            continue
        s = SIZES[name]
        line = {"design": args.design, "size": name, "sizes": s, "layers": LAYERS, "vocab": VOCAB, "dtype": "bf16",
                "data": "synthetic", "workload": "prefill 8 x 1024 tokens in one step; decode 64 sequences at context 1024"}
        if args.design == "pemolorn":
            line["pemolorn"] = bench_pemolorn(name, s, dev, steps, warmup)
            line["mumelix"] = bench_mumelix(name, s, dev, steps, warmup)
        elif args.design == "vepolix":
            line["vepolix"] = bench_vepolix(name, s, dev, steps, warmup)
            line["mumelix"] = bench_mumelix(name, s, dev, steps, warmup)
        elif args.design == "mumelix":
            line["mumelix"] = bench_mumelix(name, s, dev, steps, warmup)
            line["vekalorn"] = bench_vekalorn(name, s, dev, steps, warmup)
        else:
            line["vekalorn"] = bench_vekalorn(name, s, dev, steps, warmup)
            line["llama_w4a8"] = bench_llama(name, s, dev, steps, warmup, helpers)
        print(json.dumps(line), flush=True)
    return 0
