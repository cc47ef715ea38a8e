"""The operations the served models are made of, in two forms with one signature:

* `HipOps`   - the product path: one launch of libqserve_serve.so per call (include/qserve_serve.h), on the current stream;
* `TorchOps` - the same operations written with unfused torch tensor ops on any device.  It exists to bring a layer up and
  to test host logic (cache, scheduler, batching) where no GPU is; an engine only uses it when asked to by name - a model on
  a GPU never falls back to it.

Conventions: `x` is the float residual stream [T, D]; `h` and every other activation is in the storage type (bfloat16 or
float32); matrix products are the vendor's (`linear`), with float accumulation.
"""
import torch

BF16, F32 = 0, 1


def dtype_code(dtype):
    if dtype == torch.bfloat16:
        return BF16
    if dtype == torch.float32:
        return F32
    raise ValueError(f"the serving kernels store bfloat16 or float32, not {dtype}")


def linear(x, w):
    """x [T, in] @ w [out, in]^T in the storage type (hipBLASLt / rocBLAS through torch; float accumulation)."""
    return torch.matmul(x, w.t())


class HipOps:
    name = "hip"

    def __init__(self, dtype):
        from ..serving._lib import check, lib
        self.dtype, self.code = dtype, dtype_code(dtype)
        self.L, self.check = lib(), check

    @staticmethod
    def _s():
        return torch.cuda.current_stream().cuda_stream

    def _need(self, *ts):
        for t in ts:
            if t is not None and not (t.is_cuda and t.is_contiguous()):
                raise RuntimeError("serving kernels need contiguous tensors on the GPU")

    def embed(self, tokens, table):
        T, D = tokens.numel(), table.size(1)
        x = torch.empty((T, D), dtype=torch.float32, device=table.device)
        h = torch.empty((T, D), dtype=self.dtype, device=table.device)
        self._need(tokens, table)
        self.check(self.L.qsv_embed(x.data_ptr(), h.data_ptr(), table.data_ptr(), tokens.data_ptr(), T, D, self.code, self._s()),
                   "embed")
        return x, h

    def add_layer_norm(self, x, y, w, eps):
        """x += layer_norm(y) * w in place; returns x in the storage type."""
        h = torch.empty(x.shape, dtype=self.dtype, device=x.device)
        self._need(x, y, w)
        assert y.shape == x.shape and y.dtype == self.dtype and x.dtype == torch.float32
        self.check(self.L.qsv_add_layer_norm(x.data_ptr(), h.data_ptr(), y.data_ptr(), w.data_ptr(), eps, x.size(0), x.size(1),
                                             self.code, self._s()), "add_layer_norm")
        return h

    def layer_norm_rows(self, x, rows, w, eps):
        n = x.size(0) if rows is None else rows.numel()
        out = torch.empty((n, x.size(1)), dtype=self.dtype, device=x.device)
        self._need(x, rows, w)
        self.check(self.L.qsv_layer_norm_rows(out.data_ptr(), x.data_ptr(), 0 if rows is None else rows.data_ptr(), w.data_ptr(),
                                              eps, n, x.size(1), self.code, self._s()), "layer_norm_rows")
        return out

    def latent_prep(self, down, q_off, q_rank, q_w, kv_off, kv_rank, kv_w, rot_dim, rot_n, rope, pool, slot, pos, eps):
        T = down.size(0)
        cq = torch.empty((T, q_rank), dtype=self.dtype, device=down.device)
        self._need(down, q_w, kv_w, rope, pool, slot, pos)
        assert pool.size(-1) == kv_rank + rot_dim and slot.dtype == torch.int64 and pos.dtype == torch.int32
        assert rope is None or (rope.dtype == torch.float32 and rope.size(-1) * 2 == rot_n)
        self.check(self.L.qsv_latent_prep(down.data_ptr(), down.stride(0), q_off, q_rank, q_w.data_ptr(), cq.data_ptr(), kv_off,
                                          kv_rank, kv_w.data_ptr(), rot_dim, rot_n, 0 if rope is None else rope.data_ptr(),
                                          pool.data_ptr(), slot.data_ptr(), pos.data_ptr(), eps, T, self.code, self._s()),
                   "latent_prep")
        return cq

    def latent_query(self, q, q_abs, rope, pos, scale, heads, dim, rot_dim, rot_n, rank):
        T = q.size(0)
        qf = torch.empty((T, heads, rank + rot_dim), dtype=torch.float32, device=q.device)
        self._need(q, q_abs, rope, pos)
        assert q.numel() == T * heads * (dim + rot_dim) and q_abs.shape == (heads, T, rank)
        self.check(self.L.qsv_latent_query(qf.data_ptr(), q.data_ptr(), q_abs.data_ptr(), 0 if rope is None else rope.data_ptr(),
                                           pos.data_ptr(), scale, T, heads, dim, rot_dim, rot_n, rank, self.code, self._s()),
                   "latent_query")
        return qf

    attention_split_target = 512        # workgroups a launch of the matrix-core attention should at least have

    def latent_attention(self, qf, pool, batch, window, rank, page, variant=0, key_splits=None, q_first=0, chunk=None, bias=None,
                         keep_first=0, sink=None, pooled=None, pool_block=0):
        """batch: the step's StepBatch (block table, sequence slot and position per token, work tiles).  variant: 0 = the
        matrix-core kernel where it takes the sizes, 1 = always the wave kernel.  key_splits: None = chosen from the number
        of workgroups and the context.  q_first: the caller's promise that every query is zero before that element.
        pool [rows, R]: one pool for all heads; [G, rows, R]: head h reads pool h // (H / G), all in one launch.
        chunk: a query sees only the keys of its own chunk of that many positions.  bias: float [H, n], bias[h, min(i - j, n - 1)]
        is added to the score of query i and key j.  keep_first: the first that many positions of the sequence stay visible
        behind the window.  sink float [H]: exp(sink[h]) joins the softmax's denominator (no key, no value).  pooled (shaped like
        pool, ceil(page / pool_block) rows per page, written by `pool_blocks`): one more key / value row per block of pool_block
        positions that lies wholly before the window."""
        T, H, R = qf.shape
        assert sink is None or (sink.dtype == torch.float32 and sink.numel() == H and sink.is_contiguous())
        assert pooled is None or (window and pool_block > 0 and bias is None and not chunk and not keep_first and pooled.dim() == pool.dim()
                                  and pooled.dtype == pool.dtype and pooled.size(-1) == R)
        assert not keep_first or (window and not chunk)
        per_page = (page + pool_block - 1) // pool_block if pooled is not None else 0
        assert pooled is None or pooled.size(-2) == pool.size(-2) // page * per_page
        more = (int(keep_first or 0), 0 if sink is None else sink.data_ptr(), 0 if pooled is None else pooled.data_ptr(),
                0 if pooled is None or pooled.dim() == 2 else pooled.stride(0), int(pool_block) if pooled is not None else 0, per_page)
        assert bias is None or (bias.dtype == torch.float32 and bias.dim() == 2 and bias.size(0) == H and bias.is_contiguous())
        extra = (int(chunk or 0), 0 if bias is None else bias.data_ptr(), 0 if bias is None else bias.size(1))
        block_table, seq, pos = batch.block_table, batch.seq, batch.pos
        out = torch.empty((T, H, rank), dtype=self.dtype, device=qf.device)
        self._need(qf, pool, block_table, seq, pos, pooled)
        assert pool.size(-1) == R and block_table.dtype == torch.int32 and seq.dtype == torch.int32
        per, pool_stride = (H, 0) if pool.dim() == 2 else (H // pool.size(0), pool.stride(0))
        assert pool.dim() == 2 or H % pool.size(0) == 0
        if variant == 0 and page % 32 == 0 and self.L.qsv_latent_attention_mfma_ok(rank, R, self.code):
            tiles = batch.tiles(self.L.qsv_latent_attention_tile_tokens(per))
            # few workgroups and long contexts (decoding): cut the keys over several workgroups, merged by a second launch
            groups = tiles.size(0) * (H // per) * ((per + 31) // 32)
            span = min(batch.max_pos + 1, int(window)) if window else batch.max_pos + 1
            span = min(span, int(chunk)) if chunk else span
            span += int(keep_first or 0) + (batch.max_pos // pool_block if pooled is not None else 0)
            # (rows wider than 320 elements: one workgroup per CU at a time - a launch of one round of workgroups is the aim)
            target = self.attention_split_target // 2 if R > 320 else self.attention_split_target
            splits = max(1, min(target // max(groups, 1), span // 128, 32)) if key_splits is None else key_splits
            po = pm = None
            if splits > 1:
                po = torch.empty((splits, T, H, rank), dtype=torch.float32, device=qf.device)
                pm = torch.empty((splits, T, H, 2), dtype=torch.float32, device=qf.device)
            self.check(self.L.qsv_latent_attention_mfma(out.data_ptr(), qf.data_ptr(), pool.data_ptr(), block_table.data_ptr(),
                                                        block_table.stride(0), pos.data_ptr(), tiles.data_ptr(), tiles.size(0),
                                                        int(window or 0), H, rank, R, page, splits,
                                                        0 if po is None else po.data_ptr(), 0 if pm is None else pm.data_ptr(), T,
                                                        int(q_first), per, pool_stride, *extra, *more, self._s()), "latent_attention_mfma")
            return out
        self.check(self.L.qsv_latent_attention(out.data_ptr(), qf.data_ptr(), pool.data_ptr(), block_table.data_ptr(),
                                               block_table.stride(0), seq.data_ptr(), pos.data_ptr(), int(window or 0), T, H,
                                               rank, R, page, per, pool_stride, *extra, *more, self.code, variant, self._s()),
                   "latent_attention")
        return out

    def sigmoid_gate(self, o, g):
        """o [T, n] *= sigmoid(g [T, n]) in place; g may be a column slice of a wider matrix."""
        self._need(o)
        assert g.is_cuda and g.stride(1) == 1 and g.shape == o.shape
        self.check(self.L.qsv_sigmoid_gate(o.data_ptr(), g.data_ptr(), g.stride(0), o.size(0), o.size(1), self.code, self._s()),
                   "sigmoid_gate")
        return o

    # ---- streams, position-free norm, token shift -----------------------------------------------------------------------------
    def embed_streams(self, tokens, table, scale, streams):
        T, D = tokens.numel(), table.size(1)
        x = torch.empty((T, streams, D), dtype=torch.float32, device=table.device)
        self._need(tokens, table)
        self.check(self.L.qsv_embed_streams(x.data_ptr(), table.data_ptr(), tokens.data_ptr(), float(scale), T, streams, D, self.code,
                                            self._s()), "embed_streams")
        return x

    def hc_read(self, x, w_in, norm, shift=None, batch=None, prev=None):
        """-> the sublayer's input [T, D] (storage type): norm(sum_s w_in[s] x[:, s]), token-shifted if `shift` is given (then
        `prev` is the sequences' two-copy state [2 slots, D] and `batch` names each token's run and state rows)."""
        w, b, alpha = norm
        T, S, D = x.shape
        h = torch.empty((T, D), dtype=self.dtype, device=x.device)
        self._need(x, w_in, w, b, shift, prev)
        assert x.dtype == torch.float32 and w_in.dtype == torch.float32 and w_in.numel() == S
        p = [0, 0, 0, 0, 0]
        if shift is not None:
            assert prev.dtype == torch.float32 and prev.size(-1) == D and shift.dtype == self.dtype
            p = [shift.data_ptr(), prev.data_ptr(), batch.run_off.data_ptr(), batch.state_rd.data_ptr(), batch.state_wr.data_ptr()]
        self.check(self.L.qsv_hc_read(h.data_ptr(), x.data_ptr(), w_in.data_ptr(), w.data_ptr(), b.data_ptr(), float(alpha), *p,
                                      T, S, D, self.code, self._s()), "hc_read")
        return h

    def hc_write(self, x, y, w_mix, w_out, then_read=None):
        """All streams rewritten in place from the sublayer's output y.  then_read = (w_in, norm) of the NEXT sublayer, if it
        reads without a token shift: its input comes out of the same pass -> h [T, D] (else None)."""
        T, S, D = x.shape
        self._need(x, y, w_mix, w_out)
        assert y.shape == (T, D) and y.dtype == self.dtype and w_mix.dtype == torch.float32 and w_mix.shape == (S, S)
        h, nxt = None, [0, 0, 0, 0, 0.0]
        if then_read is not None:
            w_in, (w, b, alpha) = then_read
            h = torch.empty((T, D), dtype=self.dtype, device=x.device)
            nxt = [h.data_ptr(), w_in.data_ptr(), w.data_ptr(), b.data_ptr(), float(alpha)]
        self.check(self.L.qsv_hc_write(x.data_ptr(), y.data_ptr(), w_mix.data_ptr(), w_out.data_ptr(), T, S, D, *nxt, self.code,
                                       self._s()), "hc_write")
        return h

    def dyt_sum_rows(self, x, rows, norm):
        w, b, alpha = norm
        T, S, D = x.shape
        n = T if rows is None else rows.numel()
        out = torch.empty((n, D), dtype=self.dtype, device=x.device)
        self._need(x, rows, w, b)
        self.check(self.L.qsv_dyt_sum_rows(out.data_ptr(), x.data_ptr(), 0 if rows is None else rows.data_ptr(), w.data_ptr(),
                                           b.data_ptr(), float(alpha), n, S, D, self.code, self._s()), "dyt_sum_rows")
        return out

    def rms_pair_mean(self, a, wa, b, wb, eps):
        out = torch.empty_like(a)
        self._need(a, wa, b, wb)
        assert a.shape == b.shape and a.dtype == self.dtype and b.dtype == self.dtype
        self.check(self.L.qsv_rms_pair_mean(out.data_ptr(), a.data_ptr(), wa.data_ptr(), b.data_ptr(), wb.data_ptr(), eps, a.size(0),
                                            a.size(1), self.code, self._s()), "rms_pair_mean")
        return out

    GLU_ACTS = {"silu": 0, "gelu_tanh": 1, "clamped": 2}

    def glu(self, a, act="silu", limit=0.0):
        """a [n, 2 ff] with (gate, up) as neighbours -> act(gate) * up [n, ff]; act: silu, gelu_tanh (gelu in its tanh form), or
        clamped: g = min(gate, limit), u = clamp(up, -limit, limit) -> g sigmoid(1.702 g) (u + 1)."""
        n, ff = a.size(0), a.size(1) // 2
        out = torch.empty((n, ff), dtype=self.dtype, device=a.device)
        self._need(a)
        self.check(self.L.qsv_glu(out.data_ptr(), a.data_ptr(), n, ff, self.GLU_ACTS[act], float(limit), self.code, self._s()), "glu")
        return out

    # ---- sinusoidal positions, RMS-normed residual, whole-projection query / key norms ----------------------------------------------
    def embed_sinusoid(self, tokens, pos, table, freq, scale):
        """-> float x [T, D] = table[tokens] * scale + the sinusoidal vector of each position (freq float [(D + 1) // 2])."""
        T, D = tokens.numel(), table.size(1)
        x = torch.empty((T, D), dtype=torch.float32, device=table.device)
        self._need(tokens, pos, table, freq)
        assert freq.dtype == torch.float32 and freq.numel() == (D + 1) // 2
        self.check(self.L.qsv_embed_sinusoid(x.data_ptr(), table.data_ptr(), tokens.data_ptr(), pos.data_ptr(), freq.data_ptr(),
                                             float(scale), T, D, self.code, self._s()), "embed_sinusoid")
        return x

    def add_rms_norm(self, x, ys, w, eps):
        """x += sum of ys (up to three sublayer outputs, storage type) in place; -> rms_norm(x) * w in the storage type (None if
        w is None)."""
        ys = [y for y in ys if y is not None]
        assert len(ys) <= 3 and all(y.shape == x.shape and y.dtype == self.dtype for y in ys) and x.dtype == torch.float32
        h = None if w is None else torch.empty(x.shape, dtype=self.dtype, device=x.device)
        self._need(x, w, *ys)
        p = [y.data_ptr() for y in ys] + [0] * (3 - len(ys))
        self.check(self.L.qsv_add_rms_norm(x.data_ptr(), 0 if h is None else h.data_ptr(), *p, 0 if w is None else w.data_ptr(),
                                           float(eps), x.size(0), x.size(1), self.code, self._s()), "add_rms_norm")
        return h

    def rms_norm_rows(self, x, rows, w, eps):
        n = x.size(0) if rows is None else rows.numel()
        out = torch.empty((n, x.size(1)), dtype=self.dtype, device=x.device)
        self._need(x, rows, w)
        self.check(self.L.qsv_rms_norm_rows(out.data_ptr(), x.data_ptr(), 0 if rows is None else rows.data_ptr(), w.data_ptr(),
                                            float(eps), n, x.size(1), self.code, self._s()), "rms_norm_rows")
        return out

    def normed_attention_prep(self, proj, q_off, k_off, v_off, heads, kv_heads, dim, vdim, q_w, k_w, eps, scale, v_first, mix, pool,
                              batch):
        """-> float queries [T, heads, vdim + dim] = [0 | normed q * scale]; writes the cache rows [v' | normed k] of the step's
        tokens.  v_first: [T, kv_heads * vdim] (a column slice is fine) or None; mix: the blend's weight on v_first."""
        T = proj.size(0)
        qf = torch.empty((T, heads, vdim + dim), dtype=torch.float32, device=proj.device)
        self._need(proj, q_w, k_w, pool, batch.slot)
        assert pool.shape[0] == kv_heads and pool.shape[2] == vdim + dim and pool.dtype == self.dtype and proj.dtype == self.dtype
        assert v_first is None or (v_first.dtype == self.dtype and v_first.stride(1) == 1 and v_first.shape == (T, kv_heads * vdim))
        self.check(self.L.qsv_normed_attention_prep(qf.data_ptr(), pool.data_ptr(), pool.size(1), proj.data_ptr(), proj.stride(0),
                                                    q_off, k_off, v_off, heads, kv_heads, dim, vdim, q_w.data_ptr(), k_w.data_ptr(),
                                                    float(eps), float(scale), 0 if v_first is None else v_first.data_ptr(),
                                                    0 if v_first is None else v_first.stride(0), float(mix), batch.slot.data_ptr(),
                                                    T, self.code, self._s()), "normed_attention_prep")
        return qf

    def max_gates(self, proj, i_off, f_off, bias_i, bias_f, cap, m_state, batch, heads):
        """Exponential gates with a running maximum from the pre-activations proj[:, i_off : i_off + heads] / [f_off : ...]; m_state
        float [slots, heads].  -> (decay a, input scale b, maximum m), float [T, heads] each."""
        T = proj.size(0)
        a, b, m = (torch.empty((T, heads), dtype=torch.float32, device=proj.device) for _ in range(3))
        self._need(bias_i, bias_f, m_state)
        assert proj.stride(1) == 1 and proj.dtype == self.dtype and bias_i.dtype == bias_f.dtype == m_state.dtype == torch.float32
        assert m_state.shape[1:] == (heads,) and bias_i.numel() == bias_f.numel() == heads
        runs = batch.runs()
        el = proj.element_size()
        self.check(self.L.qsv_max_gates(a.data_ptr(), b.data_ptr(), m.data_ptr(), proj.data_ptr() + i_off * el,
                                        proj.data_ptr() + f_off * el, proj.stride(0), bias_i.data_ptr(), bias_f.data_ptr(), float(cap),
                                        m_state.data_ptr(), runs.data_ptr(), runs.size(0), heads, self.code, self._s()), "max_gates")
        return a, b, m

    # ---- attention with rotated keys and values: rotations + cache write ---------------------------------------------------------
    def attention_prep(self, proj, q_off, k_off, v_off, heads, kv_heads, dim, vdim, rot_n, rope_k, rope_v, scale, pool, batch):
        T = proj.size(0)
        qf = torch.empty((T, heads, vdim + dim), dtype=torch.float32, device=proj.device)
        self._need(proj, rope_k, rope_v, pool, batch.slot, batch.pos)
        assert pool.shape[0] == kv_heads and pool.shape[2] == vdim + dim and pool.dtype == self.dtype and proj.dtype == self.dtype
        assert rope_k.size(-1) * 2 == rot_n and rope_v.size(-1) * 2 == vdim and rope_k.size(0) > batch.max_pos < rope_v.size(0)
        self.check(self.L.qsv_attention_prep(qf.data_ptr(), pool.data_ptr(), pool.size(1), proj.data_ptr(), proj.stride(0), q_off,
                                             k_off, v_off, heads, kv_heads, dim, vdim, rot_n, rope_k.data_ptr(), rope_v.data_ptr(),
                                             float(scale), batch.slot.data_ptr(), batch.pos.data_ptr(), T, self.code, self._s()),
                   "attention_prep")
        return qf

    def rotate_heads(self, o, rope, pos, sign):
        T, H, n = o.shape
        self._need(o, rope, pos)
        assert rope.size(-1) * 2 == n and o.dtype == self.dtype
        self.check(self.L.qsv_rotate_heads(o.data_ptr(), rope.data_ptr(), pos.data_ptr(), float(sign), T, H, n, self.code, self._s()),
                   "rotate_heads")
        return o


    # ---- sandwich norms, sink / kept-first / pooled-block attention, element-wise gated recurrence -----------------------------------
    def add_normed_rms_norm(self, x, y, w_post, w_next, eps):
        """x += rms_norm(y) * w_post in place (y None: nothing is added); -> rms_norm(x) * w_next in the storage type (None if
        w_next is None).  The weights hold one number (a gain for all coordinates) or one per coordinate."""
        T, D = x.shape
        h = None if w_next is None else torch.empty((T, D), dtype=self.dtype, device=x.device)
        self._need(x, y, w_post, w_next)
        assert x.dtype == torch.float32 and (y is None or (y.shape == x.shape and y.dtype == self.dtype and w_post is not None))
        for w in (w_post, w_next):
            assert w is None or (w.dtype == self.dtype and w.numel() in (1, D))
        self.check(self.L.qsv_add_normed_rms_norm(x.data_ptr(), 0 if h is None else h.data_ptr(), 0 if y is None else y.data_ptr(),
                                                  0 if y is None else w_post.data_ptr(), int(y is not None and w_post.numel() != 1),
                                                  0 if w_next is None else w_next.data_ptr(),
                                                  int(w_next is not None and w_next.numel() != 1), float(eps), T, D, self.code,
                                                  self._s()), "add_normed_rms_norm")
        return h

    def relu_sq(self, a):
        """a <- relu(a)^2 in place."""
        self._need(a)
        self.check(self.L.qsv_relu_sq(a.data_ptr(), a.numel(), self.code, self._s()), "relu_sq")
        return a

    def qk_norm_rope_prep(self, q, k, v, heads, kv_heads, dim, vdim, q_w, k_w, per_head, eps, rope, rot_n, scale, pool, batch):
        """q [T, heads * dim], k [T, kv_heads * dim], v [T, kv_heads * vdim] (float or storage type, column slices are fine; k and v
        None: the layer caches nothing).  Queries and keys are RMS-normed per head (weight [dim], shared by the heads) or over the
        whole projection (weight as wide as it), then the first rot_n dimensions of every head turn with the position (pairs of
        neighbours; rope float [positions, 2, rot_n / 2] or None).  -> float queries [T, heads, vdim + dim] = [0 | q * scale];
        writes the cache rows [v | k] of the step's tokens into pool [kv_heads, rows, vdim + dim]."""
        T = q.size(0)
        qf = torch.empty((T, heads, vdim + dim), dtype=torch.float32, device=q.device)
        self._need(q_w, k_w, rope, pool, batch.slot, batch.pos)
        assert q.stride(1) == 1 and q.size(1) == heads * dim and q_w.dtype == self.dtype and q_w.numel() == (dim if per_head else heads * dim)
        assert rope is None or (rope.dtype == torch.float32 and rope.size(-1) * 2 == rot_n and rot_n <= dim and rope.size(0) > batch.max_pos)
        kp = [0, 0, 0, 0, 0, 0, 0]
        if k is not None:
            assert k.dtype == v.dtype == q.dtype and k.stride(1) == v.stride(1) == 1 and k.size(1) == kv_heads * dim
            assert v.size(1) == kv_heads * vdim and k_w.dtype == self.dtype and k_w.numel() == (dim if per_head else kv_heads * dim)
            assert pool.shape[0] == kv_heads and pool.shape[2] == vdim + dim and pool.dtype == self.dtype
            kp = [k.data_ptr(), k.stride(0), v.data_ptr(), v.stride(0), k_w.data_ptr(), pool.data_ptr(), pool.size(1)]
        self.check(self.L.qsv_qk_norm_rope_prep(qf.data_ptr(), q.data_ptr(), q.stride(0), *kp[:4], dtype_code(q.dtype), heads, kv_heads,
                                                dim, vdim, q_w.data_ptr(), kp[4], int(bool(per_head)), float(eps),
                                                0 if rope is None else rope.data_ptr(), int(rot_n if rope is not None else 0),
                                                float(scale), kp[5], kp[6], batch.slot.data_ptr(), batch.pos.data_ptr(), T, self.code,
                                                self._s()), "qk_norm_rope_prep")
        return qf

    def pool_blocks(self, pool, pooled, batch, block, page):
        """For every token of the step that completes a block of `block` positions: the mean of the block's cache rows (as the pool
        holds them) goes into `pooled` [kv_heads, pages * ceil(page / block), row]: the block that starts in page p at offset o
        has row p * ceil(page / block) + o // block."""
        per_page = (page + block - 1) // block
        self._need(pool, pooled, batch.block_table, batch.seq, batch.pos)
        assert pool.dim() == 3 and pooled.dim() == 3 and pooled.size(0) == pool.size(0) and pooled.size(2) == pool.size(2)
        assert pooled.size(1) == pool.size(1) // page * per_page and pooled.dtype == pool.dtype == self.dtype
        self.check(self.L.qsv_pool_blocks(pooled.data_ptr(), pooled.size(1), pool.data_ptr(), pool.size(1), batch.block_table.data_ptr(),
                                          batch.block_table.stride(0), batch.seq.data_ptr(), batch.pos.data_ptr(), batch.n_tokens,
                                          pool.size(0), pool.size(2), int(block), int(page), per_page, self.code, self._s()),
                   "pool_blocks")

    def min_gru_scan(self, proj, z_off, x_off, g_off, b_z, b_x, state, batch, width):
        """Element-wise gated recurrence S <- (1 - z) S + z c with z = sigmoid(proj[:, z_off ..] + b_z), c = u + 1/2 (u >= 0) or
        sigmoid(u) (u < 0), u = proj[:, x_off ..] + b_x; state float [slots, width].  -> S * silu(proj[:, g_off ..]) [T, width]."""
        T = proj.size(0)
        out = torch.empty((T, width), dtype=self.dtype, device=proj.device)
        self._need(b_z, b_x, state)
        assert proj.stride(1) == 1 and proj.dtype == self.dtype and b_z.dtype == b_x.dtype == self.dtype and state.dtype == torch.float32
        assert state.shape[1:] == (width,) and b_z.numel() == b_x.numel() == width and max(z_off, x_off, g_off) + width <= proj.size(1)
        runs = batch.runs()
        self.check(self.L.qsv_min_gru_scan(out.data_ptr(), proj.data_ptr(), proj.stride(0), z_off, x_off, g_off, b_z.data_ptr(),
                                           b_x.data_ptr(), state.data_ptr(), runs.data_ptr(), runs.size(0),
                                           max(n for _, _, n in batch.items), width, self.code, self._s()), "min_gru_scan")
        return out

    # ---- recurrences ----------------------------------------------------------------------------------------------------------
    def decay(self, z, bias, a_log, tau, heads, dim):
        """z [T, heads * dim] (storage type; a column slice is fine) -> float decays: a_log given: exp(-exp(a_log[h]) softplus(z +
        bias)); else sigmoid(z + bias)^(1 / tau)."""
        T = z.size(0)
        out = torch.empty((T, heads * dim), dtype=torch.float32, device=z.device)
        self._need(bias, a_log)
        assert z.stride(1) == 1 and z.size(1) == heads * dim and z.dtype == self.dtype and bias.dtype == self.dtype
        assert a_log is None or (a_log.dtype == torch.float32 and a_log.numel() == heads)
        self.check(self.L.qsv_decay(out.data_ptr(), z.data_ptr(), z.stride(0), bias.data_ptr(), 0 if a_log is None else a_log.data_ptr(),
                                    float(tau), T, heads, dim, self.code, self._s()), "decay")
        return out

    def conv_silu_unit(self, proj, off, conv_w, hist, batch, n_unit, unit_dim, act="silu"):
        """Causal convolution over time of the columns [off, off + C) of proj with per-channel taps conv_w [C, taps], then silu
        (act "none": nothing), then the first n_unit groups of unit_dim channels made unit vectors.  hist: two-copy state, the last
        taps - 1 inputs of every sequence.  -> float [T, C]."""
        T = proj.size(0)
        C, taps = conv_w.shape
        out = torch.empty((T, C), dtype=torch.float32, device=proj.device)
        self._need(proj, conv_w, hist)
        assert conv_w.dtype == torch.float32 and hist.dtype == torch.float32 and hist.size(-1) == C and proj.dtype == self.dtype
        assert hist.size(1) == max(taps - 1, 1)
        self.check(self.L.qsv_conv_silu_unit(out.data_ptr(), proj.data_ptr(), proj.stride(0), off, C, taps, conv_w.data_ptr(),
                                             hist.data_ptr(), batch.run_off.data_ptr(), batch.state_rd.data_ptr(),
                                             batch.state_wr.data_ptr(), n_unit, unit_dim, {"none": 0, "silu": 1}[act], T, self.code, self._s()),
                   "conv_silu_unit")
        return out

    def recurrent_scan(self, q, k, v, decay, beta, state, batch, heads, qk_heads, dim, vdim, q_scale, kscale=None, v_cols=None):
        """q, k [T, qk_heads * dim], v [T, heads * vdim] (float or storage type, column slices are fine), decay float [T, heads *
        dim], beta [T, heads] raw (before the sigmoid) or None, state float [slots, heads, dim, vdim] -> o float [T, heads, vdim].
        decay of shape [T, heads]: one factor per head.  kscale float [T, heads]: multiplies k where it enters the state.
        v_cols < vdim: v is [T, heads * v_cols] and the state's column v_cols is fed with ones (a normaliser), the rest with zeros."""
        T = q.size(0)
        o = torch.empty((T, heads, vdim), dtype=torch.float32, device=q.device)
        self._need(decay, state, kscale)
        assert q.dtype == k.dtype == v.dtype and q.stride(1) == k.stride(1) == v.stride(1) == 1
        head_decay = decay.shape == (T, heads) and dim != 1
        assert state.shape[1:] == (heads, dim, vdim) and state.dtype == torch.float32 and (head_decay or decay.shape == (T, heads * dim))
        assert kscale is None or (kscale.dtype == torch.float32 and kscale.shape == (T, heads))
        assert v.size(1) == heads * (v_cols or vdim)
        runs = batch.runs()
        self.check(self.L.qsv_recurrent_scan(o.data_ptr(), q.data_ptr(), q.stride(0), k.data_ptr(), k.stride(0), v.data_ptr(),
                                             v.stride(0), dtype_code(q.dtype), decay.data_ptr(),
                                             0 if beta is None else beta.data_ptr(), 0 if beta is None else beta.stride(0),
                                             0 if beta is None else dtype_code(beta.dtype), state.data_ptr(), runs.data_ptr(),
                                             runs.size(0), max(n for _, _, n in batch.items), heads, qk_heads, dim, vdim,
                                             float(q_scale), 0 if kscale is None else kscale.data_ptr(), int(head_decay),
                                             int(v_cols or 0), self._s()), "recurrent_scan")
        return o

    def head_rms_gate(self, o, w, gate, kind, eps, vdim=None, den_m=None):
        """o float [T, H, n] -> [T, H * vdim] (storage type): per head o[..., :vdim] / its root mean square * w * gate_fn(gate).
        w [vdim] (shared by the heads) or [H * vdim].  den_m float [T, H] (then n > vdim): the read-out is first divided by
        max(|o[..., vdim]|, exp(-den_m)) + 1e-6."""
        T, H, n = o.shape
        dv = n if vdim is None else vdim
        out = torch.empty((T, H * dv), dtype=self.dtype, device=o.device)
        self._need(o, w, den_m)
        assert gate.stride(1) == 1 and gate.size(1) == H * dv and gate.dtype == self.dtype and w.dtype == self.dtype
        assert w.numel() in (dv, H * dv) and (den_m is None or (n > dv and den_m.shape == (T, H) and den_m.dtype == torch.float32))
        self.check(self.L.qsv_head_rms_gate(out.data_ptr(), o.data_ptr(), w.data_ptr(), gate.data_ptr(), gate.stride(0),
                                            {"silu": 0, "sigmoid": 1}[kind], eps, T, H, dv, n, int(w.numel() != dv),
                                            0 if den_m is None else den_m.data_ptr(), self.code, self._s()), "head_rms_gate")
        return out

    def moe_route(self, h, router, top_k, groups, keep, bias=None, renorm=False, score="softmax", correction=None, group_top=1,
                  scale=1.0):
        """-> (expert indices int32 [T, top_k], weights float [T, top_k]).  score: softmax over all experts, or sigmoid per expert;
        correction float [E]: added to the scores for the CHOICE only; group_top: a group's score is its largest choice score (1)
        or the sum of its two largest (2); weights = the chosen experts' scores (renorm: divided by their sum) times scale."""
        T, E = h.size(0), router.size(0)
        idx = torch.empty((T, top_k), dtype=torch.int32, device=h.device)
        wt = torch.empty((T, top_k), dtype=torch.float32, device=h.device)
        self._need(h, router, bias, correction)
        assert bias is None or (bias.dtype == self.dtype and bias.numel() == E)
        assert correction is None or (correction.dtype == torch.float32 and correction.numel() == E)
        self.check(self.L.qsv_moe_route(idx.data_ptr(), wt.data_ptr(), h.data_ptr(), router.data_ptr(),
                                        0 if bias is None else bias.data_ptr(), int(bool(renorm)), T, h.size(1), E, top_k,
                                        groups, keep, {"softmax": 0, "sigmoid": 1}[score],
                                        0 if correction is None else correction.data_ptr(), int(group_top), float(scale),
                                        self.code, self._s()), "moe_route")
        return idx, wt

    ACTS = {"none": 0, "relu_sq": 1, "swiglu": 2, "clamped_glu": 3}

    def moe_experts(self, h, up, down, idx, wt, act="relu_sq", limit=0.0):
        """up [E, rows, D], down [E, D, ff]; y[t] = sum_k wt[t, k] * down[idx[t, k]] a(up[idx[t, k]] h[t]).  act "relu_sq":
        a = relu(.)^2, rows = ff; "swiglu": up's rows come in pairs (2f = gate, 2f + 1 = up), a_f = silu(gate_f) up_f, rows = 2 ff;
        "clamped_glu": the same pairs with g = min(gate_f, limit), u = clamp(up_f, -limit, limit), a_f = g sigmoid(1.702 g) (u + 1).
        Indices at or above E (up.size(0)) name identity experts: their output is h[t] itself."""
        T, D = h.shape
        top_k, rows = idx.size(1), up.size(1)
        a = self.ACTS[act]
        ff = rows // 2 if a >= 2 else rows
        if (self.code == BF16 and self.moe_token_slots < T * top_k <= self.moe_expert_major_slots and D % 8 == 0 and ff % 8 == 0
                and D <= 4096 and ff <= 4096):
            return self._moe_experts_expert_major(h, up, down, idx, wt, a, limit)
        if T * top_k > self.moe_sorted_above:
            return self._moe_experts_sorted(h, up, down, idx, wt, a, limit)
        act = torch.empty((T, top_k, ff), dtype=self.dtype, device=h.device)
        y = torch.empty((T, D), dtype=self.dtype, device=h.device)
        self._need(h, up, down, idx, wt)
        assert up.shape[2] == D and down.shape == (up.size(0), D, ff)
        self.check(self.L.qsv_moe_up(act.data_ptr(), h.data_ptr(), up.data_ptr(), idx.data_ptr(), T, top_k, D, rows, a, float(limit),
                                     up.size(0), self.code, self._s()), "moe_up")
        self.check(self.L.qsv_moe_down(y.data_ptr(), act.data_ptr(), down.data_ptr(), idx.data_ptr(), wt.data_ptr(), T, top_k, D,
                                       ff, h.data_ptr(), up.size(0), self.code, self._s()), "moe_down")
        return y

    # More (token, expert) slots than this: sort the slots by expert and run each expert as one matrix product.  Below it the
    # per-token kernels above are used: no host synchronisation, a fixed launch sequence.
    moe_sorted_above = 64
    # the sorted form's products: the grouped matrix-core kernel (bfloat16, widths multiples of its K step) or one vendor product per expert
    moe_grouped_kernel = True

    # (token, expert) slots: up to moe_token_slots the per-token kernels (two launches); up to moe_expert_major_slots the
    # expert-major kernels (bfloat16; every expert weight read once, no host synchronisation); above, the expert-sorted vendor
    # products (compute-bound sizes)
    moe_token_slots = 8
    moe_expert_major_slots = 1024

    def _combine(self, h, ys, inv, idx, wt, E):
        """y[t] = sum_k wt[t, k] * (ys[inv[t K + k]], or h[t] where idx[t, k] names an identity expert)."""
        T, D = h.shape
        y = torch.empty((T, D), dtype=self.dtype, device=h.device)
        self.check(self.L.qsv_moe_combine(y.data_ptr(), ys.data_ptr(), inv.data_ptr(), wt.data_ptr(), T, idx.size(1), D, idx.data_ptr(),
                                          h.data_ptr(), E, self.code, self._s()), "moe_combine")
        return y

    def _moe_experts_expert_major(self, h, up, down, idx, wt, a=1, limit=0.0):
        T, D = h.shape
        E, rows, K = up.size(0), up.size(1), idx.size(1)
        ff = rows // 2 if a >= 2 else rows
        n = T * K
        expert, order = torch.sort(idx.reshape(-1).long(), stable=True)   # order: sorted slot -> slot (t K + k)
        # first sorted slot of every expert (and the end): a search in the sorted list - no count has to reach the host.  Slots of
        # identity experts (indices from E on) sort behind the last offset and are left to the combine.
        offsets = torch.searchsorted(expert, torch.arange(E + 1, device=h.device))
        inv = torch.empty_like(order)
        inv[order] = torch.arange(n, device=h.device)                  # slot -> sorted slot
        act = torch.empty((n, ff), dtype=self.dtype, device=h.device)
        ys = torch.empty((n, D), dtype=self.dtype, device=h.device)
        self.check(self.L.qsv_expert_rows(act.data_ptr(), h.data_ptr(), order.data_ptr(), K, up.data_ptr(), offsets.data_ptr(),
                                          E, rows, D, a, float(limit), self._s()), "expert_rows(up)")
        self.check(self.L.qsv_expert_rows(ys.data_ptr(), act.data_ptr(), 0, 1, down.data_ptr(), offsets.data_ptr(), E, D, ff, 0, 0.0,
                                          self._s()), "expert_rows(down)")
        return self._combine(h, ys, inv, idx, wt, E)

    def _moe_experts_sorted(self, h, up, down, idx, wt, code=1, limit=0.0):
        """code >= 2 (gated units): the grouped kernel folds the two halves of a unit in its epilogue; with vendor products the
        first product leaves both halves ([n, 2 ff]) and `glu` folds them."""
        T, D = h.shape
        E, rows, K = up.size(0), up.size(1), idx.size(1)
        ff = rows // 2 if code >= 2 else rows
        n = T * K
        flat = idx.reshape(-1)
        order = torch.argsort(flat, stable=True)                       # sorted slot -> slot (t K + k)
        counts = torch.bincount(flat, minlength=E).tolist()[:E]        # (host synchronisation: the runs' lengths; identity experts sort last)
        inv = torch.empty_like(order)
        inv[order] = torch.arange(n, device=h.device)                  # slot -> sorted slot
        ks, ts = self.L.qsv_grouped_gemm_k_step(), self.L.qsv_grouped_gemm_tile_slots()
        if self.moe_grouped_kernel and self.code == BF16 and D % ks == 0 and ff % ks == 0:
            # own grouped matrix-core kernel: gather in its loads, the activation in the first product's epilogue
            tiles, a = [], 0
            for e, c in enumerate(counts):
                tiles += [(e, a + o, min(ts, c - o)) for o in range(0, c, ts)]
                a += c
            act = torch.empty((n, ff), dtype=self.dtype, device=h.device)
            ys = torch.empty((n, D), dtype=self.dtype, device=h.device)
            for lo in range(0, len(tiles), 65535):
                tl = torch.tensor(tiles[lo:lo + 65535], dtype=torch.int32).to(h.device)
                self.check(self.L.qsv_grouped_gemm(act.data_ptr(), h.data_ptr(), order.data_ptr(), K, up.data_ptr(), tl.data_ptr(),
                                                   tl.size(0), rows, D, code, float(limit), self._s()), "grouped_gemm(up)")
                self.check(self.L.qsv_grouped_gemm(ys.data_ptr(), act.data_ptr(), 0, 1, down.data_ptr(), tl.data_ptr(),
                                                   tl.size(0), D, ff, 0, 0.0, self._s()), "grouped_gemm(down)")
            return self._combine(h, ys, inv, idx, wt, E)
        xs = torch.empty((n, D), dtype=self.dtype, device=h.device)
        self.check(self.L.qsv_gather_rows(xs.data_ptr(), h.data_ptr(), order.data_ptr(), K, n, D, self.code, self._s()),
                   "gather_rows")
        act = torch.empty((n, rows), dtype=self.dtype, device=h.device)
        ys = torch.empty((n, D), dtype=self.dtype, device=h.device)
        at = 0
        for e, c in enumerate(counts):
            if c:
                torch.matmul(xs[at:at + c], up[e].t(), out=act[at:at + c])
            at += c
        if code >= 2:
            act = self.glu(act, "silu" if code == 2 else "clamped", limit)
        else:
            self.check(self.L.qsv_relu_sq(act.data_ptr(), act.numel(), self.code, self._s()), "relu_sq")
        at = 0
        for e, c in enumerate(counts):
            if c:
                torch.matmul(act[at:at + c], down[e].t(), out=ys[at:at + c])
            at += c
        return self._combine(h, ys, inv, idx, wt, E)


def _rotate(v, rope, pos, rot_n):
    """Interleaved-pair rotation of the first rot_n columns of v [..., n] (float); rope [P, 2, rot_n / 2]."""
    if not rot_n:
        return v
    cs = rope[pos.long()]                       # [T, 2, half]
    c, s = cs[:, 0], cs[:, 1]
    while c.dim() < v.dim():
        c, s = c.unsqueeze(1), s.unsqueeze(1)
    a, b = v[..., 0:rot_n:2], v[..., 1:rot_n:2]
    out = v.clone()
    out[..., 0:rot_n:2] = a * c - b * s
    out[..., 1:rot_n:2] = b * c + a * s
    return out


class TorchOps:
    """Unfused tensor-op form of HipOps (see the module docstring).  Same storage roundings at the same places."""
    name = "unfused"

    def __init__(self, dtype):
        self.dtype = dtype
        dtype_code(dtype)

    def embed(self, tokens, table):
        h = table[tokens.long()]
        return h.float(), h.to(self.dtype)

    @staticmethod
    def _ln(y, w, eps):
        y = y.float()
        mu = y.mean(-1, keepdim=True)
        var = ((y - mu) ** 2).mean(-1, keepdim=True)
        return (y - mu) / torch.sqrt(var + eps) * w.float()

    def add_layer_norm(self, x, y, w, eps):
        x += self._ln(y, w, eps)
        return x.to(self.dtype)

    def layer_norm_rows(self, x, rows, w, eps):
        return self._ln(x if rows is None else x[rows.long()], w, eps).to(self.dtype)

    @staticmethod
    def _rms(v, w, eps):
        v = v.float()
        return v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps) * w.float()

    def latent_prep(self, down, q_off, q_rank, q_w, kv_off, kv_rank, kv_w, rot_dim, rot_n, rope, pool, slot, pos, eps):
        cq = self._rms(down[:, q_off:q_off + q_rank], q_w, eps).to(self.dtype)
        c = self._rms(down[:, kv_off:kv_off + kv_rank], kv_w, eps)
        kr = _rotate(down[:, kv_off + kv_rank:kv_off + kv_rank + rot_dim].float(), rope, pos, rot_n)
        pool[slot] = torch.cat([c, kr], dim=-1).to(self.dtype)
        return cq

    def latent_query(self, q, q_abs, rope, pos, scale, heads, dim, rot_dim, rot_n, rank):
        T = q.size(0)
        qr = _rotate(q.view(T, heads, dim + rot_dim)[..., dim:].float(), rope, pos, rot_n)
        return (torch.cat([q_abs.transpose(0, 1).float(), qr], dim=-1) * scale).contiguous()

    def latent_attention(self, qf, pool, batch, window, rank, page, variant=0, key_splits=None, q_first=0, chunk=None, bias=None,
                         keep_first=0, sink=None, pooled=None, pool_block=0):
        T, H, R = qf.shape
        block_table, seq, pos = batch.block_table, batch.seq, batch.pos
        out = torch.empty((T, H, rank), dtype=self.dtype, device=qf.device)
        bt = block_table.long()
        pools = [pool] if pool.dim() == 2 else list(pool)
        extra = None if pooled is None else ([pooled] if pooled.dim() == 2 else list(pooled))
        per = H // len(pools)
        per_page = (page + pool_block - 1) // pool_block if pooled is not None else 0
        for t in range(T):
            p = int(pos[t])
            lo = max(0, p - window + 1) if window else 0
            if chunk:
                lo = max(lo, p - p % chunk)
            j = torch.arange(lo, p + 1, device=qf.device)
            if keep_first:
                j = torch.cat([torch.arange(0, min(int(keep_first), lo), device=qf.device), j])
            at = bt[int(seq[t]), j // page] * page + j % page
            for g, pl in enumerate(pools):
                hs = slice(g * per, (g + 1) * per)
                rows = pl[at].float()                                                # [n, R]
                s = qf[t, hs] @ rows.t()                                             # [per, n]
                if bias is not None:
                    s = s + bias[hs][:, (p - j).clamp(max=bias.size(1) - 1)]
                if extra is not None:                                                # blocks wholly before the window
                    first = torch.arange(max(0, p - window + 1) // pool_block, device=qf.device) * pool_block
                    more = extra[g][bt[int(seq[t]), first // page] * per_page + (first % page) // pool_block].float()
                    s, rows = torch.cat([qf[t, hs] @ more.t(), s], dim=-1), torch.cat([more, rows])
                if sink is not None:
                    pr = torch.softmax(torch.cat([s, sink[hs, None]], dim=-1), dim=-1)[:, :-1]
                else:
                    pr = torch.softmax(s, dim=-1)
                out[t, hs] = (pr @ rows[:, :rank]).to(self.dtype)
        return out

    def sigmoid_gate(self, o, g):
        o.copy_((o.float() * torch.sigmoid(g.float())).to(self.dtype))
        return o

    # ---- streams, position-free norm, token shift -----------------------------------------------------------------------------
    def embed_streams(self, tokens, table, scale, streams):
        x = table[tokens.long()].float() * scale
        return x[:, None, :].repeat(1, streams, 1).contiguous()

    def hc_read(self, x, w_in, norm, shift=None, batch=None, prev=None):
        w, b, alpha = norm
        n = torch.tanh(alpha * torch.einsum("s,tsd->td", w_in, x)) * w.float() + b.float()
        if shift is None:
            return n.to(self.dtype)
        before = torch.zeros_like(n)
        before[1:] = n[:-1]
        for slot, first, cnt in batch.items:
            rd, wr = int(batch.state_rd[first]), int(batch.state_wr[first + cnt - 1])
            before[first] = prev[rd] if rd >= 0 else 0.0
            prev[wr] = n[first + cnt - 1]
        return (n + (before - n) * shift.float()).to(self.dtype)

    def hc_write(self, x, y, w_mix, w_out, then_read=None):
        x.copy_(torch.einsum("sr,tsd->trd", w_mix, x) + w_out[None, :, None] * y.float()[:, None, :])
        return None if then_read is None else self.hc_read(x, then_read[0], then_read[1])

    def dyt_sum_rows(self, x, rows, norm):
        w, b, alpha = norm
        u = (x if rows is None else x[rows.long()]).sum(1)
        return (torch.tanh(alpha * u) * w.float() + b.float()).to(self.dtype)

    # ---- rotations in the halves layout (pair i = dimensions i, i + n / 2) ------------------------------------------------------
    @staticmethod
    def _rotate_halves(v, rope, pos, n, sign=1.0):
        cs = rope[pos.long()]
        c, s = cs[:, 0, None, :], cs[:, 1, None, :] * sign
        a, b = v[..., :n // 2], v[..., n // 2:n]
        return torch.cat([a * c - b * s, b * c + a * s, v[..., n:]], dim=-1)

    def attention_prep(self, proj, q_off, k_off, v_off, heads, kv_heads, dim, vdim, rot_n, rope_k, rope_v, scale, pool, batch):
        T = proj.size(0)
        q = proj[:, q_off:q_off + heads * dim].float().view(T, heads, dim)
        k = proj[:, k_off:k_off + kv_heads * dim].float().view(T, kv_heads, dim)
        v = proj[:, v_off:v_off + kv_heads * vdim].float().view(T, kv_heads, vdim)
        q = self._rotate_halves(q, rope_k, batch.pos, rot_n) * scale
        k = self._rotate_halves(k, rope_k, batch.pos, rot_n)
        v = self._rotate_halves(v, rope_v, batch.pos, vdim)
        pool[:, batch.slot] = torch.cat([v, k], dim=-1).transpose(0, 1).to(self.dtype)
        return torch.cat([torch.zeros(T, heads, vdim, device=proj.device), q], dim=-1).contiguous()

    def rotate_heads(self, o, rope, pos, sign):
        o.copy_(self._rotate_halves(o.float(), rope, pos, o.size(-1), sign).to(self.dtype))
        return o


    # ---- sandwich norms, sink / kept-first / pooled-block attention, element-wise gated recurrence -----------------------------------
    def add_normed_rms_norm(self, x, y, w_post, w_next, eps):
        if y is not None:
            x += self._rms(y, w_post, eps)
        return None if w_next is None else self._rms(x, w_next, eps).to(self.dtype)

    def relu_sq(self, a):
        a.copy_((torch.relu(a.float()) ** 2).to(a.dtype))
        return a

    def qk_norm_rope_prep(self, q, k, v, heads, kv_heads, dim, vdim, q_w, k_w, per_head, eps, rope, rot_n, scale, pool, batch):
        T = q.size(0)

        def prep(u, w, n):
            u = self._rms(u.reshape(T, n, dim), w, eps) if per_head else self._rms(u, w, eps).view(T, n, dim)
            return u if rope is None else _rotate(u, rope, batch.pos, rot_n)

        if k is not None:
            rows = torch.cat([v.float().reshape(T, kv_heads, vdim), prep(k, k_w, kv_heads)], dim=-1)
            pool[:, batch.slot] = rows.transpose(0, 1).to(self.dtype)
        return torch.cat([torch.zeros(T, heads, vdim, device=q.device), prep(q, q_w, heads) * scale], dim=-1).contiguous()

    def pool_blocks(self, pool, pooled, batch, block, page):
        per_page = (page + block - 1) // block
        bt = batch.block_table.long()
        for t in range(batch.n_tokens):
            p, s = int(batch.pos[t]), int(batch.seq[t])
            if (p + 1) % block:
                continue
            j = torch.arange(p + 1 - block, p + 1, device=pool.device)
            first = p + 1 - block
            dst = bt[s, first // page] * per_page + (first % page) // block
            pooled[:, dst] = (pool[:, bt[s, j // page] * page + j % page].float().sum(1) / block).to(self.dtype)

    def min_gru_scan(self, proj, z_off, x_off, g_off, b_z, b_x, state, batch, width):
        z = torch.sigmoid(proj[:, z_off:z_off + width].float() + b_z.float())
        u = proj[:, x_off:x_off + width].float() + b_x.float()
        c = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
        g = proj[:, g_off:g_off + width].float()
        out = torch.empty_like(z)
        for slot, first, cnt in batch.items:
            S = state[slot].clone() if int(batch.pos[first]) else torch.zeros_like(state[slot])
            for t in range(first, first + cnt):
                S = (1.0 - z[t]) * S + z[t] * c[t]
                out[t] = S
            state[slot] = S
        return (out * g * torch.sigmoid(g)).to(self.dtype)

    # ---- recurrences ----------------------------------------------------------------------------------------------------------
    def decay(self, z, bias, a_log, tau, heads, dim):
        z = z.float() + bias.float()
        if a_log is None:
            return torch.exp(-torch.nn.functional.softplus(-z) / tau).contiguous()          # sigmoid(z) ^ (1 / tau)
        rate = torch.exp(a_log.float()).repeat_interleave(dim)
        return torch.exp(-rate * torch.nn.functional.softplus(z)).contiguous()

    def conv_silu_unit(self, proj, off, conv_w, hist, batch, n_unit, unit_dim, act="silu"):
        C, taps = conv_w.shape
        xin = proj[:, off:off + C].to(self.dtype).float()
        out = torch.empty_like(xin)
        w = conv_w.float()
        for slot, first, cnt in batch.items:
            rd, wr = int(batch.state_rd[first]), int(batch.state_wr[first + cnt - 1])
            past = hist[rd][:taps - 1] if rd >= 0 else torch.zeros((taps - 1, C), device=xin.device)
            seq = torch.cat([past, xin[first:first + cnt]])
            y = sum(seq[j:j + cnt] * w[:, j] for j in range(taps))
            out[first:first + cnt] = y * torch.sigmoid(y) if act == "silu" else y
            if taps > 1:
                hist[wr] = seq[cnt:]
        if not n_unit:
            return out
        u = out[:, :n_unit * unit_dim].view(-1, n_unit, unit_dim)
        out[:, :n_unit * unit_dim] = (u / torch.sqrt((u * u).sum(-1, keepdim=True) + 1e-6)).view(-1, n_unit * unit_dim)
        return out

    def recurrent_scan(self, q, k, v, decay, beta, state, batch, heads, qk_heads, dim, vdim, q_scale, kscale=None, v_cols=None):
        T = q.size(0)
        rep = heads // qk_heads
        qf = q.float().reshape(T, qk_heads, dim).repeat_interleave(rep, 1) * q_scale
        kf = k.float().reshape(T, qk_heads, dim).repeat_interleave(rep, 1)
        if kscale is not None:
            kf = kf * kscale[:, :, None]
        vf = v.float().reshape(T, heads, v_cols or vdim)
        if v_cols and v_cols < vdim:
            ones = torch.zeros((T, heads, vdim - v_cols), device=q.device)
            ones[..., 0] = 1.0
            vf = torch.cat([vf, ones], dim=-1)
        g = decay[:, :, None].expand(T, heads, dim) if decay.shape == (T, heads) and dim != 1 else decay.view(T, heads, dim)
        bt = None if beta is None else torch.sigmoid(beta.float())
        o = torch.empty((T, heads, vdim), dtype=torch.float32, device=q.device)
        for slot, first, cnt in batch.items:
            S = state[slot].clone() if int(batch.pos[first]) else torch.zeros_like(state[slot])
            for t in range(first, first + cnt):
                S = g[t][:, :, None] * S
                if bt is None:
                    S = S + kf[t][:, :, None] * vf[t][:, None, :]
                else:
                    u = bt[t][:, None] * (vf[t] - torch.einsum("hdv,hd->hv", S, kf[t]))
                    S = S + kf[t][:, :, None] * u[:, None, :]
                o[t] = torch.einsum("hdv,hd->hv", S, qf[t])
            state[slot] = S
        return o

    def head_rms_gate(self, o, w, gate, kind, eps, vdim=None, den_m=None):
        T, H, n_cols = o.shape
        dv = n_cols if vdim is None else vdim
        if den_m is not None:
            o = o[..., :dv] / (torch.maximum(o[..., dv].abs(), torch.exp(-den_m)) + 1e-6)[..., None]
        o = o[..., :dv]
        w = w.float().view(H, dv) if w.numel() == H * dv else w.float()
        n = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps) * w
        g = gate.float().reshape(T, H, dv)
        g = g * torch.sigmoid(g) if kind == "silu" else torch.sigmoid(g)
        return (n * g).reshape(T, H * dv).to(self.dtype)

    def rms_pair_mean(self, a, wa, b, wb, eps):
        return (0.5 * (self._rms(a, wa, eps) + self._rms(b, wb, eps))).to(self.dtype)

    def glu(self, a, act="silu", limit=0.0):
        a = a.float()
        g, u = a[..., 0::2], a[..., 1::2]
        if act == "clamped":
            g, u = g.clamp(max=limit), u.clamp(-limit, limit)
            return (g * torch.sigmoid(1.702 * g) * (u + 1.0)).to(self.dtype)
        ag = g * torch.sigmoid(g) if act == "silu" else torch.nn.functional.gelu(g, approximate="tanh")
        return (ag * u).to(self.dtype)

    def moe_route(self, h, router, top_k, groups, keep, bias=None, renorm=False, score="softmax", correction=None, group_top=1,
                  scale=1.0):
        z = h.float() @ router.float().t()
        if bias is not None:
            z = z + bias.float()
        if renorm and score == "softmax" and correction is None and groups == 1:   # weights = softmax over the chosen logits only
            top = z.topk(top_k, dim=-1)
            return top.indices.int(), torch.softmax(top.values, dim=-1) * scale
        s = torch.softmax(z, dim=-1) if score == "softmax" else torch.sigmoid(z)
        c = s if correction is None else s + correction.float()
        T, E = s.shape
        per = E // groups
        gs = c.view(T, groups, per).topk(min(group_top, per), dim=-1).values.sum(-1)
        kept = torch.zeros_like(gs, dtype=torch.bool).scatter_(1, gs.topk(keep, dim=-1).indices, True)
        ok = kept[:, :, None].expand(T, groups, per).reshape(T, E)
        idx = c.masked_fill(~ok, float("-inf")).topk(top_k, dim=-1).indices
        wt = s.gather(1, idx)
        if renorm:
            wt = wt / wt.sum(-1, keepdim=True)
        return idx.int(), wt * scale

    # ---- sinusoidal positions, RMS-normed residual, whole-projection query / key norms ----------------------------------------------
    def embed_sinusoid(self, tokens, pos, table, freq, scale):
        a = pos.float()[:, None] * freq[None, :]                                    # float angles
        sc = torch.stack([torch.sin(a), torch.cos(a)], dim=-1).reshape(a.size(0), -1)[:, :table.size(1)]
        return table[tokens.long()].float() * scale + sc

    def add_rms_norm(self, x, ys, w, eps):
        ys = [y.float() for y in ys if y is not None]
        if ys:
            y = ys[0]
            if len(ys) > 1:
                y = y + (ys[1] + ys[2] if len(ys) > 2 else ys[1])
            x += y
        return None if w is None else self._rms(x, w, eps).to(self.dtype)

    def rms_norm_rows(self, x, rows, w, eps):
        return self._rms(x if rows is None else x[rows.long()], w, eps).to(self.dtype)

    def normed_attention_prep(self, proj, q_off, k_off, v_off, heads, kv_heads, dim, vdim, q_w, k_w, eps, scale, v_first, mix, pool,
                              batch):
        T = proj.size(0)
        q = self._rms(proj[:, q_off:q_off + heads * dim], q_w, eps).view(T, heads, dim) * scale
        k = self._rms(proj[:, k_off:k_off + kv_heads * dim], k_w, eps).view(T, kv_heads, dim)
        v = proj[:, v_off:v_off + kv_heads * vdim].float()
        if v_first is not None:
            v = (1.0 - mix) * v + mix * v_first.float()
        pool[:, batch.slot] = torch.cat([v.view(T, kv_heads, vdim), k], dim=-1).transpose(0, 1).to(self.dtype)
        return torch.cat([torch.zeros(T, heads, vdim, device=proj.device), q], dim=-1).contiguous()

    def max_gates(self, proj, i_off, f_off, bias_i, bias_f, cap, m_state, batch, heads):
        li = cap * torch.tanh((proj[:, i_off:i_off + heads].float() + bias_i) / cap)
        lf = torch.nn.functional.logsigmoid(cap * torch.tanh((proj[:, f_off:f_off + heads].float() + bias_f) / cap))
        a, b, m = torch.empty_like(li), torch.empty_like(li), torch.empty_like(li)
        for slot, first, cnt in batch.items:
            prev = m_state[slot].clone() if int(batch.pos[first]) else torch.zeros_like(m_state[slot])
            for t in range(first, first + cnt):
                m[t] = torch.maximum(lf[t] + prev, li[t])
                a[t], b[t] = torch.exp(lf[t] + (prev - m[t])), torch.exp(li[t] - m[t])
                prev = m[t]
            m_state[slot] = prev
        return a, b, m

    def moe_experts(self, h, up, down, idx, wt, act="relu_sq", limit=0.0):
        T, D = h.shape
        E = up.size(0)
        y = torch.zeros((T, D), dtype=torch.float32, device=h.device)
        for k in range(idx.size(1)):
            e = idx[:, k].long()
            real = e < E
            e = e.clamp(max=E - 1)
            a = torch.einsum("tfd,td->tf", up[e].float(), h.float())
            if act == "relu_sq":
                a = torch.relu(a) ** 2
            else:
                a = self.glu(a.to(self.dtype), "silu" if act == "swiglu" else "clamped", limit).float()
            a = a.to(self.dtype).float()
            o = torch.einsum("tdf,tf->td", down[e].float(), a)
            y += wt[:, k, None] * torch.where(real[:, None], o, h.float())
        return y.to(self.dtype)


def make_ops(backend, dtype, device):
    """backend: "hip" (the only one a served model uses) or "unfused" (bring-up and host-logic tests)."""
    if backend == "hip":
        if torch.device(device).type != "cuda":
            raise RuntimeError("the hip backend needs a GPU device; there is no CPU path for served models")
        return HipOps(dtype)
    if backend == "unfused":
        return TorchOps(dtype)
    raise ValueError(f"unknown backend {backend!r}")
