// serve_recurrent.hip -- matrix-state recurrences (gated linear attention, gated delta rule) and what feeds them: decays,
// the short causal convolution with its history state, unit norms, the per-head output norm with its gate; and the rotations of
// the attention that runs beside them (queries, keys and values in the halves layout, cache rows written in the same pass).
// Everything that enters a recurrence is float; the state is float in memory and in registers.
#include "serve_common.h"

namespace {
constexpr int NT = 256;
constexpr int NW = NT / 64;

__device__ __forceinline__ float softplusf(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// ---- decays ---------------------------------------------------------------------------------------------------------------
// mode 0: sigmoid(z + bias)^(1 / tau) = exp(-softplus(-(z + bias)) / tau);  mode 1: exp(-exp(a_log[head]) softplus(z + bias))
template <typename T>
__global__ __launch_bounds__(NT) void decay_kernel(float* __restrict__ out, const T* __restrict__ z, int64_t z_stride,
                                                   const T* __restrict__ bias, const float* __restrict__ a_log, float inv_tau,
                                                   int dim, int n) {
    const size_t t = blockIdx.x;
    for (int c = threadIdx.x; c < n; c += NT) {
        const float v = ld(z, t * z_stride + c) + ld(bias, c);
        out[t * n + c] = a_log ? expf(-expf(a_log[c / dim]) * softplusf(v)) : expf(-softplusf(-v) * inv_tau);
    }
}

// ---- causal convolution over time + silu (act 0: no activation), unit norm of the leading groups -----------------------------------------------------
// Workgroup = token.  Tap j (last column = the current token) reads the input taps - 1 - j tokens back: a row of this batch
// inside the run, the sequence's history state before the run's start, zero before the sequence's start.  The last token of a
// run writes the new history (the last taps - 1 inputs) into the state's other copy.  Dynamic LDS: C floats.
template <typename T>
__global__ __launch_bounds__(NT) void conv_silu_unit_kernel(float* __restrict__ out, const T* __restrict__ proj, int64_t stride,
                                                            int off, int C, int taps, const float* __restrict__ w,
                                                            float* __restrict__ hist, const int32_t* __restrict__ run_off,
                                                            const int32_t* __restrict__ state_rd,
                                                            const int32_t* __restrict__ state_wr, int n_unit, int unit_dim, int act) {
    extern __shared__ float ys[];
    const size_t t = blockIdx.x;
    const int i = run_off[t], rd = state_rd[t], wr = state_wr[t];
    const int past = taps - 1;
    for (int c = threadIdx.x; c < C; c += NT) {
        float acc = 0.f;
        for (int j = 0; j < taps; ++j) {
            const int d = past - j;
            float xv = 0.f;
            if (d <= i) xv = ld(proj, (t - d) * stride + off + c);
            else if (rd >= 0) xv = hist[((size_t)rd * past + (past + i - d)) * C + c];
            acc += w[(size_t)c * taps + j] * xv;
        }
        ys[c] = act ? acc / (1.0f + expf(-acc)) : acc;
        if (wr >= 0) {
            for (int jj = 0; jj < past; ++jj) {
                const int e = i + 1 - past + jj;            // index within the run of the input that becomes history entry jj
                float xv = 0.f;
                if (e >= 0) xv = ld(proj, (t - (i - e)) * stride + off + c);
                else if (rd >= 0) xv = hist[((size_t)rd * past + (jj + i + 1)) * C + c];
                hist[((size_t)wr * past + jj) * C + c] = xv;
            }
        }
    }
    __syncthreads();
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    for (int g = wv; g < n_unit; g += NW) {
        float s = 0.f;
        for (int e = lane; e < unit_dim; e += 64) s += ys[g * unit_dim + e] * ys[g * unit_dim + e];
        const float inv = 1.0f / sqrtf(wave_sum(s) + 1e-6f);
        for (int e = lane; e < unit_dim; e += 64) out[t * C + g * unit_dim + e] = ys[g * unit_dim + e] * inv;
    }
    for (int c = n_unit * unit_dim + threadIdx.x; c < C; c += NT) out[t * C + c] = ys[c];
}

// ---- the recurrence ---------------------------------------------------------------------------------------------------------
// Columns of S (value channels) never meet: column j of head h needs k, q and the decay of the token and its own v_j.  A
// workgroup owns a block of columns of one (run, head): a wave 64 / LPC groups of NC of them, a lane R rows of its NC columns;
// the LPC lanes of a column are neighbours and add their partial dot products through DPP moves.  The run's tokens are walked in order, CT at
// a time: the workgroup stages k, q, the decay (float, zero-padded to LPC * R rows), its v columns and sigmoid(beta) of CT
// tokens in LDS - the next CT tokens' values are already in registers while these are computed - so a token's step reads
// LDS only, and the only exchange on the state's dependency chain is the delta rule's S^T k; the read-outs' partial sums wait
// in registers until the chunk's end and are exchanged together.  The state is read once before and written once after (a run
// that starts its sequence starts from zeros).
constexpr int SCAN_CT = 16;       // tokens per staged chunk, at most
constexpr int SCAN_PFK = 24;      // staged k / q / decay values per thread and chunk, at most
constexpr int SCAN_PFV = 16;      // staged v values per thread and chunk, at most

template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
    return v + __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
// sum over the lpc neighbouring lanes of a column (lpc a power of two); every one of them gets it
__device__ __forceinline__ float column_sum(float v, int lpc) {
    if (lpc >= 2) v = dpp_add<0xB1>(v);          // quad_perm [1, 0, 3, 2]
    if (lpc >= 4) v = dpp_add<0x4E>(v);          // quad_perm [2, 3, 0, 1]
    if (lpc >= 8) v = dpp_add<0x141>(v);         // row_half_mirror: the other quad of eight lanes
    if (lpc >= 16) v = dpp_add<0x140>(v);        // row_mirror: the other half of sixteen lanes
    if (lpc >= 32) v += __shfl_xor(v, 16, 64);
    if (lpc >= 64) v += __shfl_xor(v, 32, 64);
    return v;
}

__device__ __forceinline__ float4 ld4(const float* p, size_t i) { return *(const float4*)(p + i); }
__device__ __forceinline__ float4 ld4(const bf16_t* p, size_t i) {
    const uint2 u = *(const uint2*)(p + i);
    return make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u), __uint_as_float(u.y << 16),
                       __uint_as_float(u.y & 0xffff0000u));
}

// VEC: dim, vdim, the row strides and the operands' addresses are multiples of four elements - staged four at a time.
// R rows and NC columns of the state per lane (with NC > 1 the token's k, q and decay rows are read from LDS once for NC columns).
// OCC: waves per SIMD the register allocation must leave room for (1: no demand - the compiler takes about 230 registers, two waves).
template <typename TQ, typename TB, bool DELTA, bool VEC, int R, int NC, int OCC>
__global__ __launch_bounds__(256, OCC) void recurrent_scan_kernel(float* __restrict__ o, const TQ* __restrict__ q, int64_t q_stride,
                                                             const TQ* __restrict__ k, int64_t k_stride, const TQ* __restrict__ v,
                                                             int64_t v_stride, const float* __restrict__ decay,
                                                             const TB* __restrict__ beta, int64_t beta_stride,
                                                             float* __restrict__ state, const int32_t* __restrict__ runs, int H,
                                                             int QH, int dim, int vdim, int lpc_log, int CT, float q_scale,
                                                             const float* __restrict__ kscale, int head_decay, int v_cols) {
    static_assert(R == 4 || R == 8 || R == 16, "rows per lane");
    // (the three-wave variant stages half as many tokens per chunk: fewer prefetch registers and deferred read-outs, no spills)
    constexpr int MAX_CT = OCC >= 3 ? SCAN_CT / 2 : SCAN_CT, PFK = OCC >= 3 ? SCAN_PFK / 2 : SCAN_PFK, PFV = OCC >= 3 ? SCAN_PFV / 2 : SCAN_PFV;
    extern __shared__ __attribute__((aligned(16))) float sm[];
    const int tid = threadIdx.x, nthr = blockDim.x, lane = tid & 63, wave = tid >> 6, nw = nthr >> 6;
    const int lpc = 1 << lpc_log, cols = 64 >> lpc_log;                           // cols: column groups (of NC) per wave
    const int dimp_log = lpc_log + (R == 16 ? 4 : R == 8 ? 3 : 2), DIMP = 1 << dimp_log, VB = nw * cols * NC;   // (all powers of two)
    const int vb_log = 31 - __clz(VB);
    const int row_len = 3 * DIMP + ((VB + 4) & ~3);              // floats of one staged token: k | q | decay | v | beta, 16-byte rows
    const int part = lane & (lpc - 1), cb = (wave * cols + (lane >> lpc_log)) * NC;
    const int j = blockIdx.z * VB + cb;                          // first of this lane's NC columns
    const int r0 = part * R;
    const int slot = runs[4 * blockIdx.x], first = runs[4 * blockIdx.x + 1], n = runs[4 * blockIdx.x + 2];
    const bool fresh = runs[4 * blockIdx.x + 3] == 0;
    const int h = blockIdx.y, qh = h / (H / QH);
    float* Sg = state + (((size_t)slot * H + h) * dim) * (size_t)vdim;
    float S[NC][R];
#pragma unroll
    for (int c = 0; c < NC; ++c)
#pragma unroll
        for (int i = 0; i < R; ++i) S[c][i] = (!fresh && j + c < vdim && r0 + i < dim) ? Sg[(size_t)(r0 + i) * vdim + j + c] : 0.f;

    float pk[PFK], pv[PFV], pb = 0.f;
    // requests the operands of tokens [c0, c0 + ct) of the run into registers
    auto fetch = [&](int c0, int ct) {
        const int nk = ct * 3 * DIMP, nv = ct * VB;
        if (VEC) {
#pragma unroll
            for (int i = 0; i < PFK / 4; ++i) {
                const int idx = (tid + i * nthr) * 4;
                float4 val = make_float4(0.f, 0.f, 0.f, 0.f);
                if (idx < nk) {
                    const int seg = idx >> dimp_log, r = idx & (DIMP - 1), tt = seg / 3, which = seg - 3 * tt;
                    const size_t t = (size_t)(first + c0 + tt);
                    if (r < dim) {
                        if (which == 2 && head_decay) {
                            const float g = decay[t * H + h];
                            val = make_float4(g, g, g, g);
                        } else {
                            val = which == 0 ? ld4(k, t * k_stride + (size_t)qh * dim + r)
                                : which == 1 ? ld4(q, t * q_stride + (size_t)qh * dim + r)
                                             : ld4(decay, (t * H + h) * (size_t)dim + r);
                            if (which == 0 && kscale) {
                                const float b = kscale[t * H + h];
                                val.x *= b; val.y *= b; val.z *= b; val.w *= b;
                            }
                        }
                    }
                }
                pk[4 * i] = val.x; pk[4 * i + 1] = val.y; pk[4 * i + 2] = val.z; pk[4 * i + 3] = val.w;
            }
#pragma unroll
            for (int i = 0; i < PFV / 4; ++i) {
                const int idx = (tid + i * nthr) * 4;
                float4 val = make_float4(0.f, 0.f, 0.f, 0.f);
                if (idx < nv) {
                    const int tt = idx >> vb_log, c = idx & (VB - 1), jj = blockIdx.z * VB + c;
                    if (jj < v_cols) val = ld4(v, (size_t)(first + c0 + tt) * v_stride + (size_t)h * v_cols + jj);
                    else if (jj == v_cols && jj < vdim) val.x = 1.0f;        // the state's column of ones (a state wider than v)
                }
                pv[4 * i] = val.x; pv[4 * i + 1] = val.y; pv[4 * i + 2] = val.z; pv[4 * i + 3] = val.w;
            }
        } else {
#pragma unroll
            for (int i = 0; i < PFK; ++i) {
                const int idx = tid + i * nthr;
                float val = 0.f;
                if (idx < nk) {
                    const int seg = idx >> dimp_log, r = idx & (DIMP - 1), tt = seg / 3, which = seg - 3 * tt;
                    const size_t t = (size_t)(first + c0 + tt);
                    if (r < dim)
                        val = which == 0 ? ld(k, t * k_stride + (size_t)qh * dim + r) * (kscale ? kscale[t * H + h] : 1.0f)
                            : which == 1 ? ld(q, t * q_stride + (size_t)qh * dim + r)
                                         : (head_decay ? decay[t * H + h] : decay[(t * H + h) * (size_t)dim + r]);
                }
                pk[i] = val;
            }
#pragma unroll
            for (int i = 0; i < PFV; ++i) {
                const int idx = tid + i * nthr;
                float val = 0.f;
                if (idx < nv) {
                    const int tt = idx >> vb_log, c = idx & (VB - 1), jj = blockIdx.z * VB + c;
                    if (jj < v_cols) val = ld(v, (size_t)(first + c0 + tt) * v_stride + (size_t)h * v_cols + jj);
                    else if (jj == v_cols && jj < vdim) val = 1.0f;
                }
                pv[i] = val;
            }
        }
        if (DELTA && tid < ct) pb = ld(beta, (size_t)(first + c0 + tid) * beta_stride + h);
    };
    auto stage = [&](int ct) {
        const int nk = ct * 3 * DIMP, nv = ct * VB;
        if (VEC) {
#pragma unroll
            for (int i = 0; i < PFK / 4; ++i) {
                const int idx = (tid + i * nthr) * 4;
                if (idx < nk) {
                    const int tt = (idx >> dimp_log) / 3;
                    *(float4*)(sm + tt * row_len + (idx - tt * 3 * DIMP)) = make_float4(pk[4 * i], pk[4 * i + 1], pk[4 * i + 2], pk[4 * i + 3]);
                }
            }
#pragma unroll
            for (int i = 0; i < PFV / 4; ++i) {
                const int idx = (tid + i * nthr) * 4;
                if (idx < nv) {
                    const int tt = idx >> vb_log;
                    *(float4*)(sm + tt * row_len + 3 * DIMP + (idx & (VB - 1))) = make_float4(pv[4 * i], pv[4 * i + 1], pv[4 * i + 2], pv[4 * i + 3]);
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < PFK; ++i) {
                const int idx = tid + i * nthr;
                if (idx < nk) {
                    const int tt = (idx >> dimp_log) / 3;
                    sm[tt * row_len + (idx - tt * 3 * DIMP)] = pk[i];
                }
            }
#pragma unroll
            for (int i = 0; i < PFV; ++i) {
                const int idx = tid + i * nthr;
                if (idx < nv) {
                    const int tt = idx >> vb_log;
                    sm[tt * row_len + 3 * DIMP + (idx & (VB - 1))] = pv[i];
                }
            }
        }
        if (DELTA && tid < ct) sm[tid * row_len + 3 * DIMP + VB] = 1.0f / (1.0f + expf(-pb));
    };

    fetch(0, min(CT, n));
    for (int c0 = 0; c0 < n; c0 += CT) {
        const int ct = min(CT, n - c0);
        __syncthreads();                                         // the previous chunk has been read by every wave
        stage(ct);
        __syncthreads();
        if (c0 + CT < n) fetch(c0 + CT, min(CT, n - c0 - CT));   // in flight while this chunk is computed
        float oacc[MAX_CT][NC];
#pragma unroll
        for (int tt = 0; tt < MAX_CT; ++tt) {
#pragma unroll
            for (int c = 0; c < NC; ++c) oacc[tt][c] = 0.f;
            if (tt >= ct) continue;                              // (uniform)
            const float* row = sm + tt * row_len;
            float kc[R], qc[R], gc[R], vc[NC];
#pragma unroll
            for (int i = 0; i < R; i += 4) {
                const float4 a = *(const float4*)(row + r0 + i), b = *(const float4*)(row + DIMP + r0 + i),
                             c = *(const float4*)(row + 2 * DIMP + r0 + i);
                kc[i] = a.x; kc[i + 1] = a.y; kc[i + 2] = a.z; kc[i + 3] = a.w;
                qc[i] = b.x; qc[i + 1] = b.y; qc[i + 2] = b.z; qc[i + 3] = b.w;
                gc[i] = c.x; gc[i + 1] = c.y; gc[i + 2] = c.z; gc[i + 3] = c.w;
            }
#pragma unroll
            for (int c = 0; c < NC; ++c) vc[c] = row[3 * DIMP + cb + c];
            if (DELTA) {
                const float bt = row[3 * DIMP + VB];
                float acc[NC];
#pragma unroll
                for (int c = 0; c < NC; ++c) {
                    acc[c] = 0.f;
#pragma unroll
                    for (int i = 0; i < R; ++i) {
                        S[c][i] *= gc[i];
                        acc[c] += S[c][i] * kc[i];
                    }
                }
#pragma unroll
                for (int c = 0; c < NC; ++c) {
                    const float u = (vc[c] - column_sum(acc[c], lpc)) * bt;
                    float a2 = 0.f;
#pragma unroll
                    for (int i = 0; i < R; ++i) {
                        S[c][i] += kc[i] * u;
                        a2 += S[c][i] * qc[i];
                    }
                    oacc[tt][c] = a2;
                }
            } else {
#pragma unroll
                for (int c = 0; c < NC; ++c) {
                    float a2 = 0.f;
#pragma unroll
                    for (int i = 0; i < R; ++i) {
                        S[c][i] = gc[i] * S[c][i] + kc[i] * vc[c];
                        a2 += S[c][i] * qc[i];
                    }
                    oacc[tt][c] = a2;
                }
            }
        }
#pragma unroll
        for (int tt = 0; tt < MAX_CT; ++tt)
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                const float sum = column_sum(oacc[tt][c], lpc);
                if (tt < ct && part == 0 && j + c < vdim) o[((size_t)(first + c0 + tt) * H + h) * (size_t)vdim + j + c] = sum * q_scale;
            }
    }
#pragma unroll
    for (int c = 0; c < NC; ++c)
#pragma unroll
        for (int i = 0; i < R; ++i)
            if (j + c < vdim && r0 + i < dim) Sg[(size_t)(r0 + i) * vdim + j + c] = S[c][i];
}

// ---- one token per run (decoding): no staging, no barriers - every lane fetches its 8 rows of k, q and the decay itself, the
// state makes one round trip -----------------------------------------------------------------------------------------------------
template <typename TQ, typename TB, bool DELTA>
__global__ __launch_bounds__(256) void recurrent_step_kernel(float* __restrict__ o, const TQ* __restrict__ q, int64_t q_stride,
                                                             const TQ* __restrict__ k, int64_t k_stride, const TQ* __restrict__ v,
                                                             int64_t v_stride, const float* __restrict__ decay,
                                                             const TB* __restrict__ beta, int64_t beta_stride,
                                                             float* __restrict__ state, const int32_t* __restrict__ runs, int H,
                                                             int QH, int dim, int vdim, int lpc_log, float q_scale,
                                                             const float* __restrict__ kscale, int head_decay, int v_cols) {
    constexpr int R = 8;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int lpc = 1 << lpc_log, cols = 64 >> lpc_log;
    const int part = lane & (lpc - 1), j = (blockIdx.z * 4 + wave) * cols + (lane >> lpc_log);
    const bool col_ok = j < vdim;
    const int r0 = part * R;
    const int slot = runs[4 * blockIdx.x];
    const size_t t = (size_t)runs[4 * blockIdx.x + 1];
    const bool fresh = runs[4 * blockIdx.x + 3] == 0;
    const int h = blockIdx.y, qh = h / (H / QH);
    float* Sg = state + (((size_t)slot * H + h) * dim) * (size_t)vdim + (col_ok ? j : 0);
    float S[R], kc[R], qc[R], gc[R];
    const float kb = kscale ? kscale[t * H + h] : 1.0f;
#pragma unroll
    for (int i = 0; i < R; ++i) {
        const bool ok = r0 + i < dim;
        S[i] = (!fresh && col_ok && ok) ? Sg[(size_t)(r0 + i) * vdim] : 0.f;
        kc[i] = ok ? ld(k, t * k_stride + (size_t)qh * dim + r0 + i) * kb : 0.f;
        qc[i] = ok ? ld(q, t * q_stride + (size_t)qh * dim + r0 + i) : 0.f;
        gc[i] = ok ? (head_decay ? decay[t * H + h] : decay[(t * H + h) * (size_t)dim + r0 + i]) : 0.f;
    }
    const float vc = !col_ok ? 0.f : j < v_cols ? ld(v, t * v_stride + (size_t)h * v_cols + j) : j == v_cols ? 1.0f : 0.f;
    float acc = 0.f;
    if (DELTA) {
#pragma unroll
        for (int i = 0; i < R; ++i) {
            S[i] *= gc[i];
            acc += S[i] * kc[i];
        }
        const float u = (vc - column_sum(acc, lpc)) / (1.0f + expf(-ld(beta, t * beta_stride + h)));
        acc = 0.f;
#pragma unroll
        for (int i = 0; i < R; ++i) {
            S[i] += kc[i] * u;
            acc += S[i] * qc[i];
        }
    } else {
#pragma unroll
        for (int i = 0; i < R; ++i) {
            S[i] = gc[i] * S[i] + kc[i] * vc;
            acc += S[i] * qc[i];
        }
    }
    acc = column_sum(acc, lpc);
    if (!col_ok) return;
    if (part == 0) o[(t * H + h) * (size_t)vdim + j] = acc * q_scale;
#pragma unroll
    for (int i = 0; i < R; ++i)
        if (r0 + i < dim) Sg[(size_t)(r0 + i) * vdim] = S[i];
}

// ---- per-head RMS norm of the read-out, times a weight, times a gate ------------------------------------------------------------
// gate_kind 0: silu(g), 1: sigmoid(g).  o rows are o_stride floats apart per head (>= vdim); w_stride 0: one weight row shared by
// the heads, vdim: a row per head.  den_m != NULL: before the norm the read-out is divided by max(|o[vdim]|, exp(-den_m[t, h])) +
// 1e-6, o[vdim] being the head's extra column (the normaliser's dot product with the query).
template <typename T>
__global__ __launch_bounds__(NT) void head_rms_gate_kernel(T* __restrict__ out, const float* __restrict__ o, const T* __restrict__ w,
                                                           const T* __restrict__ gate, int64_t gate_stride, int gate_kind, float eps,
                                                           int H, int vdim, int o_stride, int w_stride,
                                                           const float* __restrict__ den_m) {
    const size_t t = blockIdx.x;
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    for (int h = wv; h < H; h += NW) {
        const float* oh = o + (t * H + h) * (size_t)o_stride;
        const float sc = den_m ? 1.0f / (fmaxf(fabsf(oh[vdim]), expf(-den_m[t * H + h])) + 1e-6f) : 1.0f;
        float s = 0.f;
        for (int e = lane; e < vdim; e += 64) s += (oh[e] * sc) * (oh[e] * sc);
        const float inv = 1.0f / sqrtf(wave_sum(s) / (float)vdim + eps);
        for (int e = lane; e < vdim; e += 64) {
            const float g = ld(gate, t * gate_stride + (size_t)h * vdim + e);
            const float sg = 1.0f / (1.0f + expf(-g));
            st(out, (t * H + h) * (size_t)vdim + e, oh[e] * sc * inv * ld(w, (size_t)h * w_stride + e) * (gate_kind == 0 ? g * sg : sg));
        }
    }
}

// ---- exponential gates kept in range by a running maximum (mLSTM) ----------------------------------------------------------------
// Per (run, head) one wave; a lane takes one token of 64 at a time.  li = cap tanh((z_i + b_i) / cap), lf = logsigmoid(cap tanh((z_f
// + b_f) / cap)); m_t = max(lf_t + m_(t-1), li_t) is a scan over the maps x -> max(x + A, B), which compose to (A1 + A2, max(B1 + A2,
// B2)); decay a_t = exp(lf_t + m_(t-1) - m_t), input scale b_t = exp(li_t - m_t).  m of a run's last token goes back to the state
// (a run that starts its sequence starts from m = 0).
__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }
template <typename T>
__global__ __launch_bounds__(64) void max_gates_kernel(float* __restrict__ a_out, float* __restrict__ b_out, float* __restrict__ m_out,
                                                       const T* __restrict__ zi, const T* __restrict__ zf, int64_t z_stride,
                                                       const float* __restrict__ bias_i, const float* __restrict__ bias_f, float cap,
                                                       float* __restrict__ m_state, const int32_t* __restrict__ runs, int H) {
    const int lane = threadIdx.x;
    const int slot = runs[4 * blockIdx.x], first = runs[4 * blockIdx.x + 1], n = runs[4 * blockIdx.x + 2];
    const int h = blockIdx.y;
    float carry = runs[4 * blockIdx.x + 3] == 0 ? 0.f : m_state[(size_t)slot * H + h];
    const float inv_cap = 1.0f / cap;
    for (int c0 = 0; c0 < n; c0 += 64) {
        const bool ok = c0 + lane < n;
        const size_t t = (size_t)first + c0 + (ok ? lane : 0);
        const float li = cap * tanhf((ld(zi, t * z_stride + h) + bias_i[h]) * inv_cap);
        const float lf = log_sigmoid(cap * tanhf((ld(zf, t * z_stride + h) + bias_f[h]) * inv_cap));
        float A = ok ? lf : 0.f, B = ok ? li : -INFINITY;       // (a lane past the end is the identity map)
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const float pA = __shfl_up(A, o, 64), pB = __shfl_up(B, o, 64);
            if (lane >= o) {
                B = fmaxf(pB + A, B);
                A = pA + A;
            }
        }
        const float m = fmaxf(carry + A, B);
        float prev = __shfl_up(m, 1, 64);
        if (lane == 0) prev = carry;
        if (ok) {
            a_out[t * H + h] = expf(lf + (prev - m));            // (prev - m is exact; lf + prev would round lf away)
            b_out[t * H + h] = expf(li - m);
            m_out[t * H + h] = m;
        }
        carry = __shfl(m, min(63, n - c0 - 1), 64);
    }
    if (lane == 0) m_state[(size_t)slot * H + h] = carry;
}

// ---- rotations, halves layout: pair p of n rotated dimensions = (p, p + n / 2); rope [positions, 2, n / 2] -------------------
__device__ __forceinline__ float rot_halves(float u_lo, float u_hi, bool upper, float c, float s) {
    return upper ? u_hi * c + u_lo * s : u_lo * c - u_hi * s;
}
template <typename T>
__device__ __forceinline__ float rotated(const T* vec, int d, int n, const float* cs) {   // element d of the rotated vector
    if (d >= n) return ld(vec, d);
    const int half = n >> 1, p = d < half ? d : d - half;
    return rot_halves(ld(vec, p), ld(vec, p + half), d >= half, cs[p], cs[half + p]);
}

// qf[t, h] = [0 (vdim) | rot(q[t, h]) * scale]; pool[g, slot[t]] = [rot_v(v[t, g]) | rot(k[t, g])]
template <typename T>
__global__ __launch_bounds__(NT) void attention_prep_kernel(float* __restrict__ qf, T* __restrict__ pool, int64_t pool_rows,
                                                            const T* __restrict__ proj, int64_t stride, int q_off, int k_off,
                                                            int v_off, int H, int G, int dim, int vdim, int rot_n,
                                                            const float* __restrict__ rope_k, const float* __restrict__ rope_v,
                                                            float scale, const int64_t* __restrict__ slot,
                                                            const int32_t* __restrict__ pos) {
    const size_t t = blockIdx.x;
    const int R = vdim + dim, p = pos[t];
    const T* row = proj + t * stride;
    const float* ck = rope_k + (size_t)p * rot_n;
    const float* cv = rope_v + (size_t)p * vdim;
    for (int idx = threadIdx.x; idx < H * R; idx += NT) {
        const int h = idx / R, c = idx - h * R;
        qf[t * H * (size_t)R + idx] = c < vdim ? 0.f : rotated(row + q_off + h * dim, c - vdim, rot_n, ck) * scale;
    }
    for (int idx = threadIdx.x; idx < G * R; idx += NT) {
        const int g = idx / R, c = idx - g * R;
        const float val = c < vdim ? rotated(row + v_off + g * vdim, c, vdim, cv) : rotated(row + k_off + g * dim, c - vdim, rot_n, ck);
        st(pool, ((size_t)g * pool_rows + (size_t)slot[t]) * R + c, val);
    }
}

// o[t, h, :n] turned by sign * pos[t] in place
template <typename T>
__global__ __launch_bounds__(NT) void rotate_heads_kernel(T* __restrict__ o, const float* __restrict__ rope,
                                                          const int32_t* __restrict__ pos, float sign, int H, int n) {
    const size_t t = blockIdx.x;
    const int half = n >> 1;
    const float* cs = rope + (size_t)pos[t] * n;
    for (int idx = threadIdx.x; idx < H * half; idx += NT) {
        const int h = idx / half, p = idx - h * half;
        T* vec = o + (t * H + h) * (size_t)n;
        const float a = ld(vec, p), b = ld(vec, p + half), c = cs[p], s = cs[half + p] * sign;
        st(vec, p, a * c - b * s);
        st(vec, p + half, b * c + a * s);
    }
}
}  // namespace

extern "C" int qsv_decay(float* out, const void* z, int64_t z_stride, const void* bias, const float* a_log, float tau, int n_tokens,
                         int heads, int dim, int dtype, void* stream) {
    QSV_REQUIRE(out && z && bias && n_tokens >= 0 && heads > 0 && dim > 0 && z_stride >= (int64_t)heads * dim,
                "qsv_decay: bad arguments");
    QSV_REQUIRE(a_log || tau > 0.f, "qsv_decay: a power-sigmoid decay needs tau > 0");
    if (n_tokens == 0) return QSV_OK;
    QSV_DISPATCH(dtype, "qsv_decay",
                 hipLaunchKernelGGL(decay_kernel<T>, dim3(n_tokens), dim3(NT), 0, (hipStream_t)stream, out, (const T*)z, z_stride,
                                    (const T*)bias, a_log, a_log ? 0.f : 1.0f / tau, dim, heads * dim));
    return qsv_launch_status("qsv_decay");
}

extern "C" int qsv_conv_silu_unit(float* out, const void* proj, int64_t stride, int off, int channels, int taps, const float* w,
                                  float* hist, const int32_t* run_off, const int32_t* state_rd, const int32_t* state_wr,
                                  int n_unit, int unit_dim, int act, int n_tokens, int dtype, void* stream) {
    QSV_REQUIRE(out && proj && w && hist && run_off && state_rd && state_wr, "qsv_conv_silu_unit: null argument");
    QSV_REQUIRE(channels > 0 && taps >= 1 && off >= 0 && off + channels <= stride && n_unit >= 0 && unit_dim > 0 &&
                    (int64_t)n_unit * unit_dim <= channels && n_tokens >= 0 && (act == 0 || act == 1),
                "qsv_conv_silu_unit: bad sizes");
    QSV_REQUIRE((size_t)channels * 4 <= 64 * 1024, "qsv_conv_silu_unit: %d channels do not fit the workgroup's LDS", channels);
    if (n_tokens == 0) return QSV_OK;
    QSV_DISPATCH(dtype, "qsv_conv_silu_unit",
                 hipLaunchKernelGGL(conv_silu_unit_kernel<T>, dim3(n_tokens), dim3(NT), (size_t)channels * 4, (hipStream_t)stream, out,
                                    (const T*)proj, stride, off, channels, taps, w, hist, run_off, state_rd, state_wr, n_unit,
                                    unit_dim, act));
    return qsv_launch_status("qsv_conv_silu_unit");
}

extern "C" int qsv_recurrent_scan(float* o, const void* q, int64_t q_stride, const void* k, int64_t k_stride, const void* v,
                                  int64_t v_stride, int qkv_dtype, const float* decay, const void* beta, int64_t beta_stride,
                                  int beta_dtype, float* state, const int32_t* runs, int n_runs, int max_run, int heads, int qk_heads,
                                  int dim, int vdim, float q_scale, const float* kscale, int head_decay, int v_cols, void* stream) {
    QSV_REQUIRE(o && q && k && v && decay && state && runs, "qsv_recurrent_scan: null argument");
    if (v_cols <= 0) v_cols = vdim;
    QSV_REQUIRE(v_cols <= vdim, "qsv_recurrent_scan: %d value columns for a state of %d", v_cols, vdim);
    if (max_run == 1 && n_runs > 0 && dim <= 64 * 8 && heads > 0 && qk_heads > 0 && heads % qk_heads == 0 && vdim > 0 && heads <= 65535) {
        int lpc = 1, lpc_log = 0;
        while (lpc * 8 < dim) lpc <<= 1, ++lpc_log;
        const int per_block = 4 * (64 / lpc);
        const dim3 grid(n_runs, heads, (vdim + per_block - 1) / per_block), block(256);
        QSV_REQUIRE(grid.z <= 65535, "qsv_recurrent_scan: too many column blocks");
#define QSV_STEP(TQ, TB, DELTA)                                                                                              \
    hipLaunchKernelGGL((recurrent_step_kernel<TQ, TB, DELTA>), grid, block, 0, (hipStream_t)stream, o, (const TQ*)q, q_stride,    \
                       (const TQ*)k, k_stride, (const TQ*)v, v_stride, decay, (const TB*)beta, beta_stride, state, runs, heads,  \
                       qk_heads, dim, vdim, lpc_log, q_scale, kscale, head_decay, v_cols)
        if (beta) {
            if (qkv_dtype == QSV_F32 && beta_dtype == QSV_F32) QSV_STEP(float, float, true);
            else if (qkv_dtype == QSV_F32 && beta_dtype == QSV_BF16) QSV_STEP(float, bf16_t, true);
            else if (qkv_dtype == QSV_BF16 && beta_dtype == QSV_BF16) QSV_STEP(bf16_t, bf16_t, true);
            else QSV_REQUIRE(false, "qsv_recurrent_scan: operand types %d / %d", qkv_dtype, beta_dtype);
        } else {
            if (qkv_dtype == QSV_F32) QSV_STEP(float, float, false);
            else if (qkv_dtype == QSV_BF16) QSV_STEP(bf16_t, bf16_t, false);
            else QSV_REQUIRE(false, "qsv_recurrent_scan: operand type %d", qkv_dtype);
        }
#undef QSV_STEP
        return qsv_launch_status("qsv_recurrent_scan");
    }
    // Rows of one column per lane: 8 while that leaves the launch at no more than ~2.5 waves per SIMD, else 16 (and for the tallest
    // states).  Measured at 16 heads, 64 x 128 states: 8 x 1024 tokens (2048 / 1024 waves) 0.46 / 0.51 ms plain, 0.50 / 0.55 ms
    // delta rule; 64 single tokens (16384 / 8192 waves) 56 / 43 us; two columns per lane 0.60 / 0.75 ms.  A token's step is a
    // short chain of dependent instructions: up to the chip's fill, more and lighter waves win; beyond it, fewer and heavier ones.
    int lpc8 = 1;
    while (lpc8 * 8 < dim) lpc8 <<= 1;
    const int64_t waves8 = (int64_t)n_runs * heads * (((int64_t)vdim * lpc8 + 63) / 64);
    int R = dim <= 64 * 8 && waves8 <= 2560 ? 8 : 16;
    const int NC = 1;
    // Both forms take about 230 registers: two four-wave workgroups of the 8-row form (one of the 16-row form) per CU, and a launch
    // of more workgroups than that runs in rounds, each as long as a full one (132 columns instead of 128 at 8 x 16 (run, head)
    // pairs: 0.94 ms instead of 0.49).  A third form - 8 rows, compiled for three waves per SIMD, half the staging - holds three
    // workgroups per CU at 1.23 times the round's length; it is taken where that saves rounds (costs in rounds of the 8-row form).
    bool three = false;
    if (!beta && dim <= 64 * 8) {
        const int cols8 = 64 / lpc8, wpb8 = (vdim + cols8 - 1) / cols8 >= 4 ? 4 : (vdim + cols8 - 1) / cols8 > 1 ? 2 : 1;
        const int64_t pairs = (int64_t)n_runs * heads;
        const int64_t groups8 = pairs * ((vdim + wpb8 * cols8 - 1) / (wpb8 * cols8)) * wpb8 / 4;
        const int cols16 = cols8 * 2 > 64 ? 64 : cols8 * 2;
        const int64_t groups16 = pairs * ((vdim + 4 * cols16 - 1) / (4 * cols16));
        const double legacy = R == 8 ? (double)((groups8 + 511) / 512) : 1.12 * (double)((groups16 + 255) / 256);
        const double lean = 1.23 * (double)((groups8 + 767) / 768);
        const size_t el8 = qkv_dtype == QSV_F32 ? 4 : 2;         // (the third form has 16-byte staging only)
        const bool vec8 = dim % 4 == 0 && vdim % 4 == 0 && v_cols % 4 == 0 && (wpb8 * cols8) % 4 == 0 && q_stride % 4 == 0 &&
                          k_stride % 4 == 0 && v_stride % 4 == 0 && (uintptr_t)q % (4 * el8) == 0 && (uintptr_t)k % (4 * el8) == 0 &&
                          (uintptr_t)v % (4 * el8) == 0 && (uintptr_t)decay % 16 == 0;
        if (vec8 && lean < legacy) {
            three = true;
            R = 8;
        }
    }
    QSV_REQUIRE(heads > 0 && qk_heads > 0 && heads % qk_heads == 0 && dim > 0 && dim <= 64 * 16 && vdim > 0 && n_runs >= 0 &&
                    heads <= 65535,
                "qsv_recurrent_scan: bad sizes (%d heads over %d, state %d x %d)", heads, qk_heads, dim, vdim);
    if (n_runs == 0) return QSV_OK;
    int lpc = 1, lpc_log = 0;
    while (lpc * R < dim) lpc <<= 1, ++lpc_log;
    QSV_REQUIRE(lpc <= 64, "qsv_recurrent_scan: %d rows per lane for a state of %d rows", R, dim);
    const int cols = 64 / lpc, DIMP = lpc * R;
    const int waves_needed = (vdim + cols * NC - 1) / (cols * NC);
    // waves per workgroup: they share the staged k, q and decay (fewer: the staging loads multiply; more: the launch's waves
    // stack up on the CUs of a few large workgroups while a token's step is bound by instruction issue)
    int nw = 1;
    while (nw < 4 && nw < waves_needed) nw <<= 1;
    const int VB = nw * cols * NC, nthr = nw * 64;
    const size_t el = qkv_dtype == QSV_F32 ? 4 : 2;
    const bool vec = dim % 4 == 0 && vdim % 4 == 0 && v_cols % 4 == 0 && VB % 4 == 0 && q_stride % 4 == 0 && k_stride % 4 == 0 && v_stride % 4 == 0 &&
                     (uintptr_t)q % (4 * el) == 0 && (uintptr_t)k % (4 * el) == 0 && (uintptr_t)v % (4 * el) == 0 &&
                     (uintptr_t)decay % 16 == 0;
    const bool lean = three && vec;                              // (the variant for three waves per SIMD: half the staging)
    const int max_ct = lean ? SCAN_CT / 2 : SCAN_CT, pfk = lean ? SCAN_PFK / 2 : SCAN_PFK, pfv = lean ? SCAN_PFV / 2 : SCAN_PFV;
    int CT = max_ct;                                             // tokens per staged chunk: what the prefetch registers and 48 KiB hold
    while (CT > 1 && ((CT * 3 * DIMP + nthr - 1) / nthr > pfk || (CT * VB + nthr - 1) / nthr > pfv ||
                      (size_t)CT * (3 * DIMP + ((VB + 4) & ~3)) * 4 > 48 * 1024))
        CT >>= 1;
    QSV_REQUIRE((CT * 3 * DIMP + nthr - 1) / nthr <= pfk && (CT * VB + nthr - 1) / nthr <= pfv,
                "qsv_recurrent_scan: a state of %d rows does not fit the staging registers", dim);
    const size_t lds = (size_t)CT * (3 * DIMP + ((VB + 4) & ~3)) * 4;
    const dim3 grid(n_runs, heads, (vdim + VB - 1) / VB), block(nthr);
    QSV_REQUIRE(grid.z <= 65535, "qsv_recurrent_scan: too many column blocks");
#define QSV_SCAN_V(TQ, TB, DELTA, VEC, RR, CC, OC)                                                                              \
    hipLaunchKernelGGL((recurrent_scan_kernel<TQ, TB, DELTA, VEC, RR, CC, OC>), grid, block, lds, (hipStream_t)stream, o,        \
                       (const TQ*)q, q_stride, (const TQ*)k, k_stride, (const TQ*)v, v_stride, decay, (const TB*)beta,         \
                       beta_stride, state, runs, heads, qk_heads, dim, vdim, lpc_log, CT, q_scale, kscale, head_decay, v_cols)
#define QSV_SCAN(TQ, TB, DELTA)                                \
    do {                                                       \
        if (lean && !DELTA) QSV_SCAN_V(TQ, TB, false, true, 8, 1, 3);   \
        else if (vec && R == 8) QSV_SCAN_V(TQ, TB, DELTA, true, 8, 1, 1);   \
        else if (R == 8) QSV_SCAN_V(TQ, TB, DELTA, false, 8, 1, 1);    \
        else if (vec) QSV_SCAN_V(TQ, TB, DELTA, true, 16, 1, 1);       \
        else QSV_SCAN_V(TQ, TB, DELTA, false, 16, 1, 1);               \
    } while (0)
    if (beta) {
        if (qkv_dtype == QSV_F32 && beta_dtype == QSV_F32) QSV_SCAN(float, float, true);
        else if (qkv_dtype == QSV_F32 && beta_dtype == QSV_BF16) QSV_SCAN(float, bf16_t, true);
        else if (qkv_dtype == QSV_BF16 && beta_dtype == QSV_BF16) QSV_SCAN(bf16_t, bf16_t, true);
        else QSV_REQUIRE(false, "qsv_recurrent_scan: operand types %d / %d", qkv_dtype, beta_dtype);
    } else {
        if (qkv_dtype == QSV_F32) QSV_SCAN(float, float, false);
        else if (qkv_dtype == QSV_BF16) QSV_SCAN(bf16_t, bf16_t, false);
        else QSV_REQUIRE(false, "qsv_recurrent_scan: operand type %d", qkv_dtype);
    }
#undef QSV_SCAN
#undef QSV_SCAN_V
    return qsv_launch_status("qsv_recurrent_scan");
}

extern "C" int qsv_head_rms_gate(void* out, const float* o, const void* w, const void* gate, int64_t gate_stride, int gate_kind,
                                 float eps, int n_tokens, int heads, int vdim, int o_stride, int w_per_head, const float* den_m,
                                 int dtype, void* stream) {
    QSV_REQUIRE(out && o && w && gate && n_tokens >= 0 && heads > 0 && vdim > 0 && gate_stride >= (int64_t)heads * vdim &&
                    (gate_kind == 0 || gate_kind == 1),
                "qsv_head_rms_gate: bad arguments");
    if (o_stride <= 0) o_stride = vdim;
    QSV_REQUIRE(o_stride >= vdim && (!den_m || o_stride > vdim), "qsv_head_rms_gate: read-out rows of %d floats for %d values%s",
                o_stride, vdim, den_m ? " and the normaliser's column" : "");
    if (n_tokens == 0) return QSV_OK;
    QSV_DISPATCH(dtype, "qsv_head_rms_gate",
                 hipLaunchKernelGGL(head_rms_gate_kernel<T>, dim3(n_tokens), dim3(NT), 0, (hipStream_t)stream, (T*)out, o, (const T*)w,
                                    (const T*)gate, gate_stride, gate_kind, eps, heads, vdim, o_stride, w_per_head ? vdim : 0, den_m));
    return qsv_launch_status("qsv_head_rms_gate");
}

extern "C" int qsv_max_gates(float* a, float* b, float* m, const void* zi, const void* zf, int64_t z_stride, const float* bias_i,
                             const float* bias_f, float cap, float* m_state, const int32_t* runs, int n_runs, int heads, int dtype,
                             void* stream) {
    QSV_REQUIRE(a && b && m && zi && zf && bias_i && bias_f && m_state && runs, "qsv_max_gates: null argument");
    QSV_REQUIRE(cap > 0.f && heads > 0 && heads <= 65535 && n_runs >= 0 && z_stride >= heads, "qsv_max_gates: bad sizes");
    if (n_runs == 0) return QSV_OK;
    QSV_DISPATCH(dtype, "qsv_max_gates",
                 hipLaunchKernelGGL(max_gates_kernel<T>, dim3(n_runs, heads), dim3(64), 0, (hipStream_t)stream, a, b, m, (const T*)zi,
                                    (const T*)zf, z_stride, bias_i, bias_f, cap, m_state, runs, heads));
    return qsv_launch_status("qsv_max_gates");
}

extern "C" int qsv_attention_prep(float* qf, void* pool, int64_t pool_rows, const void* proj, int64_t stride, int q_off, int k_off,
                                  int v_off, int heads, int kv_heads, int dim, int vdim, int rot_n, const float* rope_k,
                                  const float* rope_v, float scale, const int64_t* slot, const int32_t* pos, int n_tokens,
                                  int dtype, void* stream) {
    QSV_REQUIRE(qf && pool && proj && rope_k && rope_v && slot && pos, "qsv_attention_prep: null argument");
    QSV_REQUIRE(heads > 0 && kv_heads > 0 && dim > 0 && vdim > 0 && vdim % 2 == 0 && rot_n >= 0 && rot_n % 2 == 0 && rot_n <= dim &&
                    q_off >= 0 && k_off >= 0 && v_off >= 0 && q_off + (int64_t)heads * dim <= stride &&
                    k_off + (int64_t)kv_heads * dim <= stride && v_off + (int64_t)kv_heads * vdim <= stride && n_tokens >= 0,
                "qsv_attention_prep: bad sizes");
    if (n_tokens == 0) return QSV_OK;
    QSV_DISPATCH(dtype, "qsv_attention_prep",
                 hipLaunchKernelGGL(attention_prep_kernel<T>, dim3(n_tokens), dim3(NT), 0, (hipStream_t)stream, qf, (T*)pool, pool_rows,
                                    (const T*)proj, stride, q_off, k_off, v_off, heads, kv_heads, dim, vdim, rot_n, rope_k, rope_v,
                                    scale, slot, pos));
    return qsv_launch_status("qsv_attention_prep");
}

extern "C" int qsv_rotate_heads(void* o, const float* rope, const int32_t* pos, float sign, int n_tokens, int heads, int n,
                                int dtype, void* stream) {
    QSV_REQUIRE(o && rope && pos && n_tokens >= 0 && heads > 0 && n > 0 && n % 2 == 0, "qsv_rotate_heads: bad arguments");
    if (n_tokens == 0) return QSV_OK;
    QSV_DISPATCH(dtype, "qsv_rotate_heads",
                 hipLaunchKernelGGL(rotate_heads_kernel<T>, dim3(n_tokens), dim3(NT), 0, (hipStream_t)stream, (T*)o, rope, pos, sign,
                                    heads, n));
    return qsv_launch_status("qsv_rotate_heads");
}


// ---- element-wise gated recurrence (minGRU) ---------------------------------------------------------------------------------------
// Thread = one channel of one run; the run's tokens are walked in order, UN at a time: the UN tokens' three pre-activations are
// requested together (rows of the batch, coalesced over the channels), the gates are computed, then the UN dependent steps run.
// Gates, candidate and state are float.
template <typename T>
__global__ __launch_bounds__(NT) void min_gru_scan_kernel(T* __restrict__ out, const T* __restrict__ proj, int64_t stride, int z_off,
                                                          int x_off, int g_off, const T* __restrict__ b_z, const T* __restrict__ b_x,
                                                          float* __restrict__ state, const int32_t* __restrict__ runs, int width) {
    constexpr int UN = 8;
    const int i = blockIdx.x * NT + threadIdx.x;
    if (i >= width) return;
    const int32_t* r = runs + 4 * blockIdx.y;
    const int slot = r[0], first = r[1], n = r[2], p0 = r[3];
    float S = p0 > 0 ? state[(size_t)slot * width + i] : 0.f;
    const float bz = ld(b_z, i), bx = ld(b_x, i);
    for (int t0 = 0; t0 < n; t0 += UN) {
        float z[UN], u[UN], g[UN];
#pragma unroll
        for (int j = 0; j < UN; ++j) {
            const size_t row = (size_t)(first + min(t0 + j, n - 1)) * stride;
            z[j] = ld(proj, row + z_off + i);
            u[j] = ld(proj, row + x_off + i);
            g[j] = ld(proj, row + g_off + i);
        }
#pragma unroll
        for (int j = 0; j < UN; ++j) {
            z[j] = 1.0f / (1.0f + expf(-(z[j] + bz)));
            const float uu = u[j] + bx;
            u[j] = uu >= 0.f ? uu + 0.5f : 1.0f / (1.0f + expf(-uu));
            g[j] = g[j] / (1.0f + expf(-g[j]));
        }
#pragma unroll
        for (int j = 0; j < UN; ++j) {
            if (t0 + j < n) {
                S = (1.0f - z[j]) * S + z[j] * u[j];
                st(out, (size_t)(first + t0 + j) * width + i, S * g[j]);
            }
        }
    }
    state[(size_t)slot * width + i] = S;
}
// Long runs (prompt portions): a workgroup of SEG waves owns 64 channels of one run and cuts the run's tokens into SEG segments, one
// a wave.  The recurrence S <- a S + b (a = 1 - z, b = z c) composes: a segment as a whole maps S to A S + B with A the product of
// its a and B its own scan from zero.  Pass 1: every wave walks its segment for (A, B); the waves exchange them through LDS and each
// folds its predecessors' into the state its segment starts from; pass 2: the segment again (from L2), now with outputs.
template <typename T>
__global__ __launch_bounds__(64 * 8) void min_gru_scan_segments_kernel(T* __restrict__ out, const T* __restrict__ proj, int64_t stride,
                                                                       int z_off, int x_off, int g_off, const T* __restrict__ b_z,
                                                                       const T* __restrict__ b_x, float* __restrict__ state,
                                                                       const int32_t* __restrict__ runs, int width) {
    constexpr int SEG = 8, UN = 8;
    __shared__ float sA[SEG][64], sB[SEG][64];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int ch = blockIdx.x * 64 + lane;
    const bool valid = ch < width;
    const int i = valid ? ch : width - 1;
    const int32_t* r = runs + 4 * blockIdx.y;
    const int slot = r[0], first = r[1], n = r[2], p0 = r[3];
    const int per = (n + SEG - 1) / SEG;
    const int t_lo = min(n, w * per), t_hi = min(n, t_lo + per);
    const float bz = ld(b_z, i), bx = ld(b_x, i);
    float A = 1.f, B = 0.f;
    for (int t0 = t_lo; t0 < t_hi; t0 += UN) {
        float z[UN], u[UN];
#pragma unroll
        for (int j = 0; j < UN; ++j) {
            const size_t row = (size_t)(first + min(t0 + j, t_hi - 1)) * stride;
            z[j] = ld(proj, row + z_off + i);
            u[j] = ld(proj, row + x_off + i);
        }
#pragma unroll
        for (int j = 0; j < UN; ++j) {
            const float zz = 1.0f / (1.0f + expf(-(z[j] + bz)));
            const float uu = u[j] + bx;
            const float c = uu >= 0.f ? uu + 0.5f : 1.0f / (1.0f + expf(-uu));
            if (t0 + j < t_hi) {
                A *= 1.0f - zz;
                B = (1.0f - zz) * B + zz * c;
            }
        }
    }
    sA[w][lane] = A;
    sB[w][lane] = B;
    __syncthreads();
    float S = p0 > 0 ? state[(size_t)slot * width + i] : 0.f;
    for (int k = 0; k < w; ++k) S = sA[k][lane] * S + sB[k][lane];
    for (int t0 = t_lo; t0 < t_hi; t0 += UN) {
        float z[UN], u[UN], g[UN];
#pragma unroll
        for (int j = 0; j < UN; ++j) {
            const size_t row = (size_t)(first + min(t0 + j, t_hi - 1)) * stride;
            z[j] = ld(proj, row + z_off + i);
            u[j] = ld(proj, row + x_off + i);
            g[j] = ld(proj, row + g_off + i);
        }
#pragma unroll
        for (int j = 0; j < UN; ++j) {
            z[j] = 1.0f / (1.0f + expf(-(z[j] + bz)));
            const float uu = u[j] + bx;
            u[j] = uu >= 0.f ? uu + 0.5f : 1.0f / (1.0f + expf(-uu));
            g[j] = g[j] / (1.0f + expf(-g[j]));
        }
#pragma unroll
        for (int j = 0; j < UN; ++j) {
            if (t0 + j < t_hi) {
                S = (1.0f - z[j]) * S + z[j] * u[j];
                if (valid) st(out, (size_t)(first + t0 + j) * width + i, S * g[j]);
            }
        }
    }
    if (w == SEG - 1 && valid) state[(size_t)slot * width + i] = S;     // (the last wave ends with the run's last state, also if its segment is empty)
}
extern "C" int qsv_min_gru_scan(void* out, const void* proj, int64_t stride, int z_off, int x_off, int g_off, const void* b_z,
                                const void* b_x, float* state, const int32_t* runs, int n_runs, int max_run, int width, int dtype,
                                void* stream) {
    QSV_REQUIRE(out && proj && b_z && b_x && state && runs, "qsv_min_gru_scan: null argument");
    QSV_REQUIRE(width > 0 && n_runs >= 0 && n_runs <= 65535 && z_off >= 0 && x_off >= 0 && g_off >= 0 &&
                    (int64_t)z_off + width <= stride && (int64_t)x_off + width <= stride && (int64_t)g_off + width <= stride,
                "qsv_min_gru_scan: bad sizes");
    if (n_runs == 0) return QSV_OK;
    if (max_run <= 0 || max_run > 32) {          // (0: unknown) long runs: segments of the run side by side
        QSV_DISPATCH(dtype, "qsv_min_gru_scan",
                     hipLaunchKernelGGL(min_gru_scan_segments_kernel<T>, dim3((width + 63) / 64, n_runs), dim3(64 * 8), 0,
                                        (hipStream_t)stream, (T*)out, (const T*)proj, stride, z_off, x_off, g_off, (const T*)b_z,
                                        (const T*)b_x, state, runs, width));
        return qsv_launch_status("qsv_min_gru_scan");
    }
    QSV_DISPATCH(dtype, "qsv_min_gru_scan",
                 hipLaunchKernelGGL(min_gru_scan_kernel<T>, dim3((width + NT - 1) / NT, n_runs), dim3(NT), 0, (hipStream_t)stream,
                                    (T*)out, (const T*)proj, stride, z_off, x_off, g_off, (const T*)b_z, (const T*)b_x, state, runs,
                                    width));
    return qsv_launch_status("qsv_min_gru_scan");
}
