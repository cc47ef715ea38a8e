// serve_streams.hip -- one-workgroup-per-token kernels for models that keep several residual streams: the scaled embedding
// into all streams, the read of a sublayer's input (weighted sum of the streams, the statistics-free tanh norm, the token
// shift with its per-sequence state), the rewrite of all streams from a sublayer's output, the final norm over the streams'
// sum; and two small row kernels of the same models (RMS-normed mean of two branches, gated-unit activation).
// Streams, sums and norms are float; only what leaves for a matrix product is in the storage type.
#include "serve_common.h"

namespace {
constexpr int NT = 256;
constexpr int MAX_STREAMS = 16;

template <typename T>
__global__ __launch_bounds__(NT) void embed_streams_kernel(float* __restrict__ x, const T* __restrict__ table,
                                                           const int32_t* __restrict__ tokens, float scale, int S, int D) {
    const size_t t = blockIdx.x;
    const T* row = table + (size_t)tokens[t] * D;
    for (int i = threadIdx.x; i < D; i += NT) {
        const float v = ld(row, i) * scale;
        for (int s = 0; s < S; ++s) x[(t * S + s) * D + i] = v;
    }
}

__device__ __forceinline__ float stream_sum(const float* __restrict__ x, const float* __restrict__ w_in, size_t t, int S, int D,
                                            int i) {
    float u = 0.f;
    for (int s = 0; s < S; ++s) u += w_in[s] * x[(t * S + s) * D + i];
    return u;
}

// h[t] = n + (before - n) * shift,  n = tanh(alpha * sum_s w_in[s] x[t, s]) * w + b, `before` = the same n of the previous
// token of the sequence: recomputed from the previous row of the batch inside a run, read from the sequence's state at a run's
// start (zeros when the run starts the sequence).  The last token of a run leaves its n in the state's other copy.
template <typename T>
__global__ __launch_bounds__(NT) void hc_read_kernel(T* __restrict__ h, const float* __restrict__ x, const float* __restrict__ w_in,
                                                     const T* __restrict__ nw, const T* __restrict__ nb, float alpha,
                                                     const T* __restrict__ shift, float* __restrict__ prev,
                                                     const int32_t* __restrict__ run_off, const int32_t* __restrict__ state_rd,
                                                     const int32_t* __restrict__ state_wr, int S, int D) {
    const size_t t = blockIdx.x;
    const bool shifted = shift != nullptr;
    const int off = shifted ? run_off[t] : 0, rd = shifted ? state_rd[t] : -1, wr = shifted ? state_wr[t] : -1;
    for (int i = threadIdx.x; i < D; i += NT) {
        const float w = ld(nw, i), b = ld(nb, i);
        float n = tanhf(alpha * stream_sum(x, w_in, t, S, D, i)) * w + b;
        if (shifted) {
            float before = 0.f;
            if (off > 0) before = tanhf(alpha * stream_sum(x, w_in, t - 1, S, D, i)) * w + b;
            else if (rd >= 0) before = prev[(size_t)rd * D + i];
            if (wr >= 0) prev[(size_t)wr * D + i] = n;
            n += (before - n) * ld(shift, i);
        }
        st(h, t * D + i, n);
    }
}

// x[t, r] <- sum_s mix[s, r] x[t, s] + out[r] * y[t], all streams from the old ones; and, if asked for, the next sublayer's
// input from the new streams in the same pass (no token shift there: that needs the previous token's NEW streams)
template <typename T>
__global__ __launch_bounds__(NT) void hc_write_kernel(float* __restrict__ x, const T* __restrict__ y, const float* __restrict__ mix,
                                                      const float* __restrict__ w_out, int S, int D, T* __restrict__ h_next,
                                                      const float* __restrict__ w_in_next, const T* __restrict__ nw,
                                                      const T* __restrict__ nb, float alpha) {
    const size_t t = blockIdx.x;
    for (int i = threadIdx.x; i < D; i += NT) {
        float old[MAX_STREAMS];
#pragma unroll
        for (int s = 0; s < MAX_STREAMS; ++s) old[s] = s < S ? x[(t * S + s) * D + i] : 0.f;
        const float yv = ld(y, t * D + i);
        float u = 0.f;
        for (int r = 0; r < S; ++r) {
            float a = w_out[r] * yv;
#pragma unroll
            for (int s = 0; s < MAX_STREAMS; ++s)
                if (s < S) a += mix[s * S + r] * old[s];
            x[(t * S + r) * D + i] = a;
            if (h_next) u += w_in_next[r] * a;
        }
        if (h_next) st(h_next, t * D + i, tanhf(alpha * u) * ld(nw, i) + ld(nb, i));
    }
}

// ---- the same two kernels for widths that are multiples of four: 16-byte stream accesses, four elements per thread and pass ----
__device__ __forceinline__ void ld4t(const float* p, size_t i, float (&v)[4]) {
    const float4 a = *(const float4*)(p + i);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
}
__device__ __forceinline__ void ld4t(const bf16_t* p, size_t i, float (&v)[4]) {
    const uint2 u = *(const uint2*)(p + i);
    v[0] = __uint_as_float(u.x << 16); v[1] = __uint_as_float(u.x & 0xffff0000u);
    v[2] = __uint_as_float(u.y << 16); v[3] = __uint_as_float(u.y & 0xffff0000u);
}
__device__ __forceinline__ void st4t(float* p, size_t i, const float (&v)[4]) { *(float4*)(p + i) = make_float4(v[0], v[1], v[2], v[3]); }
__device__ __forceinline__ void st4t(bf16_t* p, size_t i, const float (&v)[4]) {
    *(uint2*)(p + i) = make_uint2((unsigned)f2bf(v[0]) | ((unsigned)f2bf(v[1]) << 16), (unsigned)f2bf(v[2]) | ((unsigned)f2bf(v[3]) << 16));
}
__device__ __forceinline__ void stream_sum4(const float* __restrict__ x, const float* __restrict__ w_in, size_t t, int S, int D, int i,
                                            float (&u)[4]) {
    u[0] = u[1] = u[2] = u[3] = 0.f;
    for (int s = 0; s < S; ++s) {
        float v[4];
        ld4t(x, (t * S + s) * D + i, v);
        const float w = w_in[s];
#pragma unroll
        for (int j = 0; j < 4; ++j) u[j] += w * v[j];
    }
}

template <typename T>
__global__ __launch_bounds__(NT) void hc_read_vec_kernel(T* __restrict__ h, const float* __restrict__ x, const float* __restrict__ w_in,
                                                         const T* __restrict__ nw, const T* __restrict__ nb, float alpha,
                                                         const T* __restrict__ shift, float* __restrict__ prev,
                                                         const int32_t* __restrict__ run_off, const int32_t* __restrict__ state_rd,
                                                         const int32_t* __restrict__ state_wr, int S, int D) {
    const size_t t = blockIdx.x;
    const bool shifted = shift != nullptr;
    const int off = shifted ? run_off[t] : 0, rd = shifted ? state_rd[t] : -1, wr = shifted ? state_wr[t] : -1;
    for (int i = threadIdx.x * 4; i < D; i += NT * 4) {
        float w[4], b[4], u[4], n[4];
        ld4t(nw, i, w);
        ld4t(nb, i, b);
        stream_sum4(x, w_in, t, S, D, i, u);
#pragma unroll
        for (int j = 0; j < 4; ++j) n[j] = tanhf(alpha * u[j]) * w[j] + b[j];
        if (shifted) {
            float before[4] = {0.f, 0.f, 0.f, 0.f}, mu[4];
            if (off > 0) {
                stream_sum4(x, w_in, t - 1, S, D, i, u);
#pragma unroll
                for (int j = 0; j < 4; ++j) before[j] = tanhf(alpha * u[j]) * w[j] + b[j];
            } else if (rd >= 0) {
                ld4t(prev, (size_t)rd * D + i, before);
            }
            if (wr >= 0) st4t(prev, (size_t)wr * D + i, n);
            ld4t(shift, i, mu);
#pragma unroll
            for (int j = 0; j < 4; ++j) n[j] += (before[j] - n[j]) * mu[j];
        }
        st4t(h, t * D + i, n);
    }
}

template <typename T>
__global__ __launch_bounds__(NT) void hc_write_vec_kernel(float* __restrict__ x, const T* __restrict__ y, const float* __restrict__ mix,
                                                          const float* __restrict__ w_out, int S, int D, T* __restrict__ h_next,
                                                          const float* __restrict__ w_in_next, const T* __restrict__ nw,
                                                          const T* __restrict__ nb, float alpha) {
    const size_t t = blockIdx.x;
    for (int i = threadIdx.x * 4; i < D; i += NT * 4) {
        float old[MAX_STREAMS][4], yv[4], u[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < MAX_STREAMS; ++s)
            if (s < S) ld4t(x, (t * S + s) * D + i, old[s]);
        ld4t(y, t * D + i, yv);
        for (int r = 0; r < S; ++r) {
            float a[4];
            const float wo = w_out[r];
#pragma unroll
            for (int j = 0; j < 4; ++j) a[j] = wo * yv[j];
#pragma unroll
            for (int s = 0; s < MAX_STREAMS; ++s)
                if (s < S) {
                    const float m = mix[s * S + r];
#pragma unroll
                    for (int j = 0; j < 4; ++j) a[j] += m * old[s][j];
                }
            st4t(x, (t * S + r) * D + i, a);
            if (h_next) {
                const float wi = w_in_next[r];
#pragma unroll
                for (int j = 0; j < 4; ++j) u[j] += wi * a[j];
            }
        }
        if (h_next) {
            float w[4], b[4], n[4];
            ld4t(nw, i, w);
            ld4t(nb, i, b);
#pragma unroll
            for (int j = 0; j < 4; ++j) n[j] = tanhf(alpha * u[j]) * w[j] + b[j];
            st4t(h_next, t * D + i, n);
        }
    }
}

template <typename T>
__global__ __launch_bounds__(NT) void dyt_sum_rows_kernel(T* __restrict__ out, const float* __restrict__ x,
                                                          const int32_t* __restrict__ rows, const T* __restrict__ nw,
                                                          const T* __restrict__ nb, float alpha, int S, int D) {
    const size_t r = blockIdx.x;
    const size_t t = rows ? (size_t)rows[r] : r;
    for (int i = threadIdx.x; i < D; i += NT) {
        float u = 0.f;
        for (int s = 0; s < S; ++s) u += x[(t * S + s) * D + i];
        st(out, r * D + i, tanhf(alpha * u) * ld(nw, i) + ld(nb, i));
    }
}

// out[t] = (a[t] / rms(a[t]) * wa + b[t] / rms(b[t]) * wb) / 2
template <typename T>
__global__ __launch_bounds__(NT) void rms_pair_mean_kernel(T* __restrict__ out, const T* __restrict__ a, const T* __restrict__ wa,
                                                           const T* __restrict__ b, const T* __restrict__ wb, float eps, int D) {
    __shared__ float red[NT / 64 + 1];
    const size_t t = blockIdx.x;
    float sa = 0.f, sb = 0.f;
    for (int i = threadIdx.x; i < D; i += NT) {
        const float u = ld(a, t * D + i), v = ld(b, t * D + i);
        sa += u * u;
        sb += v * v;
    }
    const float ia = 1.0f / sqrtf(block_sum<NT>(sa, red) / (float)D + eps);
    const float ib = 1.0f / sqrtf(block_sum<NT>(sb, red) / (float)D + eps);
    for (int i = threadIdx.x; i < D; i += NT)
        st(out, t * D + i, 0.5f * (ld(a, t * D + i) * ia * ld(wa, i) + ld(b, t * D + i) * ib * ld(wb, i)));
}

// out[r, f] = act(a[r, 2f]) * a[r, 2f + 1];  act 0: silu, 1: gelu in its tanh form, 0.5 z (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3)));
// act 2: g = min(gate, limit), u = clamp(up, -limit, limit) -> g sigmoid(1.702 g) (u + 1)
template <typename T>
__global__ __launch_bounds__(NT) void glu_kernel(T* __restrict__ out, const T* __restrict__ a, int ff, int act, float limit) {
    const size_t r = blockIdx.x;
    for (int f = threadIdx.x; f < ff; f += NT) {
        float g = ld(a, (r * ff + f) * 2), u = ld(a, (r * ff + f) * 2 + 1);
        if (act == 2) {
            g = fminf(g, limit);
            u = fminf(fmaxf(u, -limit), limit);
            st(out, r * ff + f, g / (1.0f + expf(-1.702f * g)) * (u + 1.0f));
            continue;
        }
        const float ag = act == 0 ? g / (1.0f + expf(-g)) : 0.5f * g * (1.0f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g)));
        st(out, r * ff + f, ag * u);
    }
}
}  // namespace

extern "C" int qsv_embed_streams(float* x, const void* table, const int32_t* tokens, float scale, int n, int streams, int D,
                                 int dtype, void* stream) {
    QSV_REQUIRE(x && table && tokens && n >= 0 && D > 0 && streams > 0, "qsv_embed_streams: bad arguments");
    if (n == 0) return QSV_OK;
    QSV_DISPATCH(dtype, "qsv_embed_streams",
                 hipLaunchKernelGGL(embed_streams_kernel<T>, dim3(n), dim3(NT), 0, (hipStream_t)stream, x, (const T*)table, tokens,
                                    scale, streams, D));
    return qsv_launch_status("qsv_embed_streams");
}

extern "C" int qsv_hc_read(void* h, const float* x, const float* w_in, const void* norm_w, const void* norm_b, float alpha,
                           const void* shift, float* prev, const int32_t* run_off, const int32_t* state_rd,
                           const int32_t* state_wr, int n, int streams, int D, int dtype, void* stream) {
    QSV_REQUIRE(h && x && w_in && norm_w && norm_b && n >= 0 && D > 0 && streams > 0, "qsv_hc_read: bad arguments");
    QSV_REQUIRE(!shift || (prev && run_off && state_rd && state_wr), "qsv_hc_read: token shift without its state");
    if (n == 0) return QSV_OK;
    if (D % 4 == 0)
        QSV_DISPATCH(dtype, "qsv_hc_read",
                     hipLaunchKernelGGL(hc_read_vec_kernel<T>, dim3(n), dim3(NT), 0, (hipStream_t)stream, (T*)h, x, w_in,
                                        (const T*)norm_w, (const T*)norm_b, alpha, (const T*)shift, prev, run_off, state_rd, state_wr,
                                        streams, D));
    else
        QSV_DISPATCH(dtype, "qsv_hc_read",
                     hipLaunchKernelGGL(hc_read_kernel<T>, dim3(n), dim3(NT), 0, (hipStream_t)stream, (T*)h, x, w_in, (const T*)norm_w,
                                        (const T*)norm_b, alpha, (const T*)shift, prev, run_off, state_rd, state_wr, streams, D));
    return qsv_launch_status("qsv_hc_read");
}

extern "C" int qsv_hc_write(float* x, const void* y, const float* mix, const float* w_out, int n, int streams, int D, void* h_next,
                            const float* w_in_next, const void* norm_w, const void* norm_b, float alpha, int dtype, void* stream) {
    QSV_REQUIRE(x && y && mix && w_out && n >= 0 && D > 0, "qsv_hc_write: bad arguments");
    QSV_REQUIRE(!h_next || (w_in_next && norm_w && norm_b), "qsv_hc_write: the next sublayer's input without its weights");
    QSV_REQUIRE(streams > 0 && streams <= MAX_STREAMS, "qsv_hc_write: %d streams (at most %d)", streams, MAX_STREAMS);
    if (n == 0) return QSV_OK;
    if (D % 4 == 0)
        QSV_DISPATCH(dtype, "qsv_hc_write",
                     hipLaunchKernelGGL(hc_write_vec_kernel<T>, dim3(n), dim3(NT), 0, (hipStream_t)stream, x, (const T*)y, mix, w_out,
                                        streams, D, (T*)h_next, w_in_next, (const T*)norm_w, (const T*)norm_b, alpha));
    else
        QSV_DISPATCH(dtype, "qsv_hc_write",
                     hipLaunchKernelGGL(hc_write_kernel<T>, dim3(n), dim3(NT), 0, (hipStream_t)stream, x, (const T*)y, mix, w_out,
                                        streams, D, (T*)h_next, w_in_next, (const T*)norm_w, (const T*)norm_b, alpha));
    return qsv_launch_status("qsv_hc_write");
}

extern "C" int qsv_dyt_sum_rows(void* out, const float* x, const int32_t* rows, const void* norm_w, const void* norm_b,
                                float alpha, int n_rows, int streams, int D, int dtype, void* stream) {
    QSV_REQUIRE(out && x && norm_w && norm_b && n_rows >= 0 && D > 0 && streams > 0, "qsv_dyt_sum_rows: bad arguments");
    if (n_rows == 0) return QSV_OK;
    QSV_DISPATCH(dtype, "qsv_dyt_sum_rows",
                 hipLaunchKernelGGL(dyt_sum_rows_kernel<T>, dim3(n_rows), dim3(NT), 0, (hipStream_t)stream, (T*)out, x, rows,
                                    (const T*)norm_w, (const T*)norm_b, alpha, streams, D));
    return qsv_launch_status("qsv_dyt_sum_rows");
}

extern "C" int qsv_rms_pair_mean(void* out, const void* a, const void* wa, const void* b, const void* wb, float eps, int n, int D,
                                 int dtype, void* stream) {
    QSV_REQUIRE(out && a && wa && b && wb && n >= 0 && D > 0, "qsv_rms_pair_mean: bad arguments");
    if (n == 0) return QSV_OK;
    QSV_DISPATCH(dtype, "qsv_rms_pair_mean",
                 hipLaunchKernelGGL(rms_pair_mean_kernel<T>, dim3(n), dim3(NT), 0, (hipStream_t)stream, (T*)out, (const T*)a,
                                    (const T*)wa, (const T*)b, (const T*)wb, eps, D));
    return qsv_launch_status("qsv_rms_pair_mean");
}

extern "C" int qsv_glu(void* out, const void* a, int n_rows, int ff, int act, float limit, int dtype, void* stream) {
    QSV_REQUIRE(out && a && n_rows >= 0 && ff > 0 && (act == 0 || act == 1 || (act == 2 && limit > 0.f)), "qsv_glu: bad arguments");
    if (n_rows == 0) return QSV_OK;
    QSV_DISPATCH(dtype, "qsv_glu",
                 hipLaunchKernelGGL(glu_kernel<T>, dim3(n_rows), dim3(NT), 0, (hipStream_t)stream, (T*)out, (const T*)a, ff, act, limit));
    return qsv_launch_status("qsv_glu");
}
