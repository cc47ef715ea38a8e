// serve_rows.hip -- one-workgroup-per-token kernels of the serving engine: embedding, fused residual + layer norm, the
// latent projections' norms + rotary + cache write, the latent query, the output gate.  Statistics and angles are float.
#include "serve_common.h"

static thread_local char g_err[512] = "";
void qsv_set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}
extern "C" int qsv_version(void) { return 1; }
extern "C" const char* qsv_arch(void) { return "gfx950"; }
extern "C" const char* qsv_last_error(void) { return g_err; }

constexpr int NT = 256;

// ---- embedding ---------------------------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(NT) void embed_kernel(float* __restrict__ x, T* __restrict__ h, const T* __restrict__ table,
                                                   const int32_t* __restrict__ tokens, int D) {
    const size_t t = blockIdx.x;
    const T* row = table + (size_t)tokens[t] * D;
    for (int i = threadIdx.x; i < D; i += NT) {
        const float v = ld(row, i);
        x[t * D + i] = v;
        st(h, t * D + i, v);
    }
}
extern "C" int qsv_embed(float* x, void* h, const void* table, const int32_t* tokens, int n, int D, int dtype, void* stream) {
    QSV_REQUIRE(x && h && table && tokens && n >= 0 && D > 0, "qsv_embed: bad arguments");
    if (n == 0) return QSV_OK;
    QSV_DISPATCH(dtype, "qsv_embed",
                 hipLaunchKernelGGL(embed_kernel<T>, dim3(n), dim3(NT), 0, (hipStream_t)stream, x, (T*)h, (const T*)table, tokens, D));
    return qsv_launch_status("qsv_embed");
}

// ---- x += layer_norm(y) * w ; h = x -------------------------------------------------------------------------------------------
// Two reductions (mean, then the mean of squared deviations); the row of y is re-read from cache, not held in registers, so any
// width works.
template <typename T>
__global__ __launch_bounds__(NT) void add_layer_norm_kernel(float* __restrict__ x, T* __restrict__ h, const T* __restrict__ y,
                                                            const T* __restrict__ w, float eps, int D) {
    __shared__ float red[NT / 64 + 1];
    const size_t t = blockIdx.x;
    const T* yr = y + t * D;
    float s = 0.f;
    for (int i = threadIdx.x; i < D; i += NT) s += ld(yr, i);
    const float mean = block_sum<NT>(s, red) / (float)D;
    float q = 0.f;
    for (int i = threadIdx.x; i < D; i += NT) {
        const float d = ld(yr, i) - mean;
        q += d * d;
    }
    const float inv = 1.0f / sqrtf(block_sum<NT>(q, red) / (float)D + eps);
    for (int i = threadIdx.x; i < D; i += NT) {
        const float v = x[t * D + i] + (ld(yr, i) - mean) * inv * ld(w, i);
        x[t * D + i] = v;
        st(h, t * D + i, v);
    }
}
extern "C" int qsv_add_layer_norm(float* x, void* h, const void* y, const void* w, float eps, int n, int D, int dtype,
                                  void* stream) {
    QSV_REQUIRE(x && h && y && w && n >= 0 && D > 0, "qsv_add_layer_norm: bad arguments");
    if (n == 0) return QSV_OK;
    QSV_DISPATCH(dtype, "qsv_add_layer_norm",
                 hipLaunchKernelGGL(add_layer_norm_kernel<T>, dim3(n), dim3(NT), 0, (hipStream_t)stream, x, (T*)h, (const T*)y,
                                    (const T*)w, eps, D));
    return qsv_launch_status("qsv_add_layer_norm");
}

template <typename T>
__global__ __launch_bounds__(NT) void layer_norm_rows_kernel(T* __restrict__ out, const float* __restrict__ x,
                                                             const int32_t* __restrict__ rows, const T* __restrict__ w,
                                                             float eps, int D) {
    __shared__ float red[NT / 64 + 1];
    const size_t r = blockIdx.x;
    const float* xr = x + (size_t)(rows ? rows[r] : (int32_t)r) * D;
    float s = 0.f;
    for (int i = threadIdx.x; i < D; i += NT) s += xr[i];
    const float mean = block_sum<NT>(s, red) / (float)D;
    float q = 0.f;
    for (int i = threadIdx.x; i < D; i += NT) {
        const float d = xr[i] - mean;
        q += d * d;
    }
    const float inv = 1.0f / sqrtf(block_sum<NT>(q, red) / (float)D + eps);
    for (int i = threadIdx.x; i < D; i += NT) st(out, r * D + i, (xr[i] - mean) * inv * ld(w, i));
}
extern "C" int qsv_layer_norm_rows(void* out, const float* x, const int32_t* rows, const void* w, float eps, int n, int D,
                                   int dtype, void* stream) {
    QSV_REQUIRE(out && x && w && n >= 0 && D > 0, "qsv_layer_norm_rows: bad arguments");
    if (n == 0) return QSV_OK;
    QSV_DISPATCH(dtype, "qsv_layer_norm_rows",
                 hipLaunchKernelGGL(layer_norm_rows_kernel<T>, dim3(n), dim3(NT), 0, (hipStream_t)stream, (T*)out, x, rows,
                                    (const T*)w, eps, D));
    return qsv_launch_status("qsv_layer_norm_rows");
}

// ---- latent projections: two RMS norms, the rotary key part, the cache row ---------------------------------------------------
template <typename T>
__global__ __launch_bounds__(NT) void latent_prep_kernel(const T* __restrict__ down, int64_t down_stride, int q_off, int q_rank,
                                                         const T* __restrict__ q_w, T* __restrict__ cq, int kv_off, int kv_rank,
                                                         const T* __restrict__ kv_w, int rot_dim, int rot_n,
                                                         const float* __restrict__ rope, T* __restrict__ pool,
                                                         const int64_t* __restrict__ slot, const int32_t* __restrict__ pos,
                                                         float eps) {
    __shared__ float red[NT / 64 + 1];
    const size_t t = blockIdx.x;
    const T* row = down + t * down_stride;
    float s = 0.f;
    for (int i = threadIdx.x; i < q_rank; i += NT) {
        const float v = ld(row, q_off + i);
        s += v * v;
    }
    const float qinv = 1.0f / sqrtf(block_sum<NT>(s, red) / (float)q_rank + eps);
    for (int i = threadIdx.x; i < q_rank; i += NT) st(cq, t * q_rank + i, ld(row, q_off + i) * qinv * ld(q_w, i));
    s = 0.f;
    for (int i = threadIdx.x; i < kv_rank; i += NT) {
        const float v = ld(row, kv_off + i);
        s += v * v;
    }
    const float kinv = 1.0f / sqrtf(block_sum<NT>(s, red) / (float)kv_rank + eps);
    T* dst = pool + (size_t)slot[t] * (size_t)(kv_rank + rot_dim);
    for (int i = threadIdx.x; i < kv_rank; i += NT) st(dst, i, ld(row, kv_off + i) * kinv * ld(kv_w, i));
    const int half = rot_n / 2;
    const float* cs = rope ? rope + (size_t)pos[t] * (size_t)rot_n : nullptr;   // [2, half]: cos then sin
    const T* kr = row + kv_off + kv_rank;
    for (int i = threadIdx.x; i < rot_dim; i += NT) {
        float v = ld(kr, i);
        if (i < rot_n) {
            const int p = i >> 1;
            const float c = cs[p], sn = cs[half + p];
            const float u = ld(kr, 2 * p), w2 = ld(kr, 2 * p + 1);
            v = (i & 1) ? (w2 * c + u * sn) : (u * c - w2 * sn);
        }
        st(dst, kv_rank + i, v);
    }
}
extern "C" int qsv_latent_prep(const void* down, int64_t down_stride, int q_off, int q_rank, const void* q_w, void* cq,
                               int kv_off, int kv_rank, const void* kv_w, int rot_dim, int rot_n, const float* rope,
                               void* pool, const int64_t* slot, const int32_t* pos, float eps, int n, int dtype, void* stream) {
    QSV_REQUIRE(down && q_w && cq && kv_w && pool && slot && pos && n >= 0, "qsv_latent_prep: null argument");
    QSV_REQUIRE(q_rank > 0 && kv_rank > 0 && rot_dim >= 0 && rot_n >= 0 && rot_n <= rot_dim && rot_n % 2 == 0,
                "qsv_latent_prep: bad sizes (q_rank %d, kv_rank %d, rot_dim %d, rotated %d)", q_rank, kv_rank, rot_dim, rot_n);
    QSV_REQUIRE(rot_n == 0 || rope, "qsv_latent_prep: rotary part without a cos / sin table");
    QSV_REQUIRE(q_off >= 0 && kv_off >= 0 && q_off + q_rank <= down_stride && kv_off + kv_rank + rot_dim <= down_stride,
                "qsv_latent_prep: the slices do not fit a row of %lld elements", (long long)down_stride);
    if (n == 0) return QSV_OK;
    QSV_DISPATCH(dtype, "qsv_latent_prep",
                 hipLaunchKernelGGL(latent_prep_kernel<T>, dim3(n), dim3(NT), 0, (hipStream_t)stream, (const T*)down, down_stride,
                                    q_off, q_rank, (const T*)q_w, (T*)cq, kv_off, kv_rank, (const T*)kv_w, rot_dim, rot_n, rope,
                                    (T*)pool, slot, pos, eps));
    return qsv_launch_status("qsv_latent_prep");
}

// ---- the query in the latent space: [absorbed part | rotated part], scaled, float ---------------------------------------------
// One workgroup per token, all heads: the absorbed part is a strided gather ([H, T, rank] -> [T, H, rank + rot]), the rotated
// part a handful of values per head.
template <typename T>
__global__ __launch_bounds__(NT) void latent_query_kernel(float* __restrict__ qf, const T* __restrict__ q,
                                                          const T* __restrict__ q_abs, const float* __restrict__ rope,
                                                          const int32_t* __restrict__ pos, float scale, int n_tokens, int H,
                                                          int dim, int rot_dim, int rot_n, int rank) {
    const size_t t = blockIdx.x;
    const int R = rank + rot_dim;
    float* dst = qf + t * H * (size_t)R;
    for (int i = threadIdx.x; i < H * rank; i += NT) {
        const int h = i / rank, c = i - h * rank;
        dst[(size_t)h * R + c] = ld(q_abs, ((size_t)h * n_tokens + t) * (size_t)rank + c) * scale;
    }
    const int half = rot_n / 2;
    const float* cs = rope ? rope + (size_t)pos[t] * (size_t)rot_n : nullptr;
    for (int i = threadIdx.x; i < H * rot_dim; i += NT) {
        const int h = i / rot_dim, c = i - h * rot_dim;
        const T* qr = q + (t * H + h) * (size_t)(dim + rot_dim) + dim;
        float v = ld(qr, c);
        if (c < rot_n) {
            const int p = c >> 1;
            const float co = cs[p], sn = cs[half + p];
            const float u = ld(qr, 2 * p), w2 = ld(qr, 2 * p + 1);
            v = (c & 1) ? (w2 * co + u * sn) : (u * co - w2 * sn);
        }
        dst[(size_t)h * R + rank + c] = v * scale;
    }
}
extern "C" int qsv_latent_query(float* qf, const void* q, const void* q_abs, const float* rope, const int32_t* pos, float scale,
                                int n, int H, int dim, int rot_dim, int rot_n, int rank, int dtype, void* stream) {
    QSV_REQUIRE(qf && q && q_abs && pos && n >= 0 && H > 0 && dim > 0 && rank > 0, "qsv_latent_query: bad arguments");
    QSV_REQUIRE(rot_dim >= 0 && rot_n >= 0 && rot_n <= rot_dim && rot_n % 2 == 0 && (rot_n == 0 || rope),
                "qsv_latent_query: bad rotary sizes (%d of %d)", rot_n, rot_dim);
    if (n == 0) return QSV_OK;
    QSV_REQUIRE((int64_t)n * H < (1ll << 31), "qsv_latent_query: too many (token, head) pairs");
    QSV_DISPATCH(dtype, "qsv_latent_query",
                 hipLaunchKernelGGL(latent_query_kernel<T>, dim3(n), dim3(NT), 0, (hipStream_t)stream, qf, (const T*)q,
                                    (const T*)q_abs, rope, pos, scale, n, H, dim, rot_dim, rot_n, rank));
    return qsv_launch_status("qsv_latent_query");
}

// ---- output gate ---------------------------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(NT) void sigmoid_gate_kernel(T* __restrict__ o, const T* __restrict__ g, int64_t g_stride, int n) {
    const size_t t = blockIdx.x;
    for (int i = threadIdx.x; i < n; i += NT) {
        const float gate = 1.0f / (1.0f + expf(-ld(g, t * g_stride + i)));
        st(o, t * n + i, ld(o, t * n + i) * gate);
    }
}
extern "C" int qsv_sigmoid_gate(void* o, const void* g, int64_t g_stride, int n_tokens, int n, int dtype, void* stream) {
    QSV_REQUIRE(o && g && n_tokens >= 0 && n > 0 && g_stride >= n, "qsv_sigmoid_gate: bad arguments");
    if (n_tokens == 0) return QSV_OK;
    QSV_DISPATCH(dtype, "qsv_sigmoid_gate",
                 hipLaunchKernelGGL(sigmoid_gate_kernel<T>, dim3(n_tokens), dim3(NT), 0, (hipStream_t)stream, (T*)o, (const T*)g,
                                    g_stride, n));
    return qsv_launch_status("qsv_sigmoid_gate");
}

// ---- embedding with a sinusoidal position vector ---------------------------------------------------------------------------------
// x[t, 2i] = table[tok, 2i] * scale + sin(pos * freq[i]),  x[t, 2i + 1] = ... + cos(pos * freq[i]); the angle is a float product.
template <typename T>
__global__ __launch_bounds__(NT) void embed_sinusoid_kernel(float* __restrict__ x, const T* __restrict__ table,
                                                            const int32_t* __restrict__ tokens, const int32_t* __restrict__ pos,
                                                            const float* __restrict__ freq, float scale, int D) {
    const size_t t = blockIdx.x;
    const T* row = table + (size_t)tokens[t] * D;
    const float p = (float)pos[t];
    for (int i = threadIdx.x; i < D; i += NT) {
        const float a = p * freq[i >> 1];
        x[t * D + i] = ld(row, i) * scale + ((i & 1) ? cosf(a) : sinf(a));
    }
}
extern "C" int qsv_embed_sinusoid(float* x, const void* table, const int32_t* tokens, const int32_t* pos, const float* freq,
                                  float scale, int n, int D, int dtype, void* stream) {
    QSV_REQUIRE(x && table && tokens && pos && freq && n >= 0 && D > 0, "qsv_embed_sinusoid: bad arguments");
    if (n == 0) return QSV_OK;
    QSV_DISPATCH(dtype, "qsv_embed_sinusoid",
                 hipLaunchKernelGGL(embed_sinusoid_kernel<T>, dim3(n), dim3(NT), 0, (hipStream_t)stream, x, (const T*)table, tokens, pos,
                                    freq, scale, D));
    return qsv_launch_status("qsv_embed_sinusoid");
}

// ---- x += a + (b + c); h = rms_norm(x) * w -----------------------------------------------------------------------------------------
// a, b, c: the sublayers' outputs (each may be NULL); h (may be NULL: no norm) is the next layer's input in the storage type.
template <typename T>
__global__ __launch_bounds__(NT) void add_rms_norm_kernel(float* __restrict__ x, T* __restrict__ h, const T* __restrict__ a,
                                                          const T* __restrict__ b, const T* __restrict__ c, const T* __restrict__ w,
                                                          float eps, int D) {
    __shared__ float red[NT / 64 + 1];
    const size_t t = blockIdx.x;
    float s = 0.f;
    for (int i = threadIdx.x; i < D; i += NT) {
        float v = x[t * D + i];
        if (a || b || c) {
            float y = 0.f;
            if (b) y = ld(b, t * D + i);
            if (c) y += ld(c, t * D + i);
            if (a) y = ld(a, t * D + i) + y;
            v += y;
            x[t * D + i] = v;
        }
        s += v * v;
    }
    if (!h) return;
    const float inv = 1.0f / sqrtf(block_sum<NT>(s, red) / (float)D + eps);
    for (int i = threadIdx.x; i < D; i += NT) st(h, t * D + i, x[t * D + i] * inv * ld(w, i));   // (this thread's own writes)
}
// The same for widths that are multiples of four, up to 4 * NT * VPT: 16-byte accesses of the stream (8-byte of bfloat16 rows), the
// row stays in registers between the sum of squares and the scaling.
__device__ __forceinline__ float4 ld4v(const float* p, size_t i) { return *(const float4*)(p + i); }
__device__ __forceinline__ float4 ld4v(const bf16_t* p, size_t i) {
    const uint2 u = *(const uint2*)(p + i);
    return make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u), __uint_as_float(u.y << 16),
                       __uint_as_float(u.y & 0xffff0000u));
}
__device__ __forceinline__ void st4v(float* p, size_t i, float4 v) { *(float4*)(p + i) = v; }
__device__ __forceinline__ void st4v(bf16_t* p, size_t i, float4 v) {
    uint2 u;
    u.x = (uint32_t)f2bf(v.x) | ((uint32_t)f2bf(v.y) << 16);
    u.y = (uint32_t)f2bf(v.z) | ((uint32_t)f2bf(v.w) << 16);
    *(uint2*)(p + i) = u;
}
template <typename T, int VPT>
__global__ __launch_bounds__(NT) void add_rms_norm_vec_kernel(float* __restrict__ x, T* __restrict__ h, const T* __restrict__ a,
                                                              const T* __restrict__ b, const T* __restrict__ c,
                                                              const T* __restrict__ w, float eps, int D) {
    __shared__ float red[NT / 64 + 1];
    const size_t t = blockIdx.x;
    float4 v[VPT];
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
        const int i = (threadIdx.x + k * NT) * 4;
        if (i >= D) continue;
        v[k] = ld4v(x, t * D + i);
        if (a || b || c) {
            float4 y = make_float4(0.f, 0.f, 0.f, 0.f);
            if (b) y = ld4v(b, t * D + i);
            if (c) {
                const float4 z = ld4v(c, t * D + i);
                y.x += z.x; y.y += z.y; y.z += z.z; y.w += z.w;
            }
            if (a) {
                const float4 z = ld4v(a, t * D + i);
                y.x = z.x + y.x; y.y = z.y + y.y; y.z = z.z + y.z; y.w = z.w + y.w;
            }
            v[k].x += y.x; v[k].y += y.y; v[k].z += y.z; v[k].w += y.w;
            st4v(x, t * D + i, v[k]);
        }
        s += v[k].x * v[k].x + v[k].y * v[k].y + v[k].z * v[k].z + v[k].w * v[k].w;
    }
    if (!h) return;
    const float inv = 1.0f / sqrtf(block_sum<NT>(s, red) / (float)D + eps);
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
        const int i = (threadIdx.x + k * NT) * 4;
        if (i >= D) continue;
        const float4 g = ld4v(w, i);
        st4v(h, t * D + i, make_float4(v[k].x * inv * g.x, v[k].y * inv * g.y, v[k].z * inv * g.z, v[k].w * inv * g.w));
    }
}
extern "C" int qsv_add_rms_norm(float* x, void* h, const void* a, const void* b, const void* c, const void* w, float eps, int n,
                                int D, int dtype, void* stream) {
    QSV_REQUIRE(x && n >= 0 && D > 0 && (!h || w), "qsv_add_rms_norm: bad arguments");
    if (n == 0) return QSV_OK;
    const int vecs = (D / 4 + NT - 1) / NT;
    if (D % 4 == 0 && vecs <= 8) {
#define QSV_ARN(V)                                                                                                                 \
    QSV_DISPATCH(dtype, "qsv_add_rms_norm",                                                                                        \
                 hipLaunchKernelGGL((add_rms_norm_vec_kernel<T, V>), dim3(n), dim3(NT), 0, (hipStream_t)stream, x, (T*)h, (const T*)a, \
                                    (const T*)b, (const T*)c, (const T*)w, eps, D))
        if (vecs <= 1) QSV_ARN(1);
        else if (vecs <= 2) QSV_ARN(2);
        else if (vecs <= 4) QSV_ARN(4);
        else QSV_ARN(8);
#undef QSV_ARN
        return qsv_launch_status("qsv_add_rms_norm");
    }
    QSV_DISPATCH(dtype, "qsv_add_rms_norm",
                 hipLaunchKernelGGL(add_rms_norm_kernel<T>, dim3(n), dim3(NT), 0, (hipStream_t)stream, x, (T*)h, (const T*)a, (const T*)b,
                                    (const T*)c, (const T*)w, eps, D));
    return qsv_launch_status("qsv_add_rms_norm");
}

template <typename T>
__global__ __launch_bounds__(NT) void rms_norm_rows_kernel(T* __restrict__ out, const float* __restrict__ x,
                                                           const int32_t* __restrict__ rows, const T* __restrict__ w, float eps,
                                                           int D) {
    __shared__ float red[NT / 64 + 1];
    const size_t r = blockIdx.x;
    const float* xr = x + (size_t)(rows ? rows[r] : (int32_t)r) * D;
    float s = 0.f;
    for (int i = threadIdx.x; i < D; i += NT) s += xr[i] * xr[i];
    const float inv = 1.0f / sqrtf(block_sum<NT>(s, red) / (float)D + eps);
    for (int i = threadIdx.x; i < D; i += NT) st(out, r * D + i, xr[i] * inv * ld(w, i));
}
extern "C" int qsv_rms_norm_rows(void* out, const float* x, const int32_t* rows, const void* w, float eps, int n, int D, int dtype,
                                 void* stream) {
    QSV_REQUIRE(out && x && w && n >= 0 && D > 0, "qsv_rms_norm_rows: bad arguments");
    if (n == 0) return QSV_OK;
    QSV_DISPATCH(dtype, "qsv_rms_norm_rows",
                 hipLaunchKernelGGL(rms_norm_rows_kernel<T>, dim3(n), dim3(NT), 0, (hipStream_t)stream, (T*)out, x, rows, (const T*)w,
                                    eps, D));
    return qsv_launch_status("qsv_rms_norm_rows");
}

// ---- attention with queries and keys normed over all heads at once, and values blended with an earlier layer's ------------------
//   qf[t, h]          = [ 0 (vdim) | rms_norm(q[t])[h] * q_w[h] * scale ]       float [T, heads, vdim + dim]; the norm runs over all
//   pool[g, slot[t]]  = [ v'[t, g] | rms_norm(k[t])[g] * k_w[g] ]               heads * dim (kv_heads * dim) values of the projection
//   v' = (1 - mix) v + mix v_first  where v_first (row stride vf_stride, [kv_heads * vdim] per token) is given, else v.
template <typename T>
__global__ __launch_bounds__(NT) void normed_attention_prep_kernel(float* __restrict__ qf, T* __restrict__ pool, int64_t pool_rows,
                                                                   const T* __restrict__ proj, int64_t stride, int q_off, int k_off,
                                                                   int v_off, int H, int G, int dim, int vdim,
                                                                   const T* __restrict__ q_w, const T* __restrict__ k_w, float eps,
                                                                   float scale, const T* __restrict__ v_first, int64_t vf_stride,
                                                                   float mix, const int64_t* __restrict__ slot) {
    __shared__ float red[NT / 64 + 1];
    const size_t t = blockIdx.x;
    const int R = vdim + dim;
    const T* row = proj + t * stride;
    float s = 0.f;
    for (int i = threadIdx.x; i < H * dim; i += NT) {
        const float v = ld(row, q_off + i);
        s += v * v;
    }
    const float qinv = 1.0f / sqrtf(block_sum<NT>(s, red) / (float)(H * dim) + eps);
    s = 0.f;
    for (int i = threadIdx.x; i < G * dim; i += NT) {
        const float v = ld(row, k_off + i);
        s += v * v;
    }
    const float kinv = 1.0f / sqrtf(block_sum<NT>(s, red) / (float)(G * dim) + eps);
    for (int idx = threadIdx.x; idx < H * R; idx += NT) {
        const int h = idx / R, c = idx - h * R;
        const int e = h * dim + c - vdim;
        qf[t * H * (size_t)R + idx] = c < vdim ? 0.f : ld(row, q_off + e) * qinv * ld(q_w, e) * scale;
    }
    const size_t dst = (size_t)slot[t];
    for (int idx = threadIdx.x; idx < G * R; idx += NT) {
        const int g = idx / R, c = idx - g * R;
        float val;
        if (c < vdim) {
            val = ld(row, v_off + g * vdim + c);
            if (v_first) val = (1.0f - mix) * val + mix * ld(v_first, t * vf_stride + g * vdim + c);
        } else {
            const int e = g * dim + c - vdim;
            val = ld(row, k_off + e) * kinv * ld(k_w, e);
        }
        st(pool, ((size_t)g * pool_rows + dst) * R + c, val);
    }
}
extern "C" int qsv_normed_attention_prep(float* qf, void* pool, int64_t pool_rows, const void* proj, int64_t stride, int q_off,
                                         int k_off, int v_off, int heads, int kv_heads, int dim, int vdim, const void* q_w,
                                         const void* k_w, float eps, float scale, const void* v_first, int64_t vf_stride, float mix,
                                         const int64_t* slot, int n, int dtype, void* stream) {
    QSV_REQUIRE(qf && pool && proj && q_w && k_w && slot, "qsv_normed_attention_prep: null argument");
    QSV_REQUIRE(heads > 0 && kv_heads > 0 && dim > 0 && vdim > 0 && q_off >= 0 && k_off >= 0 && v_off >= 0 &&
                    q_off + (int64_t)heads * dim <= stride && k_off + (int64_t)kv_heads * dim <= stride &&
                    v_off + (int64_t)kv_heads * vdim <= stride && n >= 0 && (!v_first || vf_stride >= (int64_t)kv_heads * vdim),
                "qsv_normed_attention_prep: bad sizes");
    if (n == 0) return QSV_OK;
    QSV_DISPATCH(dtype, "qsv_normed_attention_prep",
                 hipLaunchKernelGGL(normed_attention_prep_kernel<T>, dim3(n), dim3(NT), 0, (hipStream_t)stream, qf, (T*)pool, pool_rows,
                                    (const T*)proj, stride, q_off, k_off, v_off, heads, kv_heads, dim, vdim, (const T*)q_w,
                                    (const T*)k_w, eps, scale, (const T*)v_first, vf_stride, mix, slot));
    return qsv_launch_status("qsv_normed_attention_prep");
}

// ---- sublayers between two norms: x += rms_norm(y) * w_post; h = rms_norm(x) * w_next ---------------------------------------------
// One workgroup per token, the row in registers (VPT groups of four values per thread; VPT = 0: any width, values re-read).  A
// weight is one gain (wide 0) or one per coordinate.
template <typename T>
__device__ __forceinline__ float4 gain4(const T* w, int wide, int i) {
    if (wide) return ld4v(w, i);
    const float g = ld(w, 0);
    return make_float4(g, g, g, g);
}
template <typename T, int VPT>
__global__ __launch_bounds__(NT) void add_normed_rms_norm_vec_kernel(float* __restrict__ x, T* __restrict__ h, const T* __restrict__ y,
                                                                     const T* __restrict__ w_post, int post_wide,
                                                                     const T* __restrict__ w_next, int next_wide, float eps, int D) {
    __shared__ float red[NT / 64 + 1];
    const size_t t = blockIdx.x;
    float4 v[VPT];
    float s = 0.f;
    if (y) {
        float4 u[VPT];
#pragma unroll
        for (int k = 0; k < VPT; ++k) {
            const int i = (threadIdx.x + k * NT) * 4;
            if (i >= D) continue;
            u[k] = ld4v(y, t * D + i);
            s += u[k].x * u[k].x + u[k].y * u[k].y + u[k].z * u[k].z + u[k].w * u[k].w;
        }
        const float inv = 1.0f / sqrtf(block_sum<NT>(s, red) / (float)D + eps);
        s = 0.f;
#pragma unroll
        for (int k = 0; k < VPT; ++k) {
            const int i = (threadIdx.x + k * NT) * 4;
            if (i >= D) continue;
            const float4 g = gain4(w_post, post_wide, i);
            v[k] = ld4v(x, t * D + i);
            v[k].x += u[k].x * inv * g.x; v[k].y += u[k].y * inv * g.y; v[k].z += u[k].z * inv * g.z; v[k].w += u[k].w * inv * g.w;
            st4v(x, t * D + i, v[k]);
            s += v[k].x * v[k].x + v[k].y * v[k].y + v[k].z * v[k].z + v[k].w * v[k].w;
        }
    } else {
#pragma unroll
        for (int k = 0; k < VPT; ++k) {
            const int i = (threadIdx.x + k * NT) * 4;
            if (i >= D) continue;
            v[k] = ld4v(x, t * D + i);
            s += v[k].x * v[k].x + v[k].y * v[k].y + v[k].z * v[k].z + v[k].w * v[k].w;
        }
    }
    if (!h) return;
    const float inv = 1.0f / sqrtf(block_sum<NT>(s, red) / (float)D + eps);
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
        const int i = (threadIdx.x + k * NT) * 4;
        if (i >= D) continue;
        const float4 g = gain4(w_next, next_wide, i);
        st4v(h, t * D + i, make_float4(v[k].x * inv * g.x, v[k].y * inv * g.y, v[k].z * inv * g.z, v[k].w * inv * g.w));
    }
}
template <typename T>
__global__ __launch_bounds__(NT) void add_normed_rms_norm_kernel(float* __restrict__ x, T* __restrict__ h, const T* __restrict__ y,
                                                                 const T* __restrict__ w_post, int post_wide,
                                                                 const T* __restrict__ w_next, int next_wide, float eps, int D) {
    __shared__ float red[NT / 64 + 1];
    const size_t t = blockIdx.x;
    float s = 0.f;
    if (y) {
        for (int i = threadIdx.x; i < D; i += NT) {
            const float u = ld(y, t * D + i);
            s += u * u;
        }
        const float inv = 1.0f / sqrtf(block_sum<NT>(s, red) / (float)D + eps);
        s = 0.f;
        for (int i = threadIdx.x; i < D; i += NT) {
            const float v = x[t * D + i] + ld(y, t * D + i) * inv * ld(w_post, post_wide ? i : 0);
            x[t * D + i] = v;
            s += v * v;
        }
    } else {
        for (int i = threadIdx.x; i < D; i += NT) s += x[t * D + i] * x[t * D + i];
    }
    if (!h) return;
    const float inv = 1.0f / sqrtf(block_sum<NT>(s, red) / (float)D + eps);
    for (int i = threadIdx.x; i < D; i += NT) st(h, t * D + i, x[t * D + i] * inv * ld(w_next, next_wide ? i : 0));
}
extern "C" int qsv_add_normed_rms_norm(float* x, void* h, const void* y, const void* w_post, int post_wide, const void* w_next,
                                       int next_wide, float eps, int n, int D, int dtype, void* stream) {
    QSV_REQUIRE(x && n >= 0 && D > 0 && (!h || w_next) && (!y || w_post), "qsv_add_normed_rms_norm: bad arguments");
    if (n == 0) return QSV_OK;
    const int vecs = (D / 4 + NT - 1) / NT;
    if (D % 4 == 0 && vecs <= 8) {
#define QSV_ANR(V)                                                                                                               \
    QSV_DISPATCH(dtype, "qsv_add_normed_rms_norm",                                                                               \
                 hipLaunchKernelGGL((add_normed_rms_norm_vec_kernel<T, V>), dim3(n), dim3(NT), 0, (hipStream_t)stream, x, (T*)h, \
                                    (const T*)y, (const T*)w_post, post_wide, (const T*)w_next, next_wide, eps, D))
        if (vecs <= 1) QSV_ANR(1);
        else if (vecs <= 2) QSV_ANR(2);
        else if (vecs <= 4) QSV_ANR(4);
        else QSV_ANR(8);
#undef QSV_ANR
        return qsv_launch_status("qsv_add_normed_rms_norm");
    }
    QSV_DISPATCH(dtype, "qsv_add_normed_rms_norm",
                 hipLaunchKernelGGL(add_normed_rms_norm_kernel<T>, dim3(n), dim3(NT), 0, (hipStream_t)stream, x, (T*)h, (const T*)y,
                                    (const T*)w_post, post_wide, (const T*)w_next, next_wide, eps, D));
    return qsv_launch_status("qsv_add_normed_rms_norm");
}

// ---- query / key norms (per head or over the projection), rotated pairs, cache write -----------------------------------------------
// One workgroup per token.  Statistics: per head a wave's sum over `dim`; over the projection a workgroup sum.  The rotation works
// on normed values staged in LDS (a pair's two values may sit in different threads).  Dynamic LDS: (heads + kv_heads) * dim floats.
template <typename T, typename TI>
__global__ __launch_bounds__(NT) void qk_norm_rope_prep_kernel(float* __restrict__ qf, const TI* __restrict__ q, int64_t q_stride,
                                                               const TI* __restrict__ k, int64_t k_stride, const TI* __restrict__ v,
                                                               int64_t v_stride, int H, int G, int dim, int vdim,
                                                               const T* __restrict__ q_w, const T* __restrict__ k_w, int per_head,
                                                               float eps, const float* __restrict__ rope, int rot_n, float scale,
                                                               T* __restrict__ pool, int64_t pool_rows,
                                                               const int64_t* __restrict__ slot, const int32_t* __restrict__ pos) {
    extern __shared__ float sm[];
    __shared__ float red[NT / 64 + 1];
    const size_t t = blockIdx.x;
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int NH = k ? H + G : H;                      // heads staged: the queries', then the keys'
    float* nq = sm;                                    // [NH][dim]
    const TI* qrow = q + t * q_stride;
    const TI* krow = k ? k + t * k_stride : nullptr;
    if (per_head) {
        for (int hh = wv; hh < NH; hh += NT / 64) {
            const TI* src = hh < H ? qrow + (size_t)hh * dim : krow + (size_t)(hh - H) * dim;
            const T* w = hh < H ? q_w : k_w;
            float s = 0.f;
            for (int e = lane; e < dim; e += 64) {
                const float u = ld(src, e);
                s += u * u;
            }
            const float inv = 1.0f / sqrtf(wave_sum(s) / (float)dim + eps);
            for (int e = lane; e < dim; e += 64) nq[hh * dim + e] = ld(src, e) * inv * ld(w, e);
        }
    } else {
        float s = 0.f;
        for (int i = threadIdx.x; i < H * dim; i += NT) {
            const float u = ld(qrow, i);
            s += u * u;
        }
        const float qinv = 1.0f / sqrtf(block_sum<NT>(s, red) / (float)(H * dim) + eps);
        for (int i = threadIdx.x; i < H * dim; i += NT) nq[i] = ld(qrow, i) * qinv * ld(q_w, i);
        if (k) {
            s = 0.f;
            for (int i = threadIdx.x; i < G * dim; i += NT) {
                const float u = ld(krow, i);
                s += u * u;
            }
            const float kinv = 1.0f / sqrtf(block_sum<NT>(s, red) / (float)(G * dim) + eps);
            for (int i = threadIdx.x; i < G * dim; i += NT) nq[H * dim + i] = ld(krow, i) * kinv * ld(k_w, i);
        }
    }
    __syncthreads();
    if (rope) {                                        // pairs of neighbours, each by one thread
        const int half = rot_n / 2;
        const float* cs = rope + (size_t)pos[t] * rot_n;
        for (int idx = threadIdx.x; idx < NH * half; idx += NT) {
            const int hh = idx / half, i = idx - hh * half;
            const float c = cs[i], sn = cs[half + i];
            const float a = nq[hh * dim + 2 * i], b = nq[hh * dim + 2 * i + 1];
            nq[hh * dim + 2 * i] = a * c - b * sn;
            nq[hh * dim + 2 * i + 1] = b * c + a * sn;
        }
        __syncthreads();
    }
    const int R = vdim + dim;
    for (int idx = threadIdx.x; idx < H * R; idx += NT) {
        const int h = idx / R, c = idx - h * R;
        qf[t * H * (size_t)R + idx] = c < vdim ? 0.f : nq[h * dim + c - vdim] * scale;
    }
    if (!k) return;
    const size_t dst = (size_t)slot[t];
    const TI* vrow = v + t * v_stride;
    for (int idx = threadIdx.x; idx < G * R; idx += NT) {
        const int g = idx / R, c = idx - g * R;
        st(pool, ((size_t)g * pool_rows + dst) * R + c, c < vdim ? ld(vrow, g * vdim + c) : nq[(H + g) * dim + c - vdim]);
    }
}
extern "C" int qsv_qk_norm_rope_prep(float* qf, const void* q, int64_t q_stride, const void* k, int64_t k_stride, const void* v,
                                     int64_t v_stride, int qkv_dtype, int heads, int kv_heads, int dim, int vdim, const void* q_w,
                                     const void* k_w, int per_head, float eps, const float* rope, int rot_n, float scale, void* pool,
                                     int64_t pool_rows, const int64_t* slot, const int32_t* pos, int n, int dtype, void* stream) {
    QSV_REQUIRE(qf && q && q_w && pos, "qsv_qk_norm_rope_prep: null argument");
    QSV_REQUIRE(!k || (v && k_w && pool && slot), "qsv_qk_norm_rope_prep: keys without values, weight, pool or rows");
    QSV_REQUIRE(heads > 0 && kv_heads > 0 && dim > 0 && vdim > 0 && n >= 0 && q_stride >= (int64_t)heads * dim &&
                    (!k || (k_stride >= (int64_t)kv_heads * dim && v_stride >= (int64_t)kv_heads * vdim)),
                "qsv_qk_norm_rope_prep: bad sizes");
    QSV_REQUIRE(!rope || (rot_n > 0 && rot_n % 2 == 0 && rot_n <= dim), "qsv_qk_norm_rope_prep: %d rotated dimensions of %d", rot_n, dim);
    QSV_REQUIRE(qkv_dtype == dtype || qkv_dtype == QSV_F32, "qsv_qk_norm_rope_prep: projections of type %d with storage type %d",
                qkv_dtype, dtype);
    const size_t lds = (size_t)(heads + kv_heads) * dim * 4;
    QSV_REQUIRE(lds <= 64 * 1024, "qsv_qk_norm_rope_prep: %d + %d heads of %d do not fit the workgroup's LDS", heads, kv_heads, dim);
    if (n == 0) return QSV_OK;
#define QSV_QKP(TI)                                                                                                              \
    QSV_DISPATCH(dtype, "qsv_qk_norm_rope_prep",                                                                                 \
                 hipLaunchKernelGGL((qk_norm_rope_prep_kernel<T, TI>), dim3(n), dim3(NT), lds, (hipStream_t)stream, qf, (const TI*)q, \
                                    q_stride, (const TI*)k, k_stride, (const TI*)v, v_stride, heads, kv_heads, dim, vdim,          \
                                    (const T*)q_w, (const T*)k_w, per_head, eps, rope, rot_n, scale, (T*)pool, pool_rows, slot, pos))
    if (qkv_dtype == QSV_F32) QSV_QKP(float);
    else QSV_QKP(bf16_t);
#undef QSV_QKP
    return qsv_launch_status("qsv_qk_norm_rope_prep");
}
