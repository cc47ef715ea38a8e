// serve_moe.hip -- mixture of experts: grouped top-k router and the per-token expert products (wave-per-output-row form).
//
// Router scores are float from the first product to the chosen weights.  The expert kernels keep one token's input in LDS
// and let every wave walk output rows with its lanes spread along the reduction (coalesced weight rows).
#include "serve_common.h"

namespace {
constexpr int NT = 256;
constexpr int NW = NT / 64;
constexpr int MAX_EXPERTS = 1024;

__device__ __forceinline__ void load8(const bf16_t* p, float (&v)[8]) {
    const uint4 u = *(const uint4*)p;
    const unsigned w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[2 * i] = __uint_as_float(w[i] << 16);
        v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
}
__device__ __forceinline__ void load8(const float* p, float (&v)[8]) {
    const float4 a = *(const float4*)p, b = *(const float4*)(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
// (value, index) of the largest value over a wave; ties go to the lower index.  Lanes without a candidate pass index -1.
__device__ __forceinline__ void wave_argmax(float& v, int& i) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(v, o, 64);
        const int oi = __shfl_xor(i, o, 64);
        if (oi >= 0 && (i < 0 || ov > v || (ov == v && oi < i))) {
            v = ov;
            i = oi;
        }
    }
}

// One workgroup per token.  z = router . h by the four waves (16-byte loads where the width allows), then wave 0 selects by
// repeated wave-wide argmax.  Scores s = softmax(z) over all experts (score_fn 0) or sigmoid(z) (1); the CHOICE goes by c = s +
// correction (correction may be NULL), the WEIGHTS are the chosen experts' s times `scale` (divided by their sum first if renorm).
// A group's score is its largest c (group_top 1) or the sum of its two largest (2); experts outside the `keep` best groups cannot
// be chosen, however low the others' c.  Ties go to the lower index, for groups and for experts.
template <typename T>
__global__ __launch_bounds__(NT) void moe_route_kernel(int32_t* __restrict__ idx, float* __restrict__ weight,
                                                       const T* __restrict__ h, const T* __restrict__ router,
                                                       const T* __restrict__ bias, int renorm, int D, int E, int top_k, int G,
                                                       int keep, int score_fn, const float* __restrict__ correction,
                                                       int group_top, float scale) {
    __shared__ float s[MAX_EXPERTS];
    __shared__ float c[MAX_EXPERTS];
    __shared__ float gs[MAX_EXPERTS];
    __shared__ unsigned char ok[MAX_EXPERTS];
    __shared__ unsigned char gtaken[MAX_EXPERTS];
    const size_t t = blockIdx.x;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const T* x = h + t * D;
    for (int e = w; e < E; e += NW) {
        const T* r = router + (size_t)e * D;
        float d = 0.f;
        if (D % 8 == 0) {
            for (int cc = lane * 8; cc < D; cc += 64 * 8) {
                float a[8], b[8];
                load8(r + cc, a);
                load8(x + cc, b);
#pragma unroll
                for (int q = 0; q < 8; ++q) d += a[q] * b[q];
            }
        } else {
            for (int i = lane; i < D; i += 64) d += ld(r, i) * ld(x, i);
        }
        d = wave_sum(d);
        if (lane == 0) s[e] = bias ? d + ld(bias, e) : d;
    }
    __syncthreads();
    // (the other three waves only keep the barriers company from here on: the selection is a few hundred steps of one wave)
    const bool sel = w == 0;
    if (sel) {
        if (score_fn == 0) {                                // softmax over all experts
            float mx = -INFINITY;
            for (int e = lane; e < E; e += 64) mx = fmaxf(mx, s[e]);
            mx = wave_max(mx);
            float sum = 0.f;
            for (int e = lane; e < E; e += 64) {
                const float p = expf(s[e] - mx);
                s[e] = p;
                sum += p;
            }
            const float inv = 1.0f / wave_sum(sum);
            for (int e = lane; e < E; e += 64) s[e] *= inv;
        } else {
            for (int e = lane; e < E; e += 64) s[e] = 1.0f / (1.0f + expf(-s[e]));
        }
        for (int e = lane; e < E; e += 64) {
            c[e] = correction ? s[e] + correction[e] : s[e];
            ok[e] = 0;
        }
    }
    __syncthreads();
    const int per = E / G;
    if (sel) {                                              // group scores
        for (int g = lane; g < G; g += 64) {
            float v1 = c[g * per], v2 = -INFINITY;          // the two largest
            for (int e = 1; e < per; ++e) {
                const float v = c[g * per + e];
                if (v > v1) {
                    v2 = v1;
                    v1 = v;
                } else if (v > v2) {
                    v2 = v;
                }
            }
            gs[g] = (group_top == 2 && per > 1) ? v1 + v2 : v1;
            gtaken[g] = 0;
        }
    }
    __syncthreads();
    for (int k = 0; k < keep; ++k) {                        // the `keep` best groups
        if (sel) {
            float bv = 0.f;
            int bi = -1;
            for (int g = lane; g < G; g += 64)
                if (!gtaken[g] && (bi < 0 || gs[g] > bv)) {
                    bv = gs[g];
                    bi = g;
                }
            wave_argmax(bv, bi);
            if (lane == 0) gtaken[bi] = 1;
            for (int e = lane; e < per; e += 64) ok[bi * per + e] = 1;
        }
        __syncthreads();
    }
    float chosen = 0.f;                                     // (lane 0 of the selecting wave: sum of the chosen scores)
    for (int k = 0; k < top_k; ++k) {                       // the top_k eligible experts
        if (sel) {
            float bv = 0.f;
            int bi = -1;
            for (int e = lane; e < E; e += 64)
                if (ok[e] && (bi < 0 || c[e] > bv)) {
                    bv = c[e];
                    bi = e;
                }
            wave_argmax(bv, bi);
            if (lane == 0) {
                ok[bi] = 0;
                idx[t * top_k + k] = bi;
                weight[t * top_k + k] = s[bi];
                chosen += s[bi];
            }
        }
        __syncthreads();
    }
    // weights over the chosen only: p_i / sum of the chosen p = the softmax over the chosen logits
    if (sel && lane == 0 && (renorm || scale != 1.0f))
        for (int k = 0; k < top_k; ++k) {
            float v = weight[t * top_k + k];
            if (renorm) v /= chosen;
            weight[t * top_k + k] = v * scale;
        }
}

// Activation of the first expert product.  ACT_GLU: the weight rows come in pairs (2f = gate, 2f + 1 = up) and output f is
// silu(gate) * up, so the output is half as wide as the product.
constexpr int ACT_NONE = 0, ACT_RELU_SQ = 1, ACT_GLU = 2;
// (QSV_ACT_CLAMPED_GLU runs the ACT_GLU kernels with limit > 0: g = min(gate, limit), u = clamp(up, -limit, limit), g sigmoid(1.702 g) (u + 1))
__device__ __forceinline__ float relu_sq(float d) {
    const float a = fmaxf(d, 0.f);
    return a * a;
}
__device__ __forceinline__ float glu(float g, float u, float limit) {
    if (limit > 0.f) {                                       // (uniform over the launch)
        g = fminf(g, limit);
        u = fminf(fmaxf(u, -limit), limit);
        return g / (1.0f + expf(-1.702f * g)) * (u + 1.0f);
    }
    return g / (1.0f + expf(-g)) * u;
}

// One workgroup per (token, chosen expert): act = relu(up_e . h)^2 (or the gated unit).  Dynamic LDS: D floats.  ff: weight rows.
template <typename T, int ACT>
__global__ __launch_bounds__(NT) void moe_up_kernel(T* __restrict__ act, const T* __restrict__ h, const T* __restrict__ up,
                                                    const int32_t* __restrict__ idx, int top_k, int D, int ff, float limit, int n_experts) {
    extern __shared__ float xs[];
    const size_t slot = blockIdx.x;
    if (idx[slot] >= n_experts) return;                      // an identity expert: the down kernel adds the input itself
    const size_t t = slot / top_k;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    for (int i = threadIdx.x; i < D; i += NT) xs[i] = ld(h, t * D + i);
    __syncthreads();
    const T* W = up + (size_t)idx[slot] * ff * D;
    if (ACT == ACT_GLU) {
        for (int f = w; f < ff / 2; f += NW) {
            const T* r = W + (size_t)(2 * f) * D;
            float d = 0.f, e = 0.f;
            for (int i = lane; i < D; i += 64) {
                d += ld(r, i) * xs[i];
                e += ld(r, D + i) * xs[i];
            }
            d = wave_sum(d);
            e = wave_sum(e);
            if (lane == 0) st(act, slot * (ff / 2) + f, glu(d, e, limit));
        }
        return;
    }
    for (int f = w; f < ff; f += NW) {
        const T* r = W + (size_t)f * D;
        float d = 0.f;
        for (int i = lane; i < D; i += 64) d += ld(r, i) * xs[i];
        d = wave_sum(d);
        if (lane == 0) st(act, slot * ff + f, relu_sq(d));
    }
}

// One workgroup per token: y = sum_k weight_k * down_{e_k} . act_k.  Dynamic LDS: top_k * ff floats.
template <typename T>
__global__ __launch_bounds__(NT) void moe_down_kernel(T* __restrict__ y, const T* __restrict__ act, const T* __restrict__ down,
                                                      const int32_t* __restrict__ idx, const float* __restrict__ weight,
                                                      int top_k, int D, int ff, const T* __restrict__ h, int n_experts) {
    extern __shared__ float as[];
    const size_t t = blockIdx.x;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    for (int i = threadIdx.x; i < top_k * ff; i += NT) as[i] = ld(act, t * top_k * ff + i);
    __syncthreads();
    for (int d = w; d < D; d += NW) {
        float total = 0.f;
        for (int k = 0; k < top_k; ++k) {
            if (idx[t * top_k + k] >= n_experts) {           // identity expert
                total += weight[t * top_k + k] * ld(h, t * D + d);
                continue;
            }
            const T* r = down + ((size_t)idx[t * top_k + k] * D + d) * ff;
            float v = 0.f;
            for (int i = lane; i < ff; i += 64) v += ld(r, i) * as[k * ff + i];
            total += weight[t * top_k + k] * wave_sum(v);
        }
        if (lane == 0) st(y, t * D + d, total);
    }
}

// The same two kernels for widths that are multiples of 8: 16-byte weight loads and four output rows per wave in flight at once
// (the scalar forms above wait for one row's loads before they issue the next row's: latency-bound at real layer sizes).
constexpr int ROWS = 4;      // output rows a wave works on at once

template <typename T, int ACT>
__global__ __launch_bounds__(NT) void moe_up_vec_kernel(T* __restrict__ act, const T* __restrict__ h, const T* __restrict__ up,
                                                        const int32_t* __restrict__ idx, int top_k, int D, int ff, float limit, int n_experts) {
    extern __shared__ float xs[];
    const size_t slot = blockIdx.x;
    if (idx[slot] >= n_experts) return;                      // an identity expert: the down kernel adds the input itself
    const size_t t = slot / top_k;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    for (int i = threadIdx.x; i < D; i += NT) xs[i] = ld(h, t * D + i);
    __syncthreads();
    const T* W = up + (size_t)idx[slot] * ff * D;
    for (int f0 = w * ROWS; f0 < ff; f0 += NW * ROWS) {
        float acc[ROWS] = {0.f, 0.f, 0.f, 0.f};
        for (int c = lane * 8; c < D; c += 64 * 8) {
            float x[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) x[e] = xs[c + e];
#pragma unroll
            for (int r = 0; r < ROWS; ++r) {
                if (f0 + r < ff) {
                    float v[8];
                    load8(W + (size_t)(f0 + r) * D + c, v);
#pragma unroll
                    for (int e = 0; e < 8; ++e) acc[r] += v[e] * x[e];
                }
            }
        }
        float d[ROWS];
#pragma unroll
        for (int r = 0; r < ROWS; ++r) d[r] = wave_sum(acc[r]);
        if (lane == 0) {
            if (ACT == ACT_GLU) {                               // (ROWS and ff are even: a pair never straddles two waves)
#pragma unroll
                for (int r = 0; r < ROWS; r += 2)
                    if (f0 + r < ff) st(act, slot * (ff / 2) + (f0 + r) / 2, glu(d[r], d[r + 1], limit));
            } else {
#pragma unroll
                for (int r = 0; r < ROWS; ++r)
                    if (f0 + r < ff) st(act, slot * ff + f0 + r, relu_sq(d[r]));
            }
        }
    }
}

template <typename T>
__global__ __launch_bounds__(NT) void moe_down_vec_kernel(T* __restrict__ y, const T* __restrict__ act, const T* __restrict__ down,
                                                          const int32_t* __restrict__ idx, const float* __restrict__ weight,
                                                          int top_k, int D, int ff, const T* __restrict__ h, int n_experts) {
    extern __shared__ float as[];
    const size_t t = blockIdx.x;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    for (int i = threadIdx.x; i < top_k * ff; i += NT) as[i] = ld(act, t * top_k * ff + i);
    __syncthreads();
    for (int d0 = w * ROWS; d0 < D; d0 += NW * ROWS) {
        float acc[ROWS] = {0.f, 0.f, 0.f, 0.f};
        for (int k = 0; k < top_k; ++k) {
            const float wk = weight[t * top_k + k];
            if (idx[t * top_k + k] >= n_experts) {           // identity expert: lane 0's share carries the input (the rest add zero)
                if (lane == 0) {
#pragma unroll
                    for (int r = 0; r < ROWS; ++r)
                        if (d0 + r < D) acc[r] += wk * ld(h, t * D + d0 + r);
                }
                continue;
            }
            const T* Wk = down + (size_t)idx[t * top_k + k] * D * ff;
            float part[ROWS] = {0.f, 0.f, 0.f, 0.f};
            for (int c = lane * 8; c < ff; c += 64 * 8) {
                float x[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) x[e] = as[k * ff + c + e];
#pragma unroll
                for (int r = 0; r < ROWS; ++r) {
                    if (d0 + r < D) {
                        float v[8];
                        load8(Wk + (size_t)(d0 + r) * ff + c, v);
#pragma unroll
                        for (int e = 0; e < 8; ++e) part[r] += v[e] * x[e];
                    }
                }
            }
#pragma unroll
            for (int r = 0; r < ROWS; ++r) acc[r] += wk * part[r];
        }
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            const float v = wave_sum(acc[r]);
            if (lane == 0 && d0 + r < D) st(y, t * D + d0 + r, v);
        }
    }
}

// ---- expert-major form (decoding and short portions, bfloat16): slots sorted by expert ON THE DEVICE, workgroup = (16 output rows,
// expert); a wave keeps its four weight rows in registers (packed bfloat16) and walks the tokens routed to the expert, so every
// weight is read once per step however many tokens share the expert.  No host synchronisation. ----------------------------------
typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
template <int KI, int ACT>
__global__ __launch_bounds__(NT) void expert_rows_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ X,
                                                         const int64_t* __restrict__ x_index, int div, const bf16_t* __restrict__ W,
                                                         const int64_t* __restrict__ offsets, int rows, int K, float limit) {
    const int e = blockIdx.y;
    const int64_t s0 = offsets[e], s1 = offsets[e + 1];
    if (s0 == s1) return;                                                   // nobody chose this expert
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int r0 = (blockIdx.x * NW + w) * ROWS;
    if (r0 >= rows) return;
    uint4 wr[ROWS][KI];
#pragma unroll
    for (int r = 0; r < ROWS; ++r)
#pragma unroll
        for (int i = 0; i < KI; ++i) {
            const int c = (lane + 64 * i) * 8;
            wr[r][i] = (r0 + r < rows && c < K) ? *(const uint4*)(W + ((size_t)e * rows + r0 + r) * K + c) : make_uint4(0u, 0u, 0u, 0u);
        }
    // TOK tokens at a time: their input pieces are all requested before the first is used (a token at a time, every token
    // paid a full memory round trip with nothing else in flight)
    constexpr int TOK = 4;
    for (int64_t sb = s0; sb < s1; sb += TOK) {
        uint4 xr[TOK][KI];
#pragma unroll
        for (int j = 0; j < TOK; ++j) {
            const int64_t s = sb + j < s1 ? sb + j : s1 - 1;
            const bf16_t* x = X + (size_t)(x_index ? x_index[s] / div : s) * K;
#pragma unroll
            for (int i = 0; i < KI; ++i) {
                const int c = (lane + 64 * i) * 8;
                xr[j][i] = c < K ? *(const uint4*)(x + c) : make_uint4(0u, 0u, 0u, 0u);
            }
        }
#pragma unroll
        for (int j = 0; j < TOK; ++j) {
            float acc[ROWS] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int i = 0; i < KI; ++i) {
                const unsigned xu[4] = {xr[j][i].x, xr[j][i].y, xr[j][i].z, xr[j][i].w};
#pragma unroll
                for (int r = 0; r < ROWS; ++r) {
                    const unsigned u[4] = {wr[r][i].x, wr[r][i].y, wr[r][i].z, wr[r][i].w};
#pragma unroll
                    for (int q = 0; q < 4; ++q)                           // v_dot2_f32_bf16: two products per instruction, no unpacking
                        acc[r] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf2, u[q]), __builtin_bit_cast(bf2, xu[q]), acc[r], false);
                }
            }
            if (sb + j < s1) {                                              // (wave-uniform)
                float d[ROWS];
#pragma unroll
                for (int r = 0; r < ROWS; ++r) d[r] = wave_sum(acc[r]);
                if (lane == 0) {
                    if (ACT == ACT_GLU) {
#pragma unroll
                        for (int r = 0; r < ROWS; r += 2)
                            if (r0 + r < rows) out[(size_t)(sb + j) * (rows / 2) + (r0 + r) / 2] = f2bf(glu(d[r], d[r + 1], limit));
                    } else {
#pragma unroll
                        for (int r = 0; r < ROWS; ++r)
                            if (r0 + r < rows) out[(size_t)(sb + j) * rows + r0 + r] = f2bf(ACT == ACT_RELU_SQ ? relu_sq(d[r]) : d[r]);
                    }
                }
            }
        }
    }
}

// ---- expert-sorted form (many tokens): the products are the vendor's, per expert over contiguous runs of sorted slots; these
// kernels do the permutation in, the activation, and the weighted permutation out -----------------------------------------------
template <typename T>
__global__ __launch_bounds__(NT) void gather_rows_kernel(T* __restrict__ out, const T* __restrict__ src,
                                                         const int64_t* __restrict__ order, int div, int width) {
    const size_t i = blockIdx.x;
    const T* s = src + (size_t)(order[i] / div) * width;
    for (int c = threadIdx.x; c < width; c += NT) out[i * width + c] = s[c];
}
template <typename T>
__global__ __launch_bounds__(NT) void relu_sq_kernel(T* __restrict__ a, size_t n) {
    const size_t i = (size_t)blockIdx.x * NT + threadIdx.x;
    if (i < n) {
        const float v = fmaxf(ld(a, i), 0.f);
        st(a, i, v * v);
    }
}
// y[t] = sum_k weight[t, k] * ys[inv[t top_k + k]]
template <typename T>
__global__ __launch_bounds__(NT) void moe_combine_kernel(T* __restrict__ y, const T* __restrict__ ys, const int64_t* __restrict__ inv,
                                                         const float* __restrict__ weight, int top_k, int D,
                                                         const int32_t* __restrict__ idx, const T* __restrict__ h, int n_experts) {
    const size_t t = blockIdx.x;
    for (int c = threadIdx.x; c < D; c += NT) {
        float a = 0.f;
        for (int k = 0; k < top_k; ++k) {
            const bool same = idx && idx[t * top_k + k] >= n_experts;       // an identity expert's slot has no sorted row
            a += weight[t * top_k + k] * (same ? ld(h, t * D + c) : ld(ys, (size_t)inv[t * top_k + k] * D + c));
        }
        st(y, t * D + c, a);
    }
}
}  // namespace

extern "C" int qsv_gather_rows(void* out, const void* src, const int64_t* order, int div, int n_rows, int width, int dtype,
                               void* stream) {
    QSV_REQUIRE(out && src && order && div > 0 && n_rows >= 0 && width > 0, "qsv_gather_rows: bad arguments");
    if (n_rows == 0) return QSV_OK;
    QSV_DISPATCH(dtype, "qsv_gather_rows",
                 hipLaunchKernelGGL(gather_rows_kernel<T>, dim3(n_rows), dim3(NT), 0, (hipStream_t)stream, (T*)out, (const T*)src,
                                    order, div, width));
    return qsv_launch_status("qsv_gather_rows");
}
// out[s, r] = act(W[e][r, :] . X[x_index ? x_index[s] / div : s, :]) for the sorted slots s in [offsets[e], offsets[e + 1]) of every
// expert e; W [E, rows, K] bfloat16, act: 0 nothing, 1 relu^2, 2 gated unit (row pairs; out is rows / 2 wide).  K % 8 == 0, K <= 4096.
extern "C" int qsv_expert_rows(void* out, const void* X, const int64_t* x_index, int div, const void* W, const int64_t* offsets,
                               int n_experts, int rows, int K, int act, float limit, void* stream) {
    QSV_REQUIRE(out && X && W && offsets && n_experts > 0 && rows > 0 && div > 0, "qsv_expert_rows: bad arguments");
    QSV_REQUIRE(act == ACT_NONE || act == ACT_RELU_SQ || ((act == ACT_GLU || act == QSV_ACT_CLAMPED_GLU) && rows % 2 == 0),
                "qsv_expert_rows: activation %d", act);
    QSV_REQUIRE(act != QSV_ACT_CLAMPED_GLU || limit > 0.f, "qsv_expert_rows: clamped units need a positive limit");
    if (act == QSV_ACT_CLAMPED_GLU) act = ACT_GLU;
    else limit = 0.f;
    QSV_REQUIRE(K > 0 && K % 8 == 0 && K <= 4096, "qsv_expert_rows: inner width %d (a multiple of 8, at most 4096)", K);
    QSV_REQUIRE(n_experts <= 65535, "qsv_expert_rows: too many experts");
    const dim3 grid((rows + NW * ROWS - 1) / (NW * ROWS), n_experts), block(NT);
#define QSV_ER(KI)                                                                                                           \
    do {                                                                                                                     \
        if (act == ACT_RELU_SQ)                                                                                              \
            hipLaunchKernelGGL((expert_rows_kernel<KI, ACT_RELU_SQ>), grid, block, 0, (hipStream_t)stream, (bf16_t*)out,         \
                               (const bf16_t*)X, x_index, div, (const bf16_t*)W, offsets, rows, K, limit);                          \
        else if (act == ACT_GLU)                                                                                             \
            hipLaunchKernelGGL((expert_rows_kernel<KI, ACT_GLU>), grid, block, 0, (hipStream_t)stream, (bf16_t*)out,             \
                               (const bf16_t*)X, x_index, div, (const bf16_t*)W, offsets, rows, K, limit);                          \
        else                                                                                                                 \
            hipLaunchKernelGGL((expert_rows_kernel<KI, ACT_NONE>), grid, block, 0, (hipStream_t)stream, (bf16_t*)out,            \
                               (const bf16_t*)X, x_index, div, (const bf16_t*)W, offsets, rows, K, limit);                          \
    } while (0)
    if (K <= 512) QSV_ER(1);
    else if (K <= 1024) QSV_ER(2);
    else if (K <= 2048) QSV_ER(4);
    else QSV_ER(8);
#undef QSV_ER
    return qsv_launch_status("qsv_expert_rows");
}
extern "C" int qsv_relu_sq(void* a, int64_t n, int dtype, void* stream) {
    QSV_REQUIRE(a && n >= 0 && n < (1ll << 31) * NT, "qsv_relu_sq: bad arguments");
    if (n == 0) return QSV_OK;
    QSV_DISPATCH(dtype, "qsv_relu_sq",
                 hipLaunchKernelGGL(relu_sq_kernel<T>, dim3((unsigned)((n + NT - 1) / NT)), dim3(NT), 0, (hipStream_t)stream, (T*)a,
                                    (size_t)n));
    return qsv_launch_status("qsv_relu_sq");
}
extern "C" int qsv_moe_combine(void* y, const void* ys, const int64_t* inv, const float* weight, int n, int top_k, int D,
                               const int32_t* idx, const void* h, int n_experts, int dtype, void* stream) {
    QSV_REQUIRE(y && ys && inv && weight && n >= 0 && top_k > 0 && D > 0 && (!idx || h), "qsv_moe_combine: bad arguments");
    if (n == 0) return QSV_OK;
    QSV_DISPATCH(dtype, "qsv_moe_combine",
                 hipLaunchKernelGGL(moe_combine_kernel<T>, dim3(n), dim3(NT), 0, (hipStream_t)stream, (T*)y, (const T*)ys, inv,
                                    weight, top_k, D, idx, (const T*)h, n_experts));
    return qsv_launch_status("qsv_moe_combine");
}

extern "C" int qsv_moe_route(int32_t* idx, float* weight, const void* h, const void* router, const void* bias, int renorm, int n,
                             int D, int E, int top_k, int G, int keep, int score_fn, const float* correction, int group_top,
                             float scale, int dtype, void* stream) {
    QSV_REQUIRE((score_fn == 0 || score_fn == 1) && (group_top == 1 || group_top == 2), "qsv_moe_route: score function %d, group score %d",
                score_fn, group_top);
    QSV_REQUIRE(idx && weight && h && router && n >= 0 && D > 0, "qsv_moe_route: bad arguments");
    QSV_REQUIRE(E > 0 && E <= MAX_EXPERTS && G > 0 && E % G == 0 && keep > 0 && keep <= G && top_k > 0 &&
                    top_k <= keep * (E / G),
                "qsv_moe_route: %d experts in %d groups, %d groups kept, top %d", E, G, keep, top_k);
    if (n == 0) return QSV_OK;
    QSV_DISPATCH(dtype, "qsv_moe_route",
                 hipLaunchKernelGGL(moe_route_kernel<T>, dim3(n), dim3(NT), 0, (hipStream_t)stream, idx, weight, (const T*)h,
                                    (const T*)router, (const T*)bias, renorm, D, E, top_k, G, keep, score_fn, correction,
                                    group_top, scale));
    return qsv_launch_status("qsv_moe_route");
}

extern "C" int qsv_moe_up(void* act, const void* h, const void* up, const int32_t* idx, int n, int top_k, int D, int ff,
                          int activation, float limit, int n_experts, int dtype, void* stream) {
    QSV_REQUIRE(act && h && up && idx && n >= 0 && top_k > 0 && D > 0 && ff > 0 && n_experts > 0, "qsv_moe_up: bad arguments");
    QSV_REQUIRE(activation == ACT_RELU_SQ || ((activation == ACT_GLU || activation == QSV_ACT_CLAMPED_GLU) && ff % 2 == 0),
                "qsv_moe_up: activation %d over %d rows", activation, ff);
    QSV_REQUIRE(activation != QSV_ACT_CLAMPED_GLU || limit > 0.f, "qsv_moe_up: clamped units need a positive limit");
    if (activation == QSV_ACT_CLAMPED_GLU) activation = ACT_GLU;
    else limit = 0.f;
    QSV_REQUIRE((size_t)D * 4 <= 64 * 1024, "qsv_moe_up: width %d does not fit the workgroup's LDS", D);
    if (n == 0) return QSV_OK;
#define QSV_UP(KERNEL, ACT)                                                                                                  \
    QSV_DISPATCH(dtype, "qsv_moe_up",                                                                                        \
                 hipLaunchKernelGGL((KERNEL<T, ACT>), dim3(n * top_k), dim3(NT), (size_t)D * 4, (hipStream_t)stream, (T*)act,   \
                                    (const T*)h, (const T*)up, idx, top_k, D, ff, limit, n_experts))
    if (D % 8 == 0) {
        if (activation == ACT_GLU) QSV_UP(moe_up_vec_kernel, ACT_GLU);
        else QSV_UP(moe_up_vec_kernel, ACT_RELU_SQ);
    } else {
        if (activation == ACT_GLU) QSV_UP(moe_up_kernel, ACT_GLU);
        else QSV_UP(moe_up_kernel, ACT_RELU_SQ);
    }
#undef QSV_UP
    return qsv_launch_status("qsv_moe_up");
}

extern "C" int qsv_moe_down(void* y, const void* act, const void* down, const int32_t* idx, const float* weight, int n,
                            int top_k, int D, int ff, const void* h, int n_experts, int dtype, void* stream) {
    QSV_REQUIRE(y && act && down && idx && weight && h && n >= 0 && top_k > 0 && D > 0 && ff > 0 && n_experts > 0,
                "qsv_moe_down: bad arguments");
    QSV_REQUIRE((size_t)top_k * ff * 4 <= 64 * 1024, "qsv_moe_down: %d x %d activations do not fit the workgroup's LDS", top_k, ff);
    if (n == 0) return QSV_OK;
    if (ff % 8 == 0)
        QSV_DISPATCH(dtype, "qsv_moe_down",
                     hipLaunchKernelGGL(moe_down_vec_kernel<T>, dim3(n), dim3(NT), (size_t)top_k * ff * 4, (hipStream_t)stream, (T*)y,
                                        (const T*)act, (const T*)down, idx, weight, top_k, D, ff, (const T*)h, n_experts));
    else
        QSV_DISPATCH(dtype, "qsv_moe_down",
                     hipLaunchKernelGGL(moe_down_kernel<T>, dim3(n), dim3(NT), (size_t)top_k * ff * 4, (hipStream_t)stream, (T*)y,
                                        (const T*)act, (const T*)down, idx, weight, top_k, D, ff, (const T*)h, n_experts));
    return qsv_launch_status("qsv_moe_down");
}
