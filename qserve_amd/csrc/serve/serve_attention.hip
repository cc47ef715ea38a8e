// serve_attention.hip -- softmax attention over a paged cache of latent rows (one row per token, shared by all heads).
//
// The query arrives already carried into the latent space (qsv_latent_query), so a score is one dot product of the query
// with a cache row and the output is the softmax-weighted sum of the rows' first `rank` elements.  One launch serves
// prompt portions and single decoded tokens alike: every token brings its own sequence, position and window start.
//
// Wave kernel: workgroup = one (token, head), four waves; wave w takes keys lo + KG (w + 4 n) ... in groups of KG, lanes
// spread over the row's elements (coalesced row reads), one butterfly reduction per score, online softmax per group, the
// four partial results merged through LDS.  Scores, weights and sums are float.
//
// Keys behind the window come first in a query's key list: the sequence's first `keep_first` positions that have left the window,
// or one pooled row per block of `pool_block` positions that ended before the window (from a second pool with `block_rows` rows per
// page).  A sink starts wave 0's softmax state at (maximum = sink, sum = 1): one more term of the denominator, without a value.
#include "serve_common.h"

namespace {
constexpr int NW = 4;    // waves per workgroup
constexpr int KG = 4;    // keys per softmax update

template <typename T, int EPL>
__global__ __launch_bounds__(64 * NW) void latent_attention_wave_kernel(
    T* __restrict__ out, const float* __restrict__ qf, const T* pool, const int32_t* __restrict__ block_table,
    int table_stride, const int32_t* __restrict__ seq, const int32_t* __restrict__ pos, int window, int H, int rank, int R,
    int page, int per, int64_t pool_stride, int chunk, const float* __restrict__ bias, int bias_len, int keep_first,
    const float* __restrict__ sink, const T* pooled, int64_t pooled_stride, int pool_block, int block_rows) {
    __shared__ float s_m[NW], s_l[NW];
    __shared__ float s_acc[NW][64 * EPL];
    const size_t t = blockIdx.x / H;
    const int h = blockIdx.x % H;
    pool += (size_t)(h / per) * (size_t)pool_stride;             // heads [g per, (g + 1) per) read pool g
    if (pooled) pooled += (size_t)(h / per) * (size_t)pooled_stride;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int p = pos[t];
    int lo = window > 0 ? max(0, p - window + 1) : 0;
    if (chunk > 0) lo = max(lo, p - p % chunk);                  // chunks are counted from position 0 of the sequence
    const float* brow = bias ? bias + (size_t)h * bias_len : nullptr;
    const int32_t* bt = block_table + (size_t)seq[t] * table_stride;
    const float* qrow = qf + (t * H + h) * (size_t)R;
    float q[EPL], acc[EPL];
#pragma unroll
    for (int i = 0; i < EPL; ++i) {
        const int e = lane + 64 * i;
        q[i] = e < R ? qrow[e] : 0.f;
        acc[i] = 0.f;
    }
    float m = -INFINITY, l = 0.f;
    if (sink && w == 0) {
        m = sink[h];
        l = 1.f;
    }
    // the query's keys: n_pre keys behind the window (kept first positions, or pooled blocks), then the positions lo .. p
    const int n_pre = pooled ? max(0, p - window + 1) / pool_block : min(keep_first, lo);
    const int n_keys = n_pre + p - lo + 1;
    for (int j0 = w * KG; j0 < n_keys; j0 += NW * KG) {
        float c[KG][EPL], s[KG];
#pragma unroll
        for (int k = 0; k < KG; ++k) {
            const int j = j0 + k;
            const bool ok = j < n_keys;
            const int vk = ok ? j : n_keys - 1;
            const int jj = vk < n_pre ? vk : lo + vk - n_pre;       // a position, or (with pooled rows, vk < n_pre) a block
            const T* row;
            if (pooled && vk < n_pre) {
                const int first = vk * pool_block;                    // the block's first position names its page and row
                row = pooled + ((size_t)bt[first / page] * block_rows + (size_t)((first % page) / pool_block)) * (size_t)R;
            } else {
                row = pool + ((size_t)bt[jj / page] * page + (size_t)(jj % page)) * (size_t)R;
            }
            float d = 0.f;
#pragma unroll
            for (int i = 0; i < EPL; ++i) {
                const int e = lane + 64 * i;
                c[k][i] = e < R ? ld(row, e) : 0.f;
                d += q[i] * c[k][i];
            }
            d = wave_sum(d);
            if (brow) d += brow[min(p - jj, bias_len - 1)];
            s[k] = ok ? d : -INFINITY;
        }
        float mx = m;
#pragma unroll
        for (int k = 0; k < KG; ++k) mx = fmaxf(mx, s[k]);
        const float alpha = expf(m - mx);          // first group: exp(-inf) = 0 (mx is finite: key j0 is visible)
        float pk[KG], ps = 0.f;
#pragma unroll
        for (int k = 0; k < KG; ++k) {
            pk[k] = expf(s[k] - mx);
            ps += pk[k];
        }
        l = l * alpha + ps;
        m = mx;
#pragma unroll
        for (int i = 0; i < EPL; ++i) {
            float a = acc[i] * alpha;
#pragma unroll
            for (int k = 0; k < KG; ++k) a += pk[k] * c[k][i];
            acc[i] = a;
        }
    }
    if (lane == 0) {
        s_m[w] = m;
        s_l[w] = l;
    }
#pragma unroll
    for (int i = 0; i < EPL; ++i) s_acc[w][lane + 64 * i] = acc[i];
    __syncthreads();
    float M = s_m[0];
#pragma unroll
    for (int k = 1; k < NW; ++k) M = fmaxf(M, s_m[k]);
    float f[NW], L = 0.f;
#pragma unroll
    for (int k = 0; k < NW; ++k) {
        f[k] = expf(s_m[k] - M);                   // a wave without keys has m = -inf: factor 0
        L += f[k] * s_l[k];
    }
    const float invL = 1.0f / L;
    T* o = out + (t * H + h) * (size_t)rank;
    for (int e = threadIdx.x; e < rank; e += 64 * NW) {
        float a = 0.f;
#pragma unroll
        for (int k = 0; k < NW; ++k) a += f[k] * s_acc[k][e];
        st(o, e, a * invL);
    }
}

template <typename T>
int launch_wave(void* out, const float* qf, const void* pool, const int32_t* bt, int ts, const int32_t* seq, const int32_t* pos,
                int window, int n, int H, int rank, int R, int page, int per, int64_t pool_stride, int chunk, const float* bias,
                int bias_len, int keep_first, const float* sink, const void* pooled, int64_t pooled_stride, int pool_block,
                int block_rows, hipStream_t st_) {
    const dim3 grid(n * H), block(64 * NW);
#define QSV_ATT(E)                                                                                                        \
    hipLaunchKernelGGL((latent_attention_wave_kernel<T, E>), grid, block, 0, st_, (T*)out, qf, (const T*)pool, bt, ts, seq, pos, \
                       window, H, rank, R, page, per, pool_stride, chunk, bias, bias_len, keep_first, sink, (const T*)pooled,        \
                       pooled_stride, pool_block, block_rows)
    if (R <= 64) QSV_ATT(1);
    else if (R <= 128) QSV_ATT(2);
    else if (R <= 192) QSV_ATT(3);
    else if (R <= 256) QSV_ATT(4);
    else if (R <= 384) QSV_ATT(6);
    else if (R <= 576) QSV_ATT(9);
    else if (R <= 1024) QSV_ATT(16);
    else {
        qsv_set_error("qsv_latent_attention: cache rows of %d elements (at most 1024)", R);
        return QSV_EINVAL;
    }
#undef QSV_ATT
    return QSV_OK;
}
}  // namespace

extern "C" int qsv_latent_attention(void* out, const float* qf, const void* pool, const int32_t* block_table, int table_stride,
                                    const int32_t* seq, const int32_t* pos, int window, int n, int H, int rank, int R, int page,
                                    int heads_per_pool, int64_t pool_stride, int chunk, const float* bias, int bias_len,
                                    int keep_first, const float* sink, const void* pooled, int64_t pooled_stride, int pool_block,
                                    int block_rows, int dtype, int variant, void* stream) {
    QSV_REQUIRE(out && qf && pool && block_table && seq && pos, "qsv_latent_attention: null argument");
    QSV_REQUIRE(chunk >= 0 && (!bias || bias_len > 0), "qsv_latent_attention: chunk %d, bias table of %d distances", chunk, bias_len);
    QSV_REQUIRE(n >= 0 && H > 0 && rank > 0 && R >= rank && page > 0 && table_stride > 0 && window >= 0,
                "qsv_latent_attention: bad sizes");
    QSV_REQUIRE(heads_per_pool > 0 && H % heads_per_pool == 0 && pool_stride >= 0, "qsv_latent_attention: %d heads over pools of %d",
                H, heads_per_pool);
    QSV_REQUIRE(keep_first >= 0 && (!keep_first || (window > 0 && !chunk)), "qsv_latent_attention: %d kept first positions need a window and no chunks", keep_first);
    QSV_REQUIRE(!pooled || (window > 0 && !chunk && !bias && !keep_first && pool_block > 0 && block_rows > 0 && pooled_stride >= 0 &&
                            (int64_t)block_rows * pool_block >= page),
                "qsv_latent_attention: pooled blocks of %d positions, %d rows per page of %d", pool_block, block_rows, page);
    if (n == 0) return QSV_OK;
    QSV_REQUIRE((int64_t)n * H < (1ll << 31), "qsv_latent_attention: too many (token, head) pairs");
    (void)variant;
    int rc = QSV_OK;
    QSV_DISPATCH(dtype, "qsv_latent_attention",
                 rc = launch_wave<T>(out, qf, pool, block_table, table_stride, seq, pos, window, n, H, rank, R, page, heads_per_pool,
                                     pool_stride, chunk, bias, bias_len, keep_first, sink, pooled, pooled_stride, pool_block, block_rows,
                                     (hipStream_t)stream));
    if (rc != QSV_OK) return rc;
    return qsv_launch_status("qsv_latent_attention");
}


// ---- pooled blocks: the mean of a finished block's cache rows --------------------------------------------------------------------
// Workgroup = (token, pool); only a token whose position ends a block works.  The block's rows are read as the cache holds them,
// summed in float in position order, divided once.
template <typename T>
__global__ __launch_bounds__(256) void pool_blocks_kernel(T* __restrict__ pooled, int64_t pooled_rows, const T* __restrict__ pool,
                                                          int64_t pool_rows, const int32_t* __restrict__ block_table, int table_stride,
                                                          const int32_t* __restrict__ seq, const int32_t* __restrict__ pos, int R,
                                                          int pool_block, int page, int block_rows) {
    const size_t t = blockIdx.x;
    const int g = blockIdx.y;
    const int p = pos[t];
    if ((p + 1) % pool_block) return;
    const int32_t* bt = block_table + (size_t)seq[t] * table_stride;
    const int first = p + 1 - pool_block;
    const T* src = pool + (size_t)g * pool_rows * R;
    T* dst = pooled + ((size_t)g * pooled_rows + (size_t)bt[first / page] * block_rows + (size_t)((first % page) / pool_block)) * R;
    const float inv = 1.0f / (float)pool_block;
    for (int c = threadIdx.x; c < R; c += 256) {
        float a = 0.f;
        for (int j = first; j <= p; ++j) a += ld(src, ((size_t)bt[j / page] * page + (size_t)(j % page)) * R + c);
        st(dst, c, a * inv);
    }
}
// The same for rows that are whole 16-byte pieces (VEC elements each) and at most 256 pieces wide: a row's pieces side by side over
// the lanes, the block's rows dealt to 256 / pieces row groups that sum their share at once; the groups' sums meet in LDS.
__device__ __forceinline__ void load_piece(const float* p, float (&v)[4]) {
    const float4 a = *(const float4*)p;
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
}
__device__ __forceinline__ void load_piece(const bf16_t* p, float (&v)[8]) {
    const uint4 u = *(const uint4*)p;
    const unsigned w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[2 * i] = __uint_as_float(w[i] << 16);
        v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
}
template <typename T, int VEC>
__global__ __launch_bounds__(256) void pool_blocks_vec_kernel(T* __restrict__ pooled, int64_t pooled_rows, const T* __restrict__ pool,
                                                              int64_t pool_rows, const int32_t* __restrict__ block_table,
                                                              int table_stride, const int32_t* __restrict__ seq,
                                                              const int32_t* __restrict__ pos, int R, int pool_block, int page,
                                                              int block_rows) {
    __shared__ float part[256][VEC];
    const size_t t = blockIdx.x;
    const int g = blockIdx.y;
    const int p = pos[t];
    if ((p + 1) % pool_block) return;                       // (the whole workgroup)
    const int32_t* bt = block_table + (size_t)seq[t] * table_stride;
    const int first = p + 1 - pool_block;
    const int pieces = R / VEC, groups = 256 / pieces;
    const int col = threadIdx.x % pieces, grp = threadIdx.x / pieces;
    const T* src = pool + (size_t)g * pool_rows * R;
    float acc[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc[e] = 0.f;
    if (grp < groups) {
        for (int j = first + grp; j <= p; j += groups) {
            float v[VEC];
            load_piece(src + ((size_t)bt[j / page] * page + (size_t)(j % page)) * R + col * VEC, v);
#pragma unroll
            for (int e = 0; e < VEC; ++e) acc[e] += v[e];
        }
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) part[threadIdx.x][e] = acc[e];
    __syncthreads();
    if (grp != 0) return;
    for (int k = 1; k < groups; ++k)
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[e] += part[k * pieces + col][e];
    T* dst = pooled + ((size_t)g * pooled_rows + (size_t)bt[first / page] * block_rows + (size_t)((first % page) / pool_block)) * R;
    const float inv = 1.0f / (float)pool_block;
#pragma unroll
    for (int e = 0; e < VEC; ++e) st(dst, col * VEC + e, acc[e] * inv);
}
extern "C" int qsv_pool_blocks(void* pooled, int64_t pooled_rows, const void* pool, int64_t pool_rows, const int32_t* block_table,
                               int table_stride, const int32_t* seq, const int32_t* pos, int n, int n_pools, int R, int pool_block,
                               int page, int block_rows, int dtype, void* stream) {
    QSV_REQUIRE(pooled && pool && block_table && seq && pos, "qsv_pool_blocks: null argument");
    QSV_REQUIRE(n >= 0 && n_pools > 0 && n_pools <= 65535 && R > 0 && pool_block > 0 && page > 0 && block_rows > 0 &&
                    (int64_t)block_rows * pool_block >= page && table_stride > 0,
                "qsv_pool_blocks: blocks of %d positions, %d rows per page of %d", pool_block, block_rows, page);
    if (n == 0) return QSV_OK;
    if (dtype == QSV_BF16 && R % 8 == 0 && R / 8 <= 256) {
        hipLaunchKernelGGL((pool_blocks_vec_kernel<bf16_t, 8>), dim3(n, n_pools), dim3(256), 0, (hipStream_t)stream, (bf16_t*)pooled,
                           pooled_rows, (const bf16_t*)pool, pool_rows, block_table, table_stride, seq, pos, R, pool_block, page, block_rows);
        return qsv_launch_status("qsv_pool_blocks");
    }
    if (dtype == QSV_F32 && R % 4 == 0 && R / 4 <= 256) {
        hipLaunchKernelGGL((pool_blocks_vec_kernel<float, 4>), dim3(n, n_pools), dim3(256), 0, (hipStream_t)stream, (float*)pooled,
                           pooled_rows, (const float*)pool, pool_rows, block_table, table_stride, seq, pos, R, pool_block, page, block_rows);
        return qsv_launch_status("qsv_pool_blocks");
    }
    QSV_DISPATCH(dtype, "qsv_pool_blocks",
                 hipLaunchKernelGGL(pool_blocks_kernel<T>, dim3(n, n_pools), dim3(256), 0, (hipStream_t)stream, (T*)pooled, pooled_rows,
                                    (const T*)pool, pool_rows, block_table, table_stride, seq, pos, R, pool_block, page, block_rows));
    return qsv_launch_status("qsv_pool_blocks");
}
