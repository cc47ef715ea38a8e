// serve_attention_mfma.hip -- latent attention on the bf16 matrix cores (v_mfma_f32_16x16x32_bf16), prompts and decoding.
//
// Work unit ("tile", made by the host): up to TPB consecutive tokens of ONE sequence in this step.  A workgroup of four waves
// serves a tile; a wave owns 16 query rows = TQ tokens x HP head slots (HP = heads rounded up to a power of two, at most 16;
// more than 16 heads: blockIdx.y walks head groups of 16).  Sixteen rows, not 32: a row of 576 query values and 512 output
// columns then costs a lane 72 + 128 registers and nothing spills (the 32-row form needed 144 + 256).  Keys arrive in tiles
// of 32 cache rows, staged once per workgroup in LDS in two forms: row-major (A operand of S^T = K Q^T, plain 16-byte
// reads) and transposed (A operand of O^T = C^T P^T, 8-byte reads).  With the products swapped like this a lane holds 8 of
// the 32 scores of ITS query row, so the softmax needs two exchanges (lanes ^ 16, ^ 32) and the probabilities already sit in
// B-operand order (the k-slot <-> key mapping of the second product is chosen to match the accumulator layout of the first).
// A tile with few tokens (decoding: one) does not fill four waves with rows; then the waves split the KEY tiles among them and
// merge their partial softmax results through LDS at the end.
// Scores, running maxima and sums are float; q and the probabilities enter the matrix cores as bfloat16.
//
// Keys behind the window: a workgroup's key tiles are numbered, first nA tiles of such keys, then the tiles from the window's start.
// With `keep_first` these are the tiles of the sequence's first positions that lie wholly below the window's first tile (a kept
// position inside a window tile is simply visible there); with `pooled` they are tiles of 32 consecutive BLOCKS, one row per block of
// `pool_block` positions from a second pool, each row addressed through the page of the block's first position.  A sink starts the
// softmax state of the rows' first key split at (maximum = sink, sum = 1).
#include "serve_common.h"

namespace {
typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 bf8 __attribute__((ext_vector_type(8)));
typedef unsigned int v4u __attribute__((ext_vector_type(4)));
typedef unsigned int v2u __attribute__((ext_vector_type(2)));

constexpr int NWV = 4;
constexpr int BN = 32;          // keys per tile
constexpr int VS = BN + 4;      // row stride (elements) of the transposed tile: 18 dwords, 8-byte reads of 32 lanes hit 64 banks

__device__ __forceinline__ unsigned pack_bf2(float a, float b) { return (unsigned)f2bf(a) | ((unsigned)f2bf(b) << 16); }

// RT: 32-element steps along a cache row (R <= 32 RT); CT: 16-column tiles of the output (rank <= 16 CT).
template <int RT, int CT>
__global__ __launch_bounds__(64 * NWV, (RT > 10 ? 1 : 2)) void latent_attention_mfma_kernel(
    bf16_t* __restrict__ out, const float* __restrict__ qf, const bf16_t* __restrict__ pool_base,
    const int32_t* __restrict__ block_table, int table_stride, const int32_t* __restrict__ pos, const int32_t* __restrict__ tiles,
    int window, int H, int rank, int R, int page, int HP, int TQ, float* __restrict__ part_o, float* __restrict__ part_ml,
    int n_tokens, int s_lo, int s_hi, int per, int64_t pool_stride, int chunk, const float* __restrict__ bias, int bias_len,
    int keep_first, const float* __restrict__ sink, const bf16_t* __restrict__ pooled_base, int64_t pooled_stride, int pool_block,
    int block_rows) {
    constexpr int RS = 32 * RT + 8;                      // row stride (elements) of the row-major tile
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    bf16_t* Ks = (bf16_t*)smem;                          // [BN][RS]
    bf16_t* Vt = Ks + BN * RS;                           // [16 CT][VS]
    float* scratch = (float*)smem;                       // merge phase (after the key loop)

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int col = lane & 15, g4 = lane >> 4;           // query row of this lane; k-group / accumulator row block
    const int slot = tiles[3 * blockIdx.x], t0 = tiles[3 * blockIdx.x + 1], ntok = tiles[3 * blockIdx.x + 2];
    // heads [g per, (g + 1) per) read pool g (pool_stride elements apart): blockIdx.y walks the pools' head groups of 16
    const int gpp = (per + 15) / 16, pool_id = blockIdx.y / gpp;
    const int h0 = pool_id * per + (blockIdx.y % gpp) * 16, h_end = pool_id * per + per;
    const bf16_t* __restrict__ pool = pool_base + (size_t)pool_id * (size_t)pool_stride;
    const bf16_t* __restrict__ pooled = pooled_base ? pooled_base + (size_t)pool_id * (size_t)pooled_stride : nullptr;
    const int32_t* bt = block_table + (size_t)slot * table_stride;

    // rows of this wave: group grp of TQ tokens, key split sp
    const int G = (ntok + TQ - 1) / TQ;                  // 1 .. 4
    const int S = NWV / G;
    const bool active = w < G * S;
    const int grp = active ? w % G : 0, sp = active ? w / G : 0;
    const int tok_in = grp * TQ + col / HP;              // token of this lane's query row within the tile
    const int head = h0 + col % HP;
    const bool row_ok = active && tok_in < ntok && head < h_end;
    const int t = t0 + (tok_in < ntok ? tok_in : 0);
    const int p_row = pos[t];
    int lo_row = window > 0 ? max(0, p_row - window + 1) : 0;
    if (chunk > 0) lo_row = max(lo_row, p_row - p_row % chunk);   // chunks are counted from position 0 of the sequence
    const float* brow = bias ? bias + (size_t)(row_ok ? head : 0) * bias_len : nullptr;

    // block key range (tokens of a tile are consecutive positions; read both ends)
    const int p_first = pos[t0], p_last = pos[t0 + ntok - 1];
    int lo_first = window > 0 ? max(0, p_first - window + 1) : 0;
    if (chunk > 0) lo_first = max(lo_first, p_first - p_first % chunk);   // (the first token's bound is the tile's lowest)
    const int kstart = (lo_first / BN) * BN;
    // tiles of keys behind the window, and each row's count of such keys
    const int nb_last = pooled ? max(0, p_last - window + 1) / pool_block : 0;      // blocks the tile's last token sees
    const int nb_row = pooled ? max(0, p_row - window + 1) / pool_block : 0;
    const int nA = pooled ? (nb_last + BN - 1) / BN : (keep_first > 0 ? min((keep_first + BN - 1) / BN, kstart / BN) : 0);
    const int nT = nA + (p_last - kstart) / BN + 1;
    // wave key range: rows of this wave's group
    const int gt_first = min(grp * TQ, ntok - 1), gt_last = min(grp * TQ + TQ - 1, ntok - 1);
    const int wp_last = p_first + gt_last;
    int wlo = window > 0 ? max(0, p_first + gt_first - window + 1) : 0;
    if (chunk > 0) wlo = max(wlo, (p_first + gt_first) - (p_first + gt_first) % chunk);

    // Q fragments (B operand of S^T): the 8 consecutive elements 32 s + 8 g4 of this lane's row
    v4u qfrag[RT];
    {
        const float* qrow = qf + ((size_t)t * H + (row_ok ? head : 0)) * (size_t)R;
#pragma unroll
        for (int s = 0; s < RT; ++s) {
            const int e0 = 32 * s + 8 * g4;
            float4 lo4 = make_float4(0.f, 0.f, 0.f, 0.f), hi4 = lo4;
            if (row_ok && e0 < R) {                      // R % 8 == 0: a piece of 8 is inside or outside as a whole
                lo4 = *(const float4*)(qrow + e0);
                hi4 = *(const float4*)(qrow + e0 + 4);
            }
            qfrag[s] = v4u{pack_bf2(lo4.x, lo4.y), pack_bf2(lo4.z, lo4.w), pack_bf2(hi4.x, hi4.y), pack_bf2(hi4.z, hi4.w)};
        }
    }
    v4f oacc[CT];
#pragma unroll
    for (int c = 0; c < CT; ++c) oacc[c] = v4f{0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;
    if (sink && row_ok && sp == 0 && blockIdx.z == 0) {  // the sink's term: once per row, in its first key split
        m = sink[head];
        l = g4 == 0 ? 1.f : 0.f;                         // (l is a lane's share of the row's sum)
    }

    const int chunks_per_row = R / 8;                    // 16-byte pieces of a cache row (R % 8 == 0)
    // gridDim.z > 1 (decoding with few sequences): workgroup z takes every gridDim.z-th key tile and leaves an unnormalised
    // partial result; a second launch merges them
    const int Z = gridDim.z, z = blockIdx.z;
    // One tile = 32 consecutive positions inside ONE page (page % 32 == 0): a single block-table entry per tile.  The 16-byte
    // pieces of the NEXT tile are in flight (registers) while this tile is computed from LDS.
    constexpr int NCH = (BN * 4 * RT + 64 * NWV - 1) / (64 * NWV);
    v4u stage[NCH];
    auto issue = [&](int tile) {
        if (pooled && tile < nA) {                       // 32 blocks: every row through the page of its block's first position
#pragma unroll
            for (int i = 0; i < NCH; ++i) {
                const int q = tid + 64 * NWV * i, row = q % BN, cc = q / BN;
                stage[i] = v4u{0u, 0u, 0u, 0u};
                const int b = tile * BN + row;
                if (b < nb_last && cc < chunks_per_row) {
                    const int first = b * pool_block;
                    stage[i] = *(const v4u*)(pooled + ((size_t)bt[first / page] * block_rows + (size_t)((first % page) / pool_block)) * (size_t)R + cc * 8);
                }
            }
            return;
        }
        const int k0 = tile < nA ? tile * BN : kstart + (tile - nA) * BN;
        const bf16_t* base = pool + ((size_t)bt[k0 / page] * page + (size_t)(k0 % page)) * (size_t)R;
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int q = tid + 64 * NWV * i, row = q % BN, cc = q / BN;
            stage[i] = v4u{0u, 0u, 0u, 0u};
            if (k0 + row <= p_last && cc < chunks_per_row) stage[i] = *(const v4u*)(base + (size_t)row * R + cc * 8);
        }
    };
    int ti = 0;
    if (z < nT) issue(z);
    for (int tile = z; tile < nT; tile += Z, ++ti) {
        const bool pre = tile < nA;                      // (block-uniform) a tile of keys behind the window
        const int k0 = pre ? tile * BN : kstart + (tile - nA) * BN;
        __syncthreads();                                 // the previous tile has been read
        // ---- the staged rows into LDS: row-major and transposed (lanes walk the rows: the 2-byte transposed writes of a
        //      wave fall into 32 different banks) ----
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int q = tid + 64 * NWV * i, row = q % BN, cc = q / BN;
            if (cc < 4 * RT) {
                const v4u d = stage[i];
                *(v4u*)(Ks + row * RS + cc * 8) = d;
                if (cc * 8 < 16 * CT) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        Vt[(cc * 8 + 2 * e) * VS + row] = (bf16_t)(d[e] & 0xffffu);
                        Vt[(cc * 8 + 2 * e + 1) * VS + row] = (bf16_t)(d[e] >> 16);
                    }
                }
            }
        }
        __syncthreads();
        if (tile + Z < nT) issue(tile + Z);
        // (wave-uniform; a tile below the wave's window may still hold kept first positions)
        if (!active || (ti % S) != sp || (!pre && (k0 > wp_last || (k0 + BN - 1 < wlo && k0 >= keep_first)))) continue;
        // the bias of this lane's eight (query, key) pairs: requested before the score product, added after it
        float bv[2][4];
        if (brow) {
#pragma unroll
            for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                for (int r = 0; r < 4; ++r) bv[mt][r] = brow[min(max(p_row - (k0 + 16 * mt + 4 * g4 + r), 0), bias_len - 1)];
        }
        // ---- S^T = K Q^T: two blocks of 16 keys; this lane gets keys 16 mt + 4 g4 + r of its own query row ----
        v4f sacc[2] = {v4f{0.f, 0.f, 0.f, 0.f}, v4f{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
        for (int s = 0; s < RT; ++s) {
            if (s < s_lo || s >= s_hi) continue;         // (uniform) steps where every query is zero: a leading zero part, padding
#pragma unroll
            for (int mt = 0; mt < 2; ++mt) {
                const v4u a = *(const v4u*)(Ks + (16 * mt + col) * RS + 32 * s + 8 * g4);
                sacc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf8, a), __builtin_bit_cast(bf8, qfrag[s]),
                                                                   sacc[mt], 0, 0, 0);
            }
        }
        // ---- mask + online softmax (this lane: 8 keys of its query row; the other 24 sit in lanes ^16, ^32, ^48) ----
        float tmax = -INFINITY;
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int key = k0 + 16 * mt + 4 * g4 + r;
                const bool vis = (pooled && pre) ? key < nb_row : (key <= p_row && (key >= lo_row || key < keep_first));
                if (brow) sacc[mt][r] += bv[mt][r];
                sacc[mt][r] = vis ? sacc[mt][r] : -INFINITY;
                tmax = fmaxf(tmax, sacc[mt][r]);
            }
        tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
        const float mnew = fmaxf(m, tmax);
        const float msafe = mnew == -INFINITY ? 0.f : mnew;
        const float alpha = __expf(m - msafe);           // m = -inf: 0
        float psum = 0.f;
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                sacc[mt][r] = __expf(sacc[mt][r] - msafe);
                psum += sacc[mt][r];
            }
        l = l * alpha + psum;                            // (this lane's share; the four shares are added after the loop)
        m = mnew;
        if (__any(alpha != 1.0f)) {                      // (wave-uniform: the running maxima seldom move after the first tiles)
#pragma unroll
            for (int c = 0; c < CT; ++c) oacc[c] *= alpha;
        }
        // probabilities as B operand: k-slot (g4, e) <-> key 16 (e / 4) + 4 g4 + e % 4, i.e. exactly this lane's eight scores
        const v4u pb = {pack_bf2(sacc[0][0], sacc[0][1]), pack_bf2(sacc[0][2], sacc[0][3]),
                        pack_bf2(sacc[1][0], sacc[1][1]), pack_bf2(sacc[1][2], sacc[1][3])};
        // ---- O^T += C^T P^T ----
#pragma unroll
        for (int c = 0; c < CT; ++c) {
            const bf16_t* vrow = Vt + (16 * c + col) * VS + 4 * g4;
            const v2u a0 = *(const v2u*)vrow, a1 = *(const v2u*)(vrow + 16);
            const v4u a = {a0[0], a0[1], a1[0], a1[1]};
            oacc[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf8, a), __builtin_bit_cast(bf8, pb), oacc[c], 0, 0, 0);
        }
    }
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);

    // ---- merge the key splits (waves grp + G s, s = 1 .. S - 1, into wave grp) ----
    if (S > 1) {                                         // (block-uniform)
        __syncthreads();                                 // the last tile has been read: LDS becomes scratch
        float* ml = scratch + NWV * 8 * 64 * 4;          // [NWV][64][2], behind the accumulator exchange area
        if (active && sp > 0) {
            ml[(w * 64 + lane) * 2] = m;
            ml[(w * 64 + lane) * 2 + 1] = l;
        }
        __syncthreads();
        float f[NWV];
#pragma unroll
        for (int s = 0; s < NWV; ++s) f[s] = 0.f;
        if (active && sp == 0) {
            float M = m;
            for (int s = 1; s < S; ++s) M = fmaxf(M, ml[((grp + G * s) * 64 + lane) * 2]);
            const float Ms = M == -INFINITY ? 0.f : M;
            f[0] = __expf(m - Ms);
            float L = f[0] * l;
            for (int s = 1; s < S; ++s) {
                f[s] = __expf(ml[((grp + G * s) * 64 + lane) * 2] - Ms);
                L += f[s] * ml[((grp + G * s) * 64 + lane) * 2 + 1];
            }
            l = L;
            m = M;                                       // (what a cross-workgroup merge reads)
        }
        // accumulators through LDS, MB column tiles per exchange (two barriers each)
        constexpr int MB = CT < 8 ? CT : 8;
#pragma unroll
        for (int c0 = 0; c0 < CT; c0 += MB) {
            __syncthreads();
            if (active && sp > 0) {
#pragma unroll
                for (int j = 0; j < MB; ++j)
                    if (c0 + j < CT) *(v4f*)(scratch + ((w * MB + j) * 64 + lane) * 4) = oacc[c0 + j];
            }
            __syncthreads();
            if (active && sp == 0) {
#pragma unroll
                for (int j = 0; j < MB; ++j)
                    if (c0 + j < CT) {
                        v4f a = oacc[c0 + j] * f[0];
                        for (int s = 1; s < S; ++s) a += *(const v4f*)(scratch + (((grp + G * s) * MB + j) * 64 + lane) * 4) * f[s];
                        oacc[c0 + j] = a;
                    }
            }
        }
    }
    if (!row_ok || sp != 0) return;
    if (Z > 1) {                                         // partial result of this key split: [z][t][h][rank] and (m, l)
        const size_t rowi = ((size_t)z * n_tokens + t) * H + head;
        if (g4 == 0) {
            part_ml[rowi * 2] = m;
            part_ml[rowi * 2 + 1] = l;
        }
        float* po = part_o + rowi * (size_t)rank;
#pragma unroll
        for (int c = 0; c < CT; ++c) {
            const int c0 = 16 * c + 4 * g4;
            if (c0 < rank) *(v4f*)(po + c0) = oacc[c];
        }
        return;
    }
    const float inv = 1.0f / l;
    bf16_t* o = out + ((size_t)t * H + head) * (size_t)rank;
#pragma unroll
    for (int c = 0; c < CT; ++c) {
        const int c0 = 16 * c + 4 * g4;
        if (c0 < rank) {                                 // rank % 8 == 0: the four values are all inside
            const v2u v = {pack_bf2(oacc[c][0] * inv, oacc[c][1] * inv), pack_bf2(oacc[c][2] * inv, oacc[c][3] * inv)};
            *(v2u*)(o + c0) = v;
        }
    }
}

// out[t, h] = sum_z e^(m_z - M) o_z / sum_z e^(m_z - M) l_z   (one workgroup per (token, head))
__global__ __launch_bounds__(256) void latent_attention_merge_kernel(bf16_t* __restrict__ out, const float* __restrict__ part_o,
                                                                     const float* __restrict__ part_ml, int Z, int rows, int rank) {
    const size_t r = blockIdx.x;
    float M = -INFINITY;
    for (int z = 0; z < Z; ++z) M = fmaxf(M, part_ml[((size_t)z * rows + r) * 2]);
    float L = 0.f;
    for (int z = 0; z < Z; ++z) L += __expf(part_ml[((size_t)z * rows + r) * 2] - M) * part_ml[((size_t)z * rows + r) * 2 + 1];
    const float inv = 1.0f / L;
    for (int c = threadIdx.x; c < rank; c += 256) {
        float a = 0.f;
        for (int z = 0; z < Z; ++z)
            a += __expf(part_ml[((size_t)z * rows + r) * 2] - M) * part_o[((size_t)z * rows + r) * (size_t)rank + c];
        out[r * (size_t)rank + c] = f2bf(a * inv);
    }
}

struct Geometry {
    int HP, TQ;
};
Geometry geometry(int H) {
    int hp = 1;
    while (hp < H && hp < 16) hp <<= 1;
    return {hp, 16 / hp};
}
}  // namespace

// Tokens of one sequence a work tile may hold, for `heads` heads (the host cuts a step's portions into tiles of this size).
extern "C" int qsv_latent_attention_tile_tokens(int heads) {
    if (heads <= 0) return 0;
    return NWV * geometry(heads).TQ;
}

// 1 if the matrix-core kernel takes these sizes (bfloat16 storage only), else 0 and the caller uses the wave kernel.
extern "C" int qsv_latent_attention_mfma_ok(int rank, int row_width, int dtype) {
    return dtype == QSV_BF16 && rank % 8 == 0 && row_width % 8 == 0 && row_width <= 576 && rank <= 512 && rank >= 8;   // (and page % 32 == 0)
}

// tiles: int32 [n_tiles, 3] = (sequence slot, first flat token index, tokens <= qsv_latent_attention_tile_tokens(heads)).
// key_splits > 1: every tile's keys are cut over that many workgroups (for steps with few tiles: decoding); then part_o
// (float [key_splits, n_tokens, H, rank]) and part_ml (float [key_splits, n_tokens, H, 2]) are workspace.
extern "C" int qsv_latent_attention_mfma(void* out, const float* qf, const void* pool, const int32_t* block_table,
                                         int table_stride, const int32_t* pos, const int32_t* tiles, int n_tiles, int window,
                                         int H, int rank, int R, int page, int key_splits, float* part_o, float* part_ml,
                                         int n_tokens, int q_first, int heads_per_pool, int64_t pool_stride, int chunk,
                                         const float* bias, int bias_len, int keep_first, const float* sink, const void* pooled,
                                         int64_t pooled_stride, int pool_block, int block_rows, void* stream) {
    QSV_REQUIRE(keep_first >= 0 && (!keep_first || (window > 0 && !chunk)),
                "qsv_latent_attention_mfma: %d kept first positions need a window and no chunks", keep_first);
    QSV_REQUIRE(!pooled || (window > 0 && !chunk && !bias && !keep_first && pool_block > 0 && block_rows > 0 && pooled_stride >= 0 &&
                            (int64_t)block_rows * pool_block >= page),
                "qsv_latent_attention_mfma: pooled blocks of %d positions, %d rows per page of %d", pool_block, block_rows, page);
    QSV_REQUIRE(chunk >= 0 && (!bias || bias_len > 0), "qsv_latent_attention_mfma: chunk %d, bias table of %d distances", chunk, bias_len);
    QSV_REQUIRE(out && qf && pool && block_table && pos && tiles, "qsv_latent_attention_mfma: null argument");
    QSV_REQUIRE(qsv_latent_attention_mfma_ok(rank, R, QSV_BF16) && R >= rank && H > 0 && page > 0 && page % BN == 0 && window >= 0 && n_tiles >= 0,
                "qsv_latent_attention_mfma: sizes not supported (rank %d, row %d)", rank, R);
    if (n_tiles == 0) return QSV_OK;
    QSV_REQUIRE(heads_per_pool > 0 && H % heads_per_pool == 0 && pool_stride >= 0,
                "qsv_latent_attention_mfma: %d heads over pools of %d", H, heads_per_pool);
    const Geometry g = geometry(heads_per_pool);
    QSV_REQUIRE(key_splits >= 1 && key_splits <= 64 && (key_splits == 1 || (part_o && part_ml && n_tokens > 0)),
                "qsv_latent_attention_mfma: key splits without workspace");
    const dim3 grid(n_tiles, (H / heads_per_pool) * ((heads_per_pool + 15) / 16), key_splits), block(64 * NWV);
    QSV_REQUIRE(q_first >= 0 && q_first < R, "qsv_latent_attention_mfma: first query element %d of %d", q_first, R);
    const int rt = (R + 31) / 32, ct = (rank + 15) / 16;
    const int s_lo = q_first / 32, s_hi = rt;
#define QSV_MFMA(RT, CT)                                                                                                     \
    do {                                                                                                                     \
        size_t lds = (size_t)(BN * (32 * RT + 8) + 16 * CT * VS) * 2;                                                        \
        const size_t need = (size_t)NWV * 64 * (8 * 4 + 2) * 4;       /* merge scratch */                                                                       \
        if (lds < need) lds = need;                                                                                          \
        if (lds > 64 * 1024) {   /* above the default limit of dynamic LDS: raise it for this kernel */                        \
            const hipError_t e = hipFuncSetAttribute((const void*)latent_attention_mfma_kernel<RT, CT>,                      \
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);                  \
            QSV_REQUIRE(e == hipSuccess, "qsv_latent_attention_mfma: %s", hipGetErrorString(e));                             \
        }                                                                                                                    \
        hipLaunchKernelGGL((latent_attention_mfma_kernel<RT, CT>), grid, block, lds, (hipStream_t)stream, (bf16_t*)out, qf,  \
                           (const bf16_t*)pool, block_table, table_stride, pos, tiles, window, H, rank, R, page, g.HP, g.TQ, \
                           part_o, part_ml, n_tokens, s_lo, s_hi, heads_per_pool, pool_stride, chunk, bias, bias_len,         \
                           keep_first, sink, (const bf16_t*)pooled, pooled_stride, pool_block, block_rows);                       \
    } while (0)
    if (rt <= 4 && ct <= 8) QSV_MFMA(4, 8);
    else if (rt <= 6 && ct <= 12) QSV_MFMA(6, 12);
    else if (rt <= 8 && ct <= 8) QSV_MFMA(8, 8);
    else if (rt <= 10 && ct <= 16) QSV_MFMA(10, 16);
    else QSV_MFMA(18, 32);
#undef QSV_MFMA
    if (key_splits > 1) {
        const int rc = qsv_launch_status("qsv_latent_attention_mfma");
        if (rc != QSV_OK) return rc;
        hipLaunchKernelGGL(latent_attention_merge_kernel, dim3(n_tokens * H), dim3(256), 0, (hipStream_t)stream, (bf16_t*)out,
                           part_o, part_ml, key_splits, n_tokens * H, rank);
    }
    return qsv_launch_status("qsv_latent_attention_mfma");
}
