// serve_moe_gemm.hip -- grouped expert products on the bf16 matrix cores for the prompt phase (many tokens per expert).
//
// The (token, expert) slots are sorted by expert; a work tile = up to 128 consecutive sorted slots of ONE expert (tile list made
// by the host from the run lengths).  A workgroup computes 256 weight rows x 128 slots of out[s, n] = act(W[e][n, :] . x(s)):
// both operands are contiguous along the reduction, so with the weight rows as the A operand and the slots' inputs as the B
// operand (v_mfma_f32_16x16x32_bf16) a lane ends up with 4 consecutive n of one slot - an 8-byte store.  The input row of a
// slot is fetched through an index (the gather into sorted order is part of the load), relu(.)^2 is the epilogue of the first
// product (or the gated unit: gate and up rows interleaved in the weight).  K steps of 64 through LDS (stride 72 elements: conflict-free 16-byte reads), the next step's pieces in flight in
// registers while this one is multiplied.
#include "serve_common.h"

namespace {
typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 bf8 __attribute__((ext_vector_type(8)));
typedef unsigned int v4u __attribute__((ext_vector_type(4)));
typedef unsigned int v2u __attribute__((ext_vector_type(2)));

constexpr int BNW = 256;     // weight rows per workgroup (64 per wave)
constexpr int MT = BNW / 64; // 16-row blocks per wave
constexpr int BS = 128;      // slots per tile
constexpr int KS = 64;       // reduction elements per step
constexpr int LS = KS + 8;   // LDS row stride (elements)
constexpr int CPR = KS / 8;  // 16-byte pieces per row and step
constexpr int NPA = BNW * CPR / 256, NPB = BS * CPR / 256;   // pieces per thread

__device__ __forceinline__ unsigned pack_bf2(float a, float b) { return (unsigned)f2bf(a) | ((unsigned)f2bf(b) << 16); }

// ACT: 0 nothing, 1 relu^2, 2 gated unit - weight rows 2f (gate) and 2f + 1 (up) are neighbours, so a lane's four rows are two
// whole units: out[s, f] = silu(gate) * up, N / 2 wide
template <int ACT>
__global__ __launch_bounds__(256, 2) void grouped_gemm_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ X,
                                                           const int64_t* __restrict__ x_index, int div,
                                                           const bf16_t* __restrict__ W, const int32_t* __restrict__ tiles, int N,
                                                           int K, float limit) {
    __shared__ __attribute__((aligned(16))) bf16_t As[BNW * LS];
    __shared__ __attribute__((aligned(16))) bf16_t Bs[BS * LS];
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int col = lane & 15, g4 = lane >> 4;
    const int e = tiles[3 * blockIdx.y], s_first = tiles[3 * blockIdx.y + 1], ns = tiles[3 * blockIdx.y + 2];
    const int n0 = blockIdx.x * BNW;
    // this thread's pieces of a K step: piece q = tid + 256 i is row q / CPR, 16 bytes number q % CPR
    const bf16_t* ap[NPA];
    const bf16_t* bp[NPB];
    bool aok[NPA], bok[NPB];
#pragma unroll
    for (int i = 0; i < NPA; ++i) {
        const int q = tid + 256 * i, row = q / CPR, cc = q % CPR;
        aok[i] = n0 + row < N;
        ap[i] = W + ((size_t)e * N + (aok[i] ? n0 + row : 0)) * (size_t)K + cc * 8;
    }
#pragma unroll
    for (int i = 0; i < NPB; ++i) {
        const int q = tid + 256 * i, row = q / CPR, cc = q % CPR;
        bok[i] = row < ns;
        const int64_t s = s_first + (bok[i] ? row : 0);
        bp[i] = X + (size_t)(x_index ? x_index[s] / div : s) * (size_t)K + cc * 8;
    }
    v4f acc[MT][BS / 16];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < BS / 16; ++nt) acc[mt][nt] = v4f{0.f, 0.f, 0.f, 0.f};
    const v4u zero = {0u, 0u, 0u, 0u};
    v4u ra[NPA], rb[NPB];
#pragma unroll
    for (int i = 0; i < NPA; ++i) ra[i] = aok[i] ? *(const v4u*)ap[i] : zero;
#pragma unroll
    for (int i = 0; i < NPB; ++i) rb[i] = bok[i] ? *(const v4u*)bp[i] : zero;
    for (int k0 = 0; k0 < K; k0 += KS) {
        __syncthreads();                                            // the previous step has been read
#pragma unroll
        for (int i = 0; i < NPA; ++i) {
            const int q = tid + 256 * i;
            *(v4u*)(As + (q / CPR) * LS + (q % CPR) * 8) = ra[i];
        }
#pragma unroll
        for (int i = 0; i < NPB; ++i) {
            const int q = tid + 256 * i;
            *(v4u*)(Bs + (q / CPR) * LS + (q % CPR) * 8) = rb[i];
        }
        __syncthreads();
        if (k0 + KS < K) {                                          // next step's pieces: in flight during the products
#pragma unroll
            for (int i = 0; i < NPA; ++i) ra[i] = aok[i] ? *(const v4u*)(ap[i] + k0 + KS) : zero;
#pragma unroll
            for (int i = 0; i < NPB; ++i) rb[i] = bok[i] ? *(const v4u*)(bp[i] + k0 + KS) : zero;
        }
#pragma unroll
        for (int kk = 0; kk < KS; kk += 32) {
            v4u a[MT];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) a[mt] = *(const v4u*)(As + (16 * MT * w + 16 * mt + col) * LS + kk + 8 * g4);
#pragma unroll
            for (int nt = 0; nt < BS / 16; ++nt) {
                const v4u b = *(const v4u*)(Bs + (16 * nt + col) * LS + kk + 8 * g4);
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf8, a[mt]), __builtin_bit_cast(bf8, b),
                                                                          acc[mt][nt], 0, 0, 0);
            }
        }
    }
    // this lane: slot 16 nt + col, weight rows n0 + 16 MT w + 16 mt + 4 g4 + (0 .. 3)
#pragma unroll
    for (int nt = 0; nt < BS / 16; ++nt) {
        const int sl = 16 * nt + col;
        if (sl >= ns) continue;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int n = n0 + 16 * MT * w + 16 * mt + 4 * g4;
            if (n >= N) continue;                                   // N % 4 == 0: the four rows are inside together
            v4f v = acc[mt][nt];
            if (ACT == 2) {
                float u0, u1;
                if (limit > 0.f) {                                  // clamped units: g sigmoid(1.702 g) (u + 1) (uniform over the launch)
                    const float ga = fminf(v[0], limit), gb = fminf(v[2], limit);
                    u0 = ga / (1.0f + expf(-1.702f * ga)) * (fminf(fmaxf(v[1], -limit), limit) + 1.0f);
                    u1 = gb / (1.0f + expf(-1.702f * gb)) * (fminf(fmaxf(v[3], -limit), limit) + 1.0f);
                } else {
                    u0 = v[0] / (1.0f + expf(-v[0])) * v[1];
                    u1 = v[2] / (1.0f + expf(-v[2])) * v[3];
                }
                *(unsigned*)(out + (size_t)(s_first + sl) * (N / 2) + n / 2) = pack_bf2(u0, u1);
                continue;
            }
            if (ACT == 1) {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float x = fmaxf(v[r], 0.f);
                    v[r] = x * x;
                }
            }
            const v2u pk = {pack_bf2(v[0], v[1]), pack_bf2(v[2], v[3])};
            *(v2u*)(out + (size_t)(s_first + sl) * N + n) = pk;
        }
    }
}
}  // namespace

// out[s, n] = act(W[e][n, :] . X[x_index ? x_index[s] / div : s, :]) for every tile (e, first sorted slot, slots <= qsv_grouped_gemm_tile_slots());
// W [E, N, K], all bfloat16; K % 64 == 0, N % 4 == 0.
extern "C" int qsv_grouped_gemm_tile_slots(void) { return BS; }
extern "C" int qsv_grouped_gemm_k_step(void) { return KS; }
extern "C" int qsv_grouped_gemm(void* out, const void* X, const int64_t* x_index, int div, const void* W, const int32_t* tiles,
                                int n_tiles, int N, int K, int act, float limit, void* stream) {
    QSV_REQUIRE(out && X && W && tiles && div > 0 && n_tiles >= 0, "qsv_grouped_gemm: bad arguments");
    QSV_REQUIRE(N > 0 && N % 4 == 0 && K > 0 && K % KS == 0, "qsv_grouped_gemm: N %d (a multiple of 4), K %d (a multiple of 64)", N, K);
    QSV_REQUIRE(n_tiles <= 65535, "qsv_grouped_gemm: %d tiles (at most 65535 per launch)", n_tiles);
    QSV_REQUIRE(act == QSV_ACT_NONE || act == QSV_ACT_RELU_SQ || act == QSV_ACT_GLU || (act == QSV_ACT_CLAMPED_GLU && limit > 0.f),
                "qsv_grouped_gemm: activation %d (limit %g)", act, (double)limit);
    if (act == QSV_ACT_CLAMPED_GLU) act = QSV_ACT_GLU;
    else limit = 0.f;
    if (n_tiles == 0) return QSV_OK;
    const dim3 grid((N + BNW - 1) / BNW, n_tiles), block(256);
#define QSV_GG(ACT)                                                                                                          \
    hipLaunchKernelGGL(grouped_gemm_kernel<ACT>, grid, block, 0, (hipStream_t)stream, (bf16_t*)out, (const bf16_t*)X, x_index, div, \
                       (const bf16_t*)W, tiles, N, K, limit)
    if (act == QSV_ACT_RELU_SQ) QSV_GG(1);
    else if (act == QSV_ACT_GLU) QSV_GG(2);
    else QSV_GG(0);
#undef QSV_GG
    return qsv_launch_status("qsv_grouped_gemm");
}
