// Products group by group on MFMA, bfloat16: C[row, n] = sum_k A[row, k] * W[group][n, k], every group with a matrix of its
// own (W [groups, N, K], k contiguous). Two ways to say which rows belong to which group:
//   heads   : every row has all groups; group h reads columns h * a_off .. + K of A and writes columns h * c_off .. + N of C
//             (the per-head matrices of an attention); optionally times sigmoid(gate[row, h]);
//   experts : tiles (group, first slot, rows <= 32) from tm_moe_route; a tile's rows are slots first .. first + rows - 1, and
//             slot i reads row row_src[i] / src_div of A (row_src null: row i).
// Epilogues: a plain store in bfloat16 or in 32-bit, or, with a matrix of 2 N rows (gate rows, then up rows),
// silu(gate product) * up product, or the square of relu(product) in bfloat16. A block is RT tiles of 16 rows by 64 columns; its four wavefronts take 16 columns each;
// k ascends in steps of 32 through LDS, so an element's sum has one order wherever its row stands.
#include "common.h"
#include "api.h"
#include "attention_prefill_common.h"

#define GM_BN 64
#define GM_BK 32            // k of a step through LDS (BK of the kernel): 32, or 128 for tiles of few rows, whose steps are
                            // latency and not arithmetic: four times the bytes asked for at once, a quarter of the steps

enum { GM_STORE = 0, GM_STORE_F32 = 1, GM_SILU_MUL = 2, GM_RELU2 = 3 };

template <int RT, int MODE, int BK = GM_BK, int BN = GM_BN>
__global__ __launch_bounds__(256) void grouped_mfma_kernel(const bf16_t* __restrict__ A, int lda, int a_off,
                                                           const int* __restrict__ row_src, int src_div,
                                                           const bf16_t* __restrict__ W, void* __restrict__ Cv, int ldc, int c_off,
                                                           const float* __restrict__ gate, int ldg, const int* __restrict__ tiles,
                                                           const int* __restrict__ n_tiles, int T, int K, int N, int tail, int rot_,
                                                           const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                                           const int* __restrict__ positions) {
    constexpr int BM = RT * 16;
    constexpr bool GATED = MODE == GM_SILU_MUL;
    constexpr int GM_LD = BK + 8, PPR = BK / 8;                 // 16-byte pieces a row of a step
    constexpr int NCG = BN / GM_BN;                             // groups of 64 columns a block: a wavefront has 16 columns of each
    __shared__ __align__(16) bf16_t As[BM][GM_LD];
    __shared__ __align__(16) bf16_t Bs[GATED ? 2 : 1][BN][GM_LD];
    __shared__ int src[BM];
    int group, row0, rows;
    if (tiles) {
        if ((int)blockIdx.x >= n_tiles[0]) return;
        group = tiles[3 * blockIdx.x], row0 = tiles[3 * blockIdx.x + 1], rows = tiles[3 * blockIdx.x + 2];
    } else {
        group = blockIdx.z, row0 = blockIdx.x * BM, rows = min(BM, T - row0);
    }
    const int n0 = blockIdx.y * BN;
    const int wave = threadIdx.x / TM_WAVE, lane = threadIdx.x % TM_WAVE, r = lane % 16, g = lane / 16;
    const bf16_t* Wg = W + (size_t)group * (GATED ? 2 : 1) * N * K;
    if (threadIdx.x < BM) {
        const int i = threadIdx.x;
        src[i] = i < rows ? (row_src ? row_src[row0 + i] / src_div : row0 + i) : -1;
    }
    __syncthreads();
    f32x4_t acc[NCG][RT], acu[NCG][GATED ? RT : 1];
#pragma unroll
    for (int cg = 0; cg < NCG; ++cg) {
#pragma unroll
        for (int t = 0; t < RT; ++t) acc[cg][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int t = 0; t < (GATED ? RT : 1); ++t) acu[cg][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }
    // a thread's pieces of a k-step: NA of A and NB of W (twice that with a gate); those of the step after the current one are
    // asked for before the current one is multiplied
    constexpr int NA = (BM * PPR + 255) / 256, NB = BN * PPR / 256;
    u32x4_t ha[NA], hb[NB], hu[GATED ? NB : 1];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int u = 0; u < NA; ++u) {
            const int idx = threadIdx.x + 256 * u, i = idx / PPR, c = idx % PPR;
            ha[u] = u32x4_t{0, 0, 0, 0};
            if (idx < BM * PPR && src[i] >= 0 && k0 + 8 * c < K)
                ha[u] = *(const u32x4_t*)(A + (size_t)src[i] * lda + (size_t)group * a_off + k0 + 8 * c);
        }
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            const int idx = threadIdx.x + 256 * u, bn = idx / PPR, bc = idx % PPR;
            const bool in = n0 + bn < N && k0 + 8 * bc < K;
            hb[u] = u32x4_t{0, 0, 0, 0};
            if (in) hb[u] = *(const u32x4_t*)(Wg + (size_t)(n0 + bn) * K + k0 + 8 * bc);
            if (GATED) {
                hu[u] = u32x4_t{0, 0, 0, 0};
                if (in) hu[u] = *(const u32x4_t*)(Wg + (size_t)(N + n0 + bn) * K + k0 + 8 * bc);
            }
        }
    };
    fetch(0);
    for (int k0 = 0; k0 < K; k0 += BK) {
#pragma unroll
        for (int u = 0; u < NA; ++u) {
            const int idx = threadIdx.x + 256 * u;
            if (idx < BM * PPR) *(u32x4_t*)&As[idx / PPR][8 * (idx % PPR)] = ha[u];
        }
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            const int idx = threadIdx.x + 256 * u;
            *(u32x4_t*)&Bs[0][idx / PPR][8 * (idx % PPR)] = hb[u];
            if (GATED) *(u32x4_t*)&Bs[GATED ? 1 : 0][idx / PPR][8 * (idx % PPR)] = hu[u];
        }
        __syncthreads();
        if (k0 + BK < K) fetch(k0 + BK);
#pragma unroll
        for (int kk = 0; kk < BK; kk += 32) {                   // k ascends in 32s whatever BK is: the same sums, bit for bit
            PFrag bf[NCG], bu[NCG];
#pragma unroll
            for (int cg = 0; cg < NCG; ++cg) {
                bf[cg].u = *(const u32x4_t*)&Bs[0][GM_BN * cg + 16 * wave + r][kk + 8 * g];
                if (GATED) bu[cg].u = *(const u32x4_t*)&Bs[GATED ? 1 : 0][GM_BN * cg + 16 * wave + r][kk + 8 * g];
            }
#pragma unroll
            for (int t = 0; t < RT; ++t) {
                PFrag af;
                af.u = *(const u32x4_t*)&As[16 * t + r][kk + 8 * g];
                // rows of A as the first operand: the result holds C[row 4 g + i][column r]; a piece of A read from LDS
                // meets every column group of the wavefront
#pragma unroll
                for (int cg = 0; cg < NCG; ++cg) {
                    acc[cg][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af.b, bf[cg].b, acc[cg][t], 0, 0, 0);
                    if (GATED) acu[cg][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af.b, bu[cg].b, acu[cg][t], 0, 0, 0);
                }
            }
        }
        __syncthreads();
    }
    // heads: the `tail` channels that follow a head's K input channels go behind its N output channels, their first |rot_|
    // rotated in pairs (2i, 2i + 1), or (i, i + |rot_| / 2) where rot_ < 0, by the row's position (the rotated part of a query
    // head beside its part on the latent)
    if (MODE == GM_STORE && tail > 0 && blockIdx.y == 0) {
        const int rot = rot_ < 0 ? -rot_ : rot_;
        const int half = rot / 2, rest = tail - rot;
        for (int idx = threadIdx.x; idx < rows * half; idx += 256) {
            const int row = row0 + idx / half, c = idx % half;
            const int c1 = rot_ < 0 ? c : 2 * c, c2 = rot_ < 0 ? c + half : 2 * c + 1;
            const bf16_t* sp = A + (size_t)row * lda + (size_t)group * a_off + K;
            bf16_t* dp = (bf16_t*)Cv + (size_t)row * ldc + (size_t)group * c_off + N;
            const size_t at = (size_t)positions[row] * half + c;
            float a, b;
            rotate_pair(bf16_to_f32(sp[c1]), bf16_to_f32(sp[c2]), cos_t[at], sin_t[at], a, b);
            dp[c1] = f32_to_bf16(a);
            dp[c2] = f32_to_bf16(b);
        }
        for (int idx = threadIdx.x; idx < rows * rest; idx += 256) {
            const int row = row0 + idx / rest, c = rot + idx % rest;
            ((bf16_t*)Cv)[(size_t)row * ldc + (size_t)group * c_off + N + c] = A[(size_t)row * lda + (size_t)group * a_off + K + c];
        }
    }
#pragma unroll
    for (int cg = 0; cg < NCG; ++cg) {
        const int n = n0 + GM_BN * cg + 16 * wave + r;
        if (n >= N) continue;
#pragma unroll
        for (int t = 0; t < RT; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int row = 16 * t + 4 * g + i;
                if (row >= rows) continue;
                const size_t at = (size_t)(row0 + row) * ldc + (size_t)group * c_off + n;
                float v = acc[cg][t][i];
                if (MODE == GM_SILU_MUL) {
                    const float u = acu[cg][t][i];
                    ((bf16_t*)Cv)[at] = f32_to_bf16(v / (1.0f + __expf(-v)) * u);
                } else if (MODE == GM_RELU2) {
                    v = fmaxf(v, 0.f);
                    ((bf16_t*)Cv)[at] = f32_to_bf16(v * v);
                } else if (MODE == GM_STORE_F32) {
                    ((float*)Cv)[at] = v;
                } else {
                    if (gate) v *= 1.0f / (1.0f + __expf(-gate[(size_t)(row0 + row) * ldg + group]));
                    ((bf16_t*)Cv)[at] = f32_to_bf16(v);
                }
            }
    }
}

static bool gm_aligned(const void* p) { return ((uintptr_t)p % 16) == 0; }

// Whether the per-head product takes these operands: K, the row strides of A and the heads' offsets in whole 16-byte pieces.
extern "C" int tm_heads_matmul_mfma_takes(const void* A, int lda, int a_off, const void* W, int K) {
    return gm_aligned(A) && gm_aligned(W) && K % 8 == 0 && lda % 8 == 0 && a_off % 8 == 0;
}

// C[t, h * c_off + n] = sum_k A[t, h * a_off + k] * W[h][n][k] (W [H, N, K]), times sigmoid(gate[t * ldg + h]) if gate.
// tail > 0: also C[t, h * c_off + N + c] = A[t, h * a_off + K + c] for c < tail, the first `rot` of them rotated in pairs
// (2i, 2i + 1), or (i, i + rot / 2) with half_pairs, by positions[t] (cos_t, sin_t [positions, rot / 2]).
extern "C" int tm_heads_matmul_mfma(const void* A, int lda, int a_off, const void* W, void* C, int ldc, int c_off, const float* gate,
                                    int ldg, int T, int H, int K, int N, int tail, int rot, const float* cos_t, const float* sin_t,
                                    const int* positions, int half_pairs, hipStream_t stream) {
    if (!A || !W || !C || T < 0 || H <= 0 || H > 65535 || K <= 0 || N <= 0 || tail < 0 || rot < 0 || rot > tail || rot % 2 ||
        a_off < K + tail || c_off < N + tail || !tm_heads_matmul_mfma_takes(A, lda, a_off, W, K) || (gate && ldg < H) ||
        (rot && (!cos_t || !sin_t || !positions)))
        return TM_ERR_ARG;
    if (T == 0) return TM_OK;
    dim3 grid((T + 63) / 64, (N + GM_BN - 1) / GM_BN, H);
    if (grid.y > 65535) return TM_ERR_ARG;
    grouped_mfma_kernel<4, GM_STORE><<<grid, 256, 0, stream>>>((const bf16_t*)A, lda, a_off, nullptr, 1, (const bf16_t*)W, C, ldc, c_off,
                                                               gate, ldg, nullptr, nullptr, T, K, N, tail, half_pairs ? -rot : rot, cos_t, sin_t,
                                                               positions);
    TM_CHECK_LAUNCH();
    return TM_OK;
}

// The experts' products of moe.hip on MFMA: the same operands, bfloat16, K and F multiples of 8, the route's tiles of
// tile_rows = 32, 64 or 128 rows (the larger, the fewer times an expert's matrices are read).
extern "C" int tm_moe_mfma_takes(const void* x, int ldx, const void* Wgu, const void* Wd, const void* act, int K, int F) {
    return gm_aligned(x) && gm_aligned(Wgu) && gm_aligned(Wd) && gm_aligned(act) && K % 8 == 0 && F % 8 == 0 && ldx % 8 == 0;
}

extern "C" int tm_moe_gate_up_mfma(const void* x, int ldx, const int* slot_pair, int top, const void* W, void* act, const int* tiles,
                                   const int* n_tiles, int max_tiles, int tile_rows, int K, int F, hipStream_t stream) {
    if (tile_rows != 32 && tile_rows != 64 && tile_rows != 128) return TM_ERR_ARG;
    if (!x || !slot_pair || !W || !act || !tiles || !n_tiles || top <= 0 || K <= 0 || F <= 0 || ldx < K || max_tiles < 0 || K % 8 ||
        ldx % 8 || !gm_aligned(x) || !gm_aligned(W))
        return TM_ERR_ARG;
    if (max_tiles == 0) return TM_OK;
    dim3 grid(max_tiles, (F + GM_BN - 1) / GM_BN);
    if (grid.y > 65535) return TM_ERR_ARG;
#define GM_GO(RT_, BK_, BN_)                                                                                                             \
    grouped_mfma_kernel<RT_, GM_SILU_MUL, BK_, BN_><<<dim3(max_tiles, (F + BN_ - 1) / BN_), 256, 0, stream>>>((const bf16_t*)x, ldx, 0, slot_pair, top, (const bf16_t*)W, act, F, \
                                                                    0, nullptr, 0, tiles, n_tiles, 0, K, F, 0, 0, nullptr, nullptr, nullptr)
    // (64 columns a block whatever the tile: with a gate a wavefront holds two results a column)
    if (tile_rows == 32) GM_GO(2, 128, GM_BN); else if (tile_rows == 64) GM_GO(4, GM_BK, GM_BN); else GM_GO(8, GM_BK, GM_BN);
#undef GM_GO
    TM_CHECK_LAUNCH();
    return TM_OK;
}

// Experts without a gate: act[slot] = relu(x[t] . W[e]^T)^2, W [E, F, K].
extern "C" int tm_moe_up_act_mfma(const void* x, int ldx, const int* slot_pair, int top, const void* W, void* act, const int* tiles,
                                  const int* n_tiles, int max_tiles, int tile_rows, int K, int F, hipStream_t stream) {
    if (tile_rows != 32 && tile_rows != 64 && tile_rows != 128) return TM_ERR_ARG;
    if (!x || !slot_pair || !W || !act || !tiles || !n_tiles || top <= 0 || K <= 0 || F <= 0 || ldx < K || max_tiles < 0 || K % 8 ||
        ldx % 8 || !gm_aligned(x) || !gm_aligned(W))
        return TM_ERR_ARG;
    if (max_tiles == 0) return TM_OK;
    dim3 grid(max_tiles, (F + GM_BN - 1) / GM_BN);
    if (grid.y > 65535) return TM_ERR_ARG;
#define GM_GO(RT_, BK_, BN_)                                                                                                             \
    grouped_mfma_kernel<RT_, GM_RELU2, BK_, BN_><<<dim3(max_tiles, (F + BN_ - 1) / BN_), 256, 0, stream>>>((const bf16_t*)x, ldx, 0, slot_pair, top, (const bf16_t*)W, act, F, \
                                                                 0, nullptr, 0, tiles, n_tiles, 0, K, F, 0, 0, nullptr, nullptr, nullptr)
    // tiles of 128 rows take 128 columns a block (a piece of A read from LDS meets two column groups) where that still
    // leaves two blocks a CU to choose from
    if (tile_rows == 32) GM_GO(2, 128, GM_BN); else if (tile_rows == 64) GM_GO(4, GM_BK, GM_BN);
    else if ((long long)max_tiles * ((F + 127) / 128) >= 512) GM_GO(8, GM_BK, 128); else GM_GO(8, GM_BK, GM_BN);
#undef GM_GO
    TM_CHECK_LAUNCH();
    return TM_OK;
}

extern "C" int tm_moe_down_mfma(const void* act, const void* W, float* part, const int* tiles, const int* n_tiles, int max_tiles,
                                int tile_rows, int F, int N, hipStream_t stream) {
    if (tile_rows != 32 && tile_rows != 64 && tile_rows != 128) return TM_ERR_ARG;
    if (!act || !W || !part || !tiles || !n_tiles || F <= 0 || N <= 0 || max_tiles < 0 || F % 8 || !gm_aligned(act) || !gm_aligned(W))
        return TM_ERR_ARG;
    if (max_tiles == 0) return TM_OK;
    dim3 grid(max_tiles, (N + GM_BN - 1) / GM_BN);
    if (grid.y > 65535) return TM_ERR_ARG;
#define GM_GO(RT_, BK_, BN_)                                                                                                              \
    grouped_mfma_kernel<RT_, GM_STORE_F32, BK_, BN_><<<dim3(max_tiles, (N + BN_ - 1) / BN_), 256, 0, stream>>>((const bf16_t*)act, F, 0, nullptr, 1, (const bf16_t*)W, part, N, 0, \
                                                                     nullptr, 0, tiles, n_tiles, 0, F, N, 0, 0, nullptr, nullptr, nullptr)
    // tiles of 128 rows take 128 columns a block (a piece of A read from LDS meets two column groups) where that still
    // leaves two blocks a CU to choose from
    if (tile_rows == 32) GM_GO(2, 128, GM_BN); else if (tile_rows == 64) GM_GO(4, GM_BK, GM_BN);
    else if ((long long)max_tiles * ((N + 127) / 128) >= 512) GM_GO(8, GM_BK, 128); else GM_GO(8, GM_BK, GM_BN);
#undef GM_GO
    TM_CHECK_LAUNCH();
    return TM_OK;
}
