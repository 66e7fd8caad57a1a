// A feed-forward of many small experts of which every token uses a few, chosen by a table row of its token id or by a
// router.
//
//   pair p = (token t = p / top, choice k = p % top) goes to expert e(p) = table[id[t] * top + k]  (ids null: table[p])
//   tm_moe_router    z [T, E] (32-bit router outputs) -> s = softmax(z); the `top` largest of s + correction are chosen
//                    (ties: the lower index), chosen[t, k] in descending order, weight[t, k] = s / (sum of the chosen s + 1e-20);
//                    with `over_chosen` the `top` largest z are chosen and the weights are the softmax over the chosen z only
//   tm_moe_route     sorts the pairs by expert: slot_pair[slot] = p, pair_slot[p] = slot, and cuts every expert's run of
//                    slots into tiles of `tile_rows` rows: tiles[i] = (expert, first slot, rows), n_tiles[0] = their number
//   tm_moe_gate_up   act[slot] = silu(x[t] . Wg[e]^T) * (x[t] . Wu[e]^T)          W [E, 2F, K]: gate rows, then up rows
//   tm_moe_down      part[slot] = act[slot] . Wd[e]^T  (32-bit)                    Wd [E, N, F]
//   tm_moe_combine   y[t] = sum_k weight * part[pair_slot[t * top + k]], k ascending, rounded once
//   tm_moe_up_act    act[slot] = relu(x[t] . Wu[e]^T)^2                           W [E, F, K]: experts without a gate
//   tm_moe_combine_weighted   y[t] = sum_k weight[t, k] * (part[slot of the pair], or x[t] for a pair that has no slot: an
//                    expert >= `real` stands for the input itself) + sigmoid(shared_gate[t]) * shared[t]
//
// All of it runs from device data (no count crosses to the host), so a step can be recorded into a graph. Which slot a
// pair gets inside its expert's run may differ from run to run (the cursor is an atomic counter); a row's result does not
// depend on its slot: every element is summed over k in ascending order by one thread.
#include "common.h"
#include "api.h"

#define MR_THREADS 1024
#define MOE_MAX_EXPERTS 1024

__global__ __launch_bounds__(MR_THREADS) void moe_route_kernel(const int* __restrict__ ids, const int* __restrict__ table, int T,
                                                               int top, int E, int real, int tile_rows, int* __restrict__ slot_pair,
                                                               int* __restrict__ pair_slot, int* __restrict__ tiles,
                                                               int* __restrict__ n_tiles) {
    __shared__ int cnt[MOE_MAX_EXPERTS];
    __shared__ int off[MOE_MAX_EXPERTS + 1];
    const int P = T * top;
    for (int e = threadIdx.x; e < E; e += MR_THREADS) cnt[e] = 0;
    __syncthreads();
    for (int p = threadIdx.x; p < P; p += MR_THREADS) {
        const int e = ids ? table[(size_t)ids[p / top] * top + p % top] : table[p];
        if (e < real) atomicAdd(&cnt[e], 1);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int at = 0, n = 0;
        for (int e = 0; e < real; ++e) {
            off[e] = at;
            for (int r = 0; r < cnt[e]; r += tile_rows) {
                tiles[3 * n] = e;
                tiles[3 * n + 1] = at + r;
                tiles[3 * n + 2] = min(tile_rows, cnt[e] - r);
                ++n;
            }
            at += cnt[e];
            cnt[e] = 0;
        }
        off[real] = at;
        n_tiles[0] = n;
    }
    __syncthreads();
    for (int p = threadIdx.x; p < P; p += MR_THREADS) {
        const int e = ids ? table[(size_t)ids[p / top] * top + p % top] : table[p];
        if (e >= real) {                        // an expert without matrices: the pair has no slot
            pair_slot[p] = -1;
            continue;
        }
        const int slot = off[e] + atomicAdd(&cnt[e], 1);
        slot_pair[slot] = p;
        pair_slot[p] = slot;
    }
}

// ids null: table is [T, top], the experts of every pair as a router chose them. real: experts real .. E - 1 have no matrices.
extern "C" int tm_moe_route_chosen(const int* ids, const int* table, int T, int top, int E, int real, int tile_rows, int* slot_pair,
                                   int* pair_slot, int* tiles, int* n_tiles, hipStream_t stream) {
    if (!table || !slot_pair || !pair_slot || !tiles || !n_tiles || T < 0 || top <= 0 || E <= 0 || E > MOE_MAX_EXPERTS || real < 0 ||
        real > E || tile_rows <= 0 || (long long)T * top > 0x3fffffffLL)
        return TM_ERR_ARG;
    moe_route_kernel<<<1, MR_THREADS, 0, stream>>>(ids, table, T, top, E, real, tile_rows, slot_pair, pair_slot, tiles, n_tiles);
    TM_CHECK_LAUNCH();
    return TM_OK;
}

extern "C" int tm_moe_route(const int* ids, const int* table, int T, int top, int E, int tile_rows, int* slot_pair, int* pair_slot,
                            int* tiles, int* n_tiles, hipStream_t stream) {
    if (!ids || !table || !slot_pair || !pair_slot || !tiles || !n_tiles || T < 0 || top <= 0 || E <= 0 || E > MOE_MAX_EXPERTS ||
        tile_rows <= 0 || (long long)T * top > 0x3fffffffLL)
        return TM_ERR_ARG;
    moe_route_kernel<<<1, MR_THREADS, 0, stream>>>(ids, table, T, top, E, E, tile_rows, slot_pair, pair_slot, tiles, n_tiles);
    TM_CHECK_LAUNCH();
    return TM_OK;
}

// ------------------------------------------------------------------------------------------------ grouped products

#define MG_TM 32            // rows of a tile (tile_rows of the route)
#define MG_TN 64
#define MG_TK 16

// MODE 1 (gated): C[slot, n] = silu(a . W[e][n]) * (a . W[e][F + n]), a = A[slot_pair[slot] / top]; C of type T.
// MODE 2         : C[slot, n] = relu(a . W[e][n])^2, the same a; C of type T.
// MODE 0         : C[slot, n] = A[slot] . W[e][n]; C float32.
template <typename T, int MODE>
__global__ __launch_bounds__(256) void moe_product_kernel(const T* __restrict__ A, int lda, const int* __restrict__ slot_pair, int top,
                                                          const T* __restrict__ W, void* __restrict__ Cv, int ldc,
                                                          const int* __restrict__ tiles, const int* __restrict__ n_tiles, int K,
                                                          int N) {
    constexpr bool GATED = MODE == 1, GATHER = MODE != 0;
    if ((int)blockIdx.x >= n_tiles[0]) return;
    __shared__ float As[MG_TM][MG_TK + 1];
    __shared__ float Bs[GATED ? 2 : 1][MG_TK][MG_TN + 1];
    __shared__ int src[MG_TM];
    const int e = tiles[3 * blockIdx.x], slot0 = tiles[3 * blockIdx.x + 1], rows = tiles[3 * blockIdx.x + 2];
    const int n0 = blockIdx.y * MG_TN;
    const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
    const T* We = W + (size_t)e * (GATED ? 2 : 1) * N * K;
    if (threadIdx.x < MG_TM)
        src[threadIdx.x] = threadIdx.x < rows ? (GATHER ? slot_pair[slot0 + threadIdx.x] / top : slot0 + (int)threadIdx.x) : -1;
    __syncthreads();
    float acc[2][4] = {}, acu[2][4] = {};
    for (int k0 = 0; k0 < K; k0 += MG_TK) {
        for (int i = threadIdx.x; i < MG_TM * MG_TK; i += 256) {
            const int r = i / MG_TK, k = i % MG_TK;
            As[r][k] = (src[r] >= 0 && k0 + k < K) ? Elem<T>::load(A + (size_t)src[r] * lda + k0 + k) : 0.f;
        }
        for (int i = threadIdx.x; i < MG_TK * MG_TN; i += 256) {
            const int n = i / MG_TK, k = i % MG_TK;
            const bool in = n0 + n < N && k0 + k < K;
            Bs[0][k][n] = in ? Elem<T>::load(We + (size_t)(n0 + n) * K + k0 + k) : 0.f;
            if (GATED) Bs[1][k][n] = in ? Elem<T>::load(We + (size_t)(N + n0 + n) * K + k0 + k) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < MG_TK; ++k) {
            const float a0 = As[ty * 2][k], a1 = As[ty * 2 + 1][k];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float b = Bs[0][k][tx * 4 + j];
                acc[0][j] += a0 * b;
                acc[1][j] += a1 * b;
                if (GATED) {
                    const float u = Bs[1][k][tx * 4 + j];
                    acu[0][j] += a0 * u;
                    acu[1][j] += a1 * u;
                }
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int r = ty * 2 + i;
        if (r >= rows) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n >= N) continue;
            if (GATED) {
                const float g = acc[i][j], u = acu[i][j];
                Elem<T>::store((T*)Cv + (size_t)(slot0 + r) * ldc + n, g / (1.0f + __expf(-g)) * u);
            } else if (MODE == 2) {
                const float a = fmaxf(acc[i][j], 0.f);
                Elem<T>::store((T*)Cv + (size_t)(slot0 + r) * ldc + n, a * a);
            } else {
                ((float*)Cv)[(size_t)(slot0 + r) * ldc + n] = acc[i][j];
            }
        }
    }
}

extern "C" int tm_moe_gate_up(const void* x, int ldx, const int* slot_pair, int top, const void* W, void* act, const int* tiles,
                              const int* n_tiles, int max_tiles, int K, int F, int dtype, hipStream_t stream) {
    if (!x || !slot_pair || !W || !act || !tiles || !n_tiles || top <= 0 || K <= 0 || F <= 0 || ldx < K || max_tiles < 0) return TM_ERR_ARG;
    if (dtype != TM_F32 && dtype != TM_BF16) return TM_ERR_ARG;
    if (max_tiles == 0) return TM_OK;
    dim3 grid(max_tiles, (F + MG_TN - 1) / MG_TN);
    if (grid.y > 65535) return TM_ERR_ARG;
    if (dtype == TM_F32)
        moe_product_kernel<float, 1><<<grid, 256, 0, stream>>>((const float*)x, ldx, slot_pair, top, (const float*)W, act, F, tiles,
                                                                  n_tiles, K, F);
    else
        moe_product_kernel<bf16_t, 1><<<grid, 256, 0, stream>>>((const bf16_t*)x, ldx, slot_pair, top, (const bf16_t*)W, act, F, tiles,
                                                                   n_tiles, K, F);
    TM_CHECK_LAUNCH();
    return TM_OK;
}

extern "C" int tm_moe_up_act(const void* x, int ldx, const int* slot_pair, int top, const void* W, void* act, const int* tiles,
                             const int* n_tiles, int max_tiles, int K, int F, int dtype, hipStream_t stream) {
    if (!x || !slot_pair || !W || !act || !tiles || !n_tiles || top <= 0 || K <= 0 || F <= 0 || ldx < K || max_tiles < 0) return TM_ERR_ARG;
    if (dtype != TM_F32 && dtype != TM_BF16) return TM_ERR_ARG;
    if (max_tiles == 0) return TM_OK;
    dim3 grid(max_tiles, (F + MG_TN - 1) / MG_TN);
    if (grid.y > 65535) return TM_ERR_ARG;
    if (dtype == TM_F32)
        moe_product_kernel<float, 2><<<grid, 256, 0, stream>>>((const float*)x, ldx, slot_pair, top, (const float*)W, act, F, tiles,
                                                               n_tiles, K, F);
    else
        moe_product_kernel<bf16_t, 2><<<grid, 256, 0, stream>>>((const bf16_t*)x, ldx, slot_pair, top, (const bf16_t*)W, act, F, tiles,
                                                                n_tiles, K, F);
    TM_CHECK_LAUNCH();
    return TM_OK;
}

extern "C" int tm_moe_down(const void* act, const void* W, float* part, const int* tiles, const int* n_tiles, int max_tiles, int F,
                           int N, int dtype, hipStream_t stream) {
    if (!act || !W || !part || !tiles || !n_tiles || F <= 0 || N <= 0 || max_tiles < 0) return TM_ERR_ARG;
    if (dtype != TM_F32 && dtype != TM_BF16) return TM_ERR_ARG;
    if (max_tiles == 0) return TM_OK;
    dim3 grid(max_tiles, (N + MG_TN - 1) / MG_TN);
    if (grid.y > 65535) return TM_ERR_ARG;
    if (dtype == TM_F32)
        moe_product_kernel<float, 0><<<grid, 256, 0, stream>>>((const float*)act, F, nullptr, 1, (const float*)W, part, N, tiles,
                                                                   n_tiles, F, N);
    else
        moe_product_kernel<bf16_t, 0><<<grid, 256, 0, stream>>>((const bf16_t*)act, F, nullptr, 1, (const bf16_t*)W, part, N, tiles,
                                                                    n_tiles, F, N);
    TM_CHECK_LAUNCH();
    return TM_OK;
}

template <typename T>
__global__ __launch_bounds__(256) void moe_combine_kernel(const float* __restrict__ part, const int* __restrict__ pair_slot,
                                                          T* __restrict__ y, int top, float weight, int N) {
    const int t = blockIdx.x;
    for (int c = threadIdx.x; c < N; c += 256) {
        float s = 0.f;
        for (int k = 0; k < top; ++k) s += weight * part[(size_t)pair_slot[t * top + k] * N + c];
        Elem<T>::store(y + (size_t)t * N + c, s);
    }
}

extern "C" int tm_moe_combine(const float* part, const int* pair_slot, void* y, int T, int top, float weight, int N, int dtype,
                              hipStream_t stream) {
    if (!part || !pair_slot || !y || T < 0 || top <= 0 || N <= 0) return TM_ERR_ARG;
    if (dtype != TM_F32 && dtype != TM_BF16) return TM_ERR_ARG;
    if (T == 0) return TM_OK;
    if (dtype == TM_F32)
        moe_combine_kernel<float><<<T, 256, 0, stream>>>(part, pair_slot, (float*)y, top, weight, N);
    else
        moe_combine_kernel<bf16_t><<<T, 256, 0, stream>>>(part, pair_slot, (bf16_t*)y, top, weight, N);
    TM_CHECK_LAUNCH();
    return TM_OK;
}

// ------------------------------------------------------------------------------------------------ a router

// A wavefront a token; lane l holds experts l, l + 64, ... (RT_MAX_PER_LANE of them: 1, 4 or 16 by the number of experts).
// Everything is 32-bit.
template <int RT_MAX_PER_LANE>
__global__ __launch_bounds__(TM_WAVE) void moe_router_kernel(const float* __restrict__ z, int ldz, const float* __restrict__ correction,
                                                             int E, int top, int* __restrict__ chosen, float* __restrict__ weight,
                                                             int over_chosen) {
    const int t = blockIdx.x, lane = threadIdx.x;
    const float* zr = z + (size_t)t * ldz;
    float s[RT_MAX_PER_LANE], c[RT_MAX_PER_LANE];
    float m = -INFINITY;
#pragma unroll
    for (int i = 0; i < RT_MAX_PER_LANE; ++i) {
        const int e = lane + i * TM_WAVE;
        s[i] = e < E ? zr[e] : -INFINITY;
        m = fmaxf(m, s[i]);
    }
    m = wave_max(m);
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < RT_MAX_PER_LANE; ++i) {
        const int e = lane + i * TM_WAVE;
        c[i] = s[i];                             // the output itself: what `over_chosen` ranks
        s[i] = e < E ? expf(s[i] - m) : 0.f;     // m is the largest output, which is chosen first: these are the chosen ones' terms too
        sum += s[i];
    }
    sum = wave_sum(sum);
    if (!over_chosen) {
#pragma unroll
        for (int i = 0; i < RT_MAX_PER_LANE; ++i) {
            const int e = lane + i * TM_WAVE;
            s[i] = s[i] / sum;
            c[i] = e < E ? s[i] + (correction ? correction[e] : 0.f) : -INFINITY;
        }
    }
    float total = 0.f;
    for (int k = 0; k < top; ++k) {
        float best = -INFINITY;
        int at = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < RT_MAX_PER_LANE; ++i)
            if (c[i] > best) best = c[i], at = lane + i * TM_WAVE;      // within a lane e ascends: the first of equals stays
        const float top_v = wave_max(best);
        int cand = (best == top_v) ? at : 0x7fffffff;
#pragma unroll
        for (int o = TM_WAVE / 2; o > 0; o >>= 1) cand = min(cand, __shfl_xor(cand, o, TM_WAVE));
        float sc = 0.f;
#pragma unroll
        for (int i = 0; i < RT_MAX_PER_LANE; ++i)
            if (lane + i * TM_WAVE == cand) sc = s[i], c[i] = -INFINITY;
        sc = wave_sum(sc);                   // one lane holds it, the others 0
        total += sc;
        if (lane == 0) {
            chosen[(size_t)t * top + k] = cand;
            weight[(size_t)t * top + k] = sc;
        }
    }
    __syncthreads();                         // lane 0's scores, seen by the lanes that scale them
    const float inv = over_chosen ? 1.f / total : 1.f / (total + 1e-20f);
    for (int k = lane; k < top; k += TM_WAVE) weight[(size_t)t * top + k] *= inv;
}

extern "C" int tm_moe_router(const float* z, int ldz, const float* correction, int T, int E, int top, int* chosen, float* weight,
                             int over_chosen, hipStream_t stream) {
    if (!z || !chosen || !weight || T < 0 || E <= 0 || E > MOE_MAX_EXPERTS || top <= 0 || top > E || ldz < E) return TM_ERR_ARG;
    if (T == 0) return TM_OK;
    if (over_chosen && correction) return TM_ERR_ARG;
    if (E <= TM_WAVE) moe_router_kernel<1><<<T, TM_WAVE, 0, stream>>>(z, ldz, correction, E, top, chosen, weight, over_chosen);
    else if (E <= 4 * TM_WAVE) moe_router_kernel<4><<<T, TM_WAVE, 0, stream>>>(z, ldz, correction, E, top, chosen, weight, over_chosen);
    else moe_router_kernel<MOE_MAX_EXPERTS / TM_WAVE><<<T, TM_WAVE, 0, stream>>>(z, ldz, correction, E, top, chosen, weight, over_chosen);
    TM_CHECK_LAUNCH();
    return TM_OK;
}

// A block is a token and 256 columns: few tokens still make many blocks, and a thread's loads (the pair's slot, then its row)
// wait once, not once a column.
template <typename T>
__global__ __launch_bounds__(256) void moe_combine_weighted_kernel(const float* __restrict__ part, const int* __restrict__ pair_slot,
                                                                   const float* __restrict__ weight, const T* __restrict__ x, int ldx,
                                                                   const float* __restrict__ shared, const float* __restrict__ shared_gate,
                                                                   int ldg, T* __restrict__ y, int top, int N) {
    const int t = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
    if (c >= N) return;
    const float sg = (shared && shared_gate) ? 1.f / (1.f + expf(-shared_gate[(size_t)t * ldg])) : 1.f;
    float s = 0.f;
    for (int k = 0; k < top; ++k) {
        const int slot = pair_slot[t * top + k];
        const float v = slot >= 0 ? part[(size_t)slot * N + c] : Elem<T>::load(x + (size_t)t * ldx + c);
        s += weight[(size_t)t * top + k] * v;
    }
    if (shared) s += sg * shared[(size_t)t * N + c];
    Elem<T>::store(y + (size_t)t * N + c, s);
}

// shared (float32 [T, N]) and shared_gate (float32, one number a token, rows ldg apart) may be null.
extern "C" int tm_moe_combine_weighted(const float* part, const int* pair_slot, const float* weight, const void* x, int ldx,
                                       const float* shared, const float* shared_gate, int ldg, void* y, int T, int top, int N, int dtype,
                                       hipStream_t stream) {
    if (!part || !pair_slot || !weight || !x || !y || T < 0 || top <= 0 || N <= 0 || ldx < N || (shared_gate && ldg < 1)) return TM_ERR_ARG;
    if (dtype != TM_F32 && dtype != TM_BF16) return TM_ERR_ARG;
    if (T == 0) return TM_OK;
    const dim3 grid(T, (N + 255) / 256);
    if (grid.y > 65535) return TM_ERR_ARG;
    if (dtype == TM_F32)
        moe_combine_weighted_kernel<float><<<grid, 256, 0, stream>>>(part, pair_slot, weight, (const float*)x, ldx, shared, shared_gate, ldg,
                                                                  (float*)y, top, N);
    else
        moe_combine_weighted_kernel<bf16_t><<<grid, 256, 0, stream>>>(part, pair_slot, weight, (const bf16_t*)x, ldx, shared, shared_gate, ldg,
                                                                   (bf16_t*)y, top, N);
    TM_CHECK_LAUNCH();
    return TM_OK;
}
