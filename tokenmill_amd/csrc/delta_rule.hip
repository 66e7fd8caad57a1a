// The gated delta rule: a recurrent mixer whose state per request and head is a matrix S [D, Dv] of 32-bit floats,
//
//   S <- g_t S;   u_t = beta_t (v_t - S^T k_t);   S <- S + k_t u_t^T;   o_t = S^T q_t
//
// with one decay g_t in (0, 1) and one step size beta_t in (0, 1) per token and head, unit vectors q_t (times D^-1/2) and
// k_t, advanced token by token in the order of the positions, within a step's portion and from one step to the next (the
// state lives in the request's state slot between steps). H value heads share G <= H query/key heads (head h reads q/k
// head h / (H / G)).
//
//   tm_delta_prepare     per token: the short causal convolution over time of the q | k | v channels of the stacked
//                        projection (the rows before the step's first from the request's convolution state), silu, the two
//                        unit norms, k . q, beta = sigmoid(b) and g = exp(-exp(A_log) softplus(a + dt_bias)); all written
//                        as one 32-bit row [q (G D) | k (G D) | v (H Dv) | beta (H) | g (H) | k.q (G)]
//   tm_delta_conv_state  then the convolution state becomes the last taps - 1 projection rows the request has seen
//   tm_delta_scan        the recurrence over those rows; writes o in 32-bit
//   tm_delta_combine     chains the segments of a long portion (each scanned from zero and from the identity) into every
//                        segment's true start state
//   tm_pair_norm_mean    out = (rms_norm(a; wa) + rms_norm(b; wb)) / 2: two sublayers side by side, each normed over the width
//
// The columns of S are independent of each other: with d_k = S^T k and d_q = S^T q taken on the state as the token finds it,
//   u = beta (v - g d_k),   o = g d_q + u (k . q),   S <- g S + k u^T
// is the same recurrence with one round of sums a token instead of two. The scan is dealt over (request, head, 16 columns)
// blocks; a lane keeps a sixteenth of a column's D rows in registers, and a column's sixteen partial sums are added in a fixed
// order; a request's rows reach its block through LDS, a tile of tokens at a time. A token's result depends on its
// request's state and tokens only, never on the step's other rows; how the prompt was cut changes it by 32-bit rounding at
// most (a long portion is scanned in segments, whose sums are ordered otherwise than the plain chain's). Everything that
// enters the recurrence is 32-bit.
#include "common.h"
#include "api.h"

#define DP_THREADS 256
#define DR_MAX_TAPS 16

__device__ __forceinline__ float silu_f32(float z) { return z / (1.0f + expf(-z)); }

// A channel of a token behind the convolution and silu: `taps` rows ending at the token, those before the step's first row from
// the request's convolution state.
template <typename T>
__device__ __forceinline__ float delta_conv_channel(const T* __restrict__ proj, int ld, const T* __restrict__ conv_w,
                                                    const T* __restrict__ st, int C, int taps, int first, int i, int c) {
    float acc = 0.f;
    for (int j = 0; j < taps; ++j) {
        const int at = i - (taps - 1) + j;                   // < 0: before this step's rows, in the state
        const float x = at >= 0 ? Elem<T>::load(proj + (size_t)(first + at) * ld + c)
                                : Elem<T>::load(st + (size_t)(taps - 1 + at) * C + c);
        acc += Elem<T>::load(conv_w + (size_t)c * taps + j) * x;
    }
    return silu_f32(acc);
}

// grid (T, G + ceil(H Dv / 256)); a block is a token and either one q/k head (a thread a channel of q and of k; the head's three
// sums by the block's fixed tree) or 256 channels of v; the first block of v also makes the token's step sizes and decays. Few
// tokens still make many blocks, and a thread's loads are a handful.
template <typename T>
__global__ __launch_bounds__(DP_THREADS) void delta_prepare_kernel(const T* __restrict__ proj, int ld, const T* __restrict__ conv_w,
                                                                   const T* __restrict__ conv_state, const float* __restrict__ ba,
                                                                   int ldba, const float* __restrict__ a_log,
                                                                   const float* __restrict__ dt_bias, const int* __restrict__ cu,
                                                                   const int* __restrict__ slots, const int* __restrict__ seq_of_token,
                                                                   float* __restrict__ out, int ldo, int H, int G, int D, int Dv,
                                                                   int taps, float unit_eps) {
    __shared__ float red[DP_THREADS / TM_WAVE];
    const int t = blockIdx.x, unit = blockIdx.y;
    const int s = seq_of_token[t];
    const int first = cu[s], i = t - first;                  // the token's place among its request's rows of this step
    const int C = 2 * G * D + H * Dv;
    const T* st = conv_state + (size_t)slots[s] * (taps - 1) * C;
    float* o = out + (size_t)t * ldo;
    if (unit < G) {                                          // D <= 256: a thread has one channel of the head's q and one of its k
        const int c = threadIdx.x;
        const bool in = c < D;
        const float q = in ? delta_conv_channel<T>(proj, ld, conv_w, st, C, taps, first, i, unit * D + c) : 0.f;
        const float k = in ? delta_conv_channel<T>(proj, ld, conv_w, st, C, taps, first, i, G * D + unit * D + c) : 0.f;
        const float sq = block_sum<DP_THREADS>(q * q, red), sk = block_sum<DP_THREADS>(k * k, red), qk = block_sum<DP_THREADS>(q * k, red);
        const float iq = (1.0f / sqrtf((float)D)) / sqrtf(sq + unit_eps), ik = 1.0f / sqrtf(sk + unit_eps);
        if (in) {
            o[unit * D + c] = q * iq;
            o[G * D + unit * D + c] = k * ik;
        }
        if (c == 0) o[C + 2 * H + unit] = qk * iq * ik;
        return;
    }
    const int c = 2 * G * D + (unit - G) * DP_THREADS + threadIdx.x;
    if (c < C) o[c] = delta_conv_channel<T>(proj, ld, conv_w, st, C, taps, first, i, c);
    if (unit == G)
        for (int h = threadIdx.x; h < H; h += DP_THREADS) {
            const float b = ba[(size_t)t * ldba + h];
            const float a = ba[(size_t)t * ldba + H + h] + dt_bias[h];
            const float sp = fmaxf(a, 0.f) + log1pf(expf(-fabsf(a)));            // softplus
            o[C + h] = 1.0f / (1.0f + expf(-b));
            o[C + H + h] = expf(-expf(a_log[h]) * sp);
        }
}

extern "C" int tm_delta_prepare(const void* proj, int ld, const void* conv_w, const void* conv_state, const float* ba, int ldba,
                                const float* a_log, const float* dt_bias, const int* cu_q_lens, const int* state_slots,
                                const int* seq_of_token, float* out, int ldo, int T, int H, int G, int D, int Dv, int taps,
                                float unit_eps, int dtype, hipStream_t stream) {
    if (!proj || !conv_w || !ba || !a_log || !dt_bias || !cu_q_lens || !state_slots || !seq_of_token || !out || T < 0 || H <= 0 ||
        G <= 0 || H % G || D <= 0 || D > DP_THREADS || Dv <= 0 || taps < 1 || taps > DR_MAX_TAPS || (taps > 1 && !conv_state) ||
        ldba < 2 * H || !(unit_eps > 0.f))
        return TM_ERR_ARG;
    const long long C = 2LL * G * D + (long long)H * Dv;
    const long long units = G + ((long long)H * Dv + DP_THREADS - 1) / DP_THREADS;
    if (ld < C || ldo < C + 2 * H + G || units > 65535) return TM_ERR_ARG;
    if (dtype != TM_F32 && dtype != TM_BF16) return TM_ERR_ARG;
    if (T == 0) return TM_OK;
    const dim3 grid(T, (unsigned)units);
    if (dtype == TM_F32)
        delta_prepare_kernel<float><<<grid, DP_THREADS, 0, stream>>>((const float*)proj, ld, (const float*)conv_w, (const float*)conv_state,
                                                                     ba, ldba, a_log, dt_bias, cu_q_lens, state_slots, seq_of_token, out,
                                                                     ldo, H, G, D, Dv, taps, unit_eps);
    else
        delta_prepare_kernel<bf16_t><<<grid, DP_THREADS, 0, stream>>>((const bf16_t*)proj, ld, (const bf16_t*)conv_w,
                                                                      (const bf16_t*)conv_state, ba, ldba, a_log, dt_bias, cu_q_lens,
                                                                      state_slots, seq_of_token, out, ldo, H, G, D, Dv, taps, unit_eps);
    TM_CHECK_LAUNCH();
    return TM_OK;
}

// grid (S, channel blocks): a thread reads all it needs of its channel before it writes.
template <typename T>
__global__ __launch_bounds__(DP_THREADS) void delta_conv_state_kernel(const T* __restrict__ proj, int ld, T* __restrict__ state,
                                                                      const int* __restrict__ cu, const int* __restrict__ slots, int C,
                                                                      int taps) {
    const int s = blockIdx.x;
    const int first = cu[s], n = cu[s + 1] - first;
    if (n <= 0) return;
    T* st = state + (size_t)slots[s] * (taps - 1) * C;
    const int keep = taps - 1;
    for (int c = blockIdx.y * DP_THREADS + threadIdx.x; c < C; c += gridDim.y * DP_THREADS) {
        T next[DR_MAX_TAPS - 1];
        for (int k = 0; k < keep; ++k) {
            const int at = n - keep + k;                     // the row that becomes state row k
            next[k] = at >= 0 ? proj[(size_t)(first + at) * ld + c] : st[(size_t)(keep + at) * C + c];
        }
        for (int k = 0; k < keep; ++k) st[(size_t)k * C + c] = next[k];
    }
}

extern "C" int tm_delta_conv_state(const void* proj, int ld, void* state, const int* cu_q_lens, const int* state_slots, int S, int C,
                                   int taps, int dtype, hipStream_t stream) {
    if (!proj || S < 0 || C <= 0 || ld < C || taps < 1 || taps > DR_MAX_TAPS || (taps > 1 && !state) || !cu_q_lens || !state_slots)
        return TM_ERR_ARG;
    if (dtype != TM_F32 && dtype != TM_BF16) return TM_ERR_ARG;
    if (S == 0 || taps == 1) return TM_OK;
    const int by = (C + DP_THREADS - 1) / DP_THREADS;
    dim3 grid(S, by > 8 ? 8 : by);
    if (dtype == TM_F32)
        delta_conv_state_kernel<float><<<grid, DP_THREADS, 0, stream>>>((const float*)proj, ld, (float*)state, cu_q_lens, state_slots, C, taps);
    else
        delta_conv_state_kernel<bf16_t><<<grid, DP_THREADS, 0, stream>>>((const bf16_t*)proj, ld, (bf16_t*)state, cu_q_lens, state_slots, C, taps);
    TM_CHECK_LAUNCH();
    return TM_OK;
}

// ------------------------------------------------------------------------------------------------ the recurrence

#define DR_PARTS 16                         // lanes that share a column's rows: a row of 16 lanes, whose sum the data-parallel moves give
#define DR_COLS 16                          // columns of a block (four wavefronts with four columns each)
#define DR_THREADS 256
#define DR_TT 16                            // tokens of a tile

// The sum over the 16 lanes of a row, in every one of them: neighbours, pairs, the mirrored half row, the mirrored row.
__device__ __forceinline__ float row16_sum(float v) {
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true));     // quad_perm [1, 0, 3, 2]
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true));     // quad_perm [2, 3, 0, 1]
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true));    // row_half_mirror
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, true));    // row_mirror
    return v;
}

// grid (ceil(Dv / 16), H, S); a block is four wavefronts and 16 columns of S. Sixteen lanes share a column's rows: lane =
// column * 16 + part; part p keeps rows p * R .. p * R + R - 1 of its column, R = ceil(D / 16) <= RMAX, so a token costs a lane
// 3 R multiply-adds and the chain from token to token is short. The request's rows come through LDS in tiles of 16 tokens, each
// token's [q | k | beta g k.q . | v of the block's columns] (W = 2 D + 20 floats): the block's threads fetch a tile together,
// consecutive threads consecutive floats, into registers while the tile before is worked on (CPM: floats of a token a thread
// fetches at most), and put it down in the other of two buffers. VEC: R is a multiple of 4, so a lane reads its q and k from
// LDS as float4. o null: only the states are wanted. use_v 0: the values count as zero and the state's Dv columns need not be the
// rows' row_dv (a scan from the identity gives the product of the tokens' transitions g (I - beta k k^T)).
template <int RMAX, int CPM, bool VEC>
__global__ __launch_bounds__(DR_THREADS) void delta_scan_kernel(const float* __restrict__ rows, int ld, float* __restrict__ o,
                                                               float* __restrict__ state, const int* __restrict__ cu_q_lens,
                                                               const int* __restrict__ state_slots, int H, int G, int D, int Dv,
                                                               int row_dv, int use_v) {
    extern __shared__ __align__(16) float tile_s[];                       // [2][DR_TT][W]
    const int tid = threadIdx.x, part = tid % DR_PARTS, mine = tid / DR_PARTS;
    const int e = blockIdx.x * DR_COLS + mine;
    const int h = blockIdx.y, s = blockIdx.z;
    const int g = h / (H / G);
    const int R = (D + DR_PARTS - 1) / DR_PARTS;
    const int d0 = part * R;
    const bool col = e < Dv;
    const int t0 = cu_q_lens[s], t1 = cu_q_lens[s + 1];
    if (t1 <= t0) return;                                                 // the whole block
    const int C = 2 * G * D + H * row_dv, W = 2 * D + 4 + DR_COLS;
    // where in a prepared row the floats come from that this thread fetches of every token (-1: none)
    int from[CPM];
#pragma unroll
    for (int j = 0; j < CPM; ++j) {
        const int c = tid + DR_THREADS * j;
        int at = -1;
        if (c < D) at = g * D + c;
        else if (c < 2 * D) at = G * D + g * D + (c - D);
        else if (c == 2 * D) at = C + h;
        else if (c == 2 * D + 1) at = C + H + h;
        else if (c == 2 * D + 2) at = C + 2 * H + g;
        else if (use_v && c >= 2 * D + 4 && c < W && blockIdx.x * DR_COLS + (c - 2 * D - 4) < Dv)
            at = 2 * G * D + h * row_dv + blockIdx.x * DR_COLS + (c - 2 * D - 4);
        from[j] = at;
    }
    float held[DR_TT * CPM];
    auto fetch = [&](int first) {
#pragma unroll
        for (int tt = 0; tt < DR_TT; ++tt)
#pragma unroll
            for (int j = 0; j < CPM; ++j)
                held[tt * CPM + j] = (from[j] >= 0 && first + tt < t1) ? rows[(size_t)(first + tt) * ld + from[j]] : 0.f;
    };
    float* st = state + (((size_t)state_slots[s] * H + h) * D) * Dv + (col ? e : 0);
    float S[RMAX];
#pragma unroll
    for (int i = 0; i < RMAX; ++i) S[i] = (col && i < R && d0 + i < D) ? st[(size_t)(d0 + i) * Dv] : 0.f;
    fetch(t0);
    int which = 0;
    for (int first = t0; first < t1; first += DR_TT) {
        float* cur = tile_s + which * DR_TT * W;
#pragma unroll
        for (int tt = 0; tt < DR_TT; ++tt)
#pragma unroll
            for (int j = 0; j < CPM; ++j) {
                const int c = tid + DR_THREADS * j;
                if (c < W) cur[tt * W + c] = held[tt * CPM + j];
            }
        // every wavefront is done with the tile before the last (this buffer's last use) when it comes here, so one barrier a
        // tile orders both the stores above against the reads below and the reads of two tiles ago against these stores
        __syncthreads();
        if (first + DR_TT < t1) fetch(first + DR_TT);                     // in flight while this tile is worked on
        const int n = min(DR_TT, t1 - first);
        float* out = o + ((size_t)first * H + h) * Dv + e;
        for (int tt = 0; tt < n; ++tt) {
            const float* row = cur + tt * W;
            float kk[RMAX];
            float dk = 0.f, dq = 0.f;
            if (VEC) {
#pragma unroll
                for (int i = 0; i < RMAX; i += 4)
                    if (i < R) {
                        const float4 q4 = *(const float4*)(row + d0 + i), k4 = *(const float4*)(row + D + d0 + i);
                        kk[i] = k4.x, kk[i + 1] = k4.y, kk[i + 2] = k4.z, kk[i + 3] = k4.w;
                        dk += S[i] * k4.x, dq += S[i] * q4.x;
                        dk += S[i + 1] * k4.y, dq += S[i + 1] * q4.y;
                        dk += S[i + 2] * k4.z, dq += S[i + 2] * q4.z;
                        dk += S[i + 3] * k4.w, dq += S[i + 3] * q4.w;
                    }
            } else {
#pragma unroll
                for (int i = 0; i < RMAX; ++i) {
                    const bool in = i < R && d0 + i < D;
                    kk[i] = in ? row[D + d0 + i] : 0.f;
                    if (in) {
                        dk += S[i] * kk[i];
                        dq += S[i] * row[d0 + i];
                    }
                }
            }
            dk = row16_sum(dk);
            dq = row16_sum(dq);
            const float beta = row[2 * D], decay = row[2 * D + 1], kq = row[2 * D + 2], v = row[2 * D + 4 + mine];
            const float u = beta * (v - decay * dk);
#pragma unroll
            for (int i = 0; i < RMAX; ++i)
                if (i < R) S[i] = decay * S[i] + kk[i] * u;
            if (o && col && part == 0) out[(size_t)tt * H * Dv] = decay * dq + u * kq;
        }
        which ^= 1;
    }
#pragma unroll
    for (int i = 0; i < RMAX; ++i)
        if (col && i < R && d0 + i < D) st[(size_t)(d0 + i) * Dv] = S[i];
}

extern "C" int tm_delta_scan(const float* rows, int ld, float* o, float* state, const int* cu_q_lens, const int* state_slots, int S,
                             int H, int G, int D, int Dv, int row_dv, int use_v, hipStream_t stream) {
    if (!rows || !state || !cu_q_lens || !state_slots || S < 0 || H <= 0 || G <= 0 || H % G || D <= 0 || D > 256 || Dv <= 0 ||
        row_dv <= 0 || (use_v && row_dv != Dv) || (o && !use_v) || H > 65535 || S > 65535 ||
        (long long)ld < 2LL * G * D + (long long)H * row_dv + 2 * H + G)
        return TM_ERR_ARG;
    if (S == 0) return TM_OK;
    const dim3 grid((Dv + DR_COLS - 1) / DR_COLS, H, S);
    const int W = 2 * D + 4 + DR_COLS;
    const size_t lds = (size_t)2 * DR_TT * W * sizeof(float);              // 68 KB at most
    const bool vec = D % (4 * DR_PARTS) == 0;
#define DR_GO(RM, CPM_)                                                                                                          \
    do {                                                                                                                         \
        auto kernel = vec ? delta_scan_kernel<RM, CPM_, true> : delta_scan_kernel<RM, CPM_, false>;                              \
        if (lds > 64 * 1024 && hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) \
            return TM_ERR_LAUNCH;                                                                                                \
        kernel<<<grid, DR_THREADS, lds, stream>>>(rows, ld, o, state, cu_q_lens, state_slots, H, G, D, Dv, row_dv, use_v);       \
    } while (0)
    if (D <= 64) DR_GO(4, 1);                       // W <= 148
    else if (D <= 128) DR_GO(8, 2);                 // W <= 276
    else DR_GO(16, 3);                              // W <= 532
#undef DR_GO
    TM_CHECK_LAUNCH();
    return TM_OK;
}

// A prompt in segments: the recurrence is linear in the state, S_end = M S_start + B over any run of tokens, with M the product
// of the tokens' transitions (a scan from the identity without values) and B what the run builds from a zero state. This chains
// the segments of every request: start[j] = S; S <- trans[j] S + local[j], from the request's own state, which becomes the last S.
// grid (ceil(Dv / 16), H, requests); a block keeps 16 columns of S in LDS. A thread owns one row d of the new S and NC of the 16
// columns (DP: D rounded up to 64, 128 or 256; 256 / DP groups of threads share the columns): it streams its row of M once,
// sixteen bytes at a time, against the columns it reads from LDS with all its wavefront; every sum over d' in ascending order.
template <int DP>
__global__ __launch_bounds__(DR_THREADS) void delta_combine_kernel(const float* __restrict__ trans, const float* __restrict__ local,
                                                                  float* __restrict__ start, float* __restrict__ state,
                                                                  const int* __restrict__ state_slots, const int* __restrict__ first_seg,
                                                                  int H, int D, int Dv) {
    extern __shared__ __align__(16) float col_s[];                        // [D][16]
    constexpr int NC = DR_COLS * DP / DR_THREADS;                         // columns of a thread: 4, 8 or 16
    const int d = threadIdx.x % DP, c0 = threadIdx.x / DP * NC;
    const int e0 = blockIdx.x * DR_COLS;
    const int h = blockIdx.y, s = blockIdx.z;
    float* st = state + (((size_t)state_slots[s] * H + h) * D) * Dv;
    for (int idx = threadIdx.x; idx < D * DR_COLS; idx += DR_THREADS) {
        const int dd = idx / DR_COLS, e = e0 + idx % DR_COLS;
        col_s[idx] = e < Dv ? st[(size_t)dd * Dv + e] : 0.f;
    }
    __syncthreads();
    for (int seg = first_seg[s]; seg < first_seg[s + 1]; ++seg) {
        const size_t at = ((size_t)seg * H + h) * D;
        for (int idx = threadIdx.x; idx < D * DR_COLS; idx += DR_THREADS) {
            const int dd = idx / DR_COLS, e = e0 + idx % DR_COLS;
            if (e < Dv) start[(at + dd) * Dv + e] = col_s[idx];
        }
        float acc[NC];
#pragma unroll
        for (int j = 0; j < NC; ++j) acc[j] = (d < D && e0 + c0 + j < Dv) ? local[(at + d) * Dv + e0 + c0 + j] : 0.f;
        if (d < D) {
            const float* m = trans + (at + d) * D;
            if (D % 4 == 0) {
#pragma unroll 4
                for (int k = 0; k < D; k += 4) {
                    const float4 m4 = *(const float4*)(m + k);
#pragma unroll
                    for (int j = 0; j < NC; ++j) {
                        acc[j] += m4.x * col_s[k * DR_COLS + c0 + j];
                        acc[j] += m4.y * col_s[(k + 1) * DR_COLS + c0 + j];
                        acc[j] += m4.z * col_s[(k + 2) * DR_COLS + c0 + j];
                        acc[j] += m4.w * col_s[(k + 3) * DR_COLS + c0 + j];
                    }
                }
            } else {
                for (int k = 0; k < D; ++k) {
                    const float mk = m[k];
#pragma unroll
                    for (int j = 0; j < NC; ++j) acc[j] += mk * col_s[k * DR_COLS + c0 + j];
                }
            }
        }
        __syncthreads();                                                  // every row has read the old columns
        if (d < D)
#pragma unroll
            for (int j = 0; j < NC; ++j) col_s[d * DR_COLS + c0 + j] = acc[j];
        __syncthreads();
    }
    for (int idx = threadIdx.x; idx < D * DR_COLS; idx += DR_THREADS) {
        const int dd = idx / DR_COLS, e = e0 + idx % DR_COLS;
        if (e < Dv) st[(size_t)dd * Dv + e] = col_s[idx];
    }
}

extern "C" int tm_delta_combine(const float* trans, const float* local, float* start, float* state, const int* state_slots,
                                const int* first_seg, int S, int H, int D, int Dv, hipStream_t stream) {
    if (!trans || !local || !start || !state || !state_slots || !first_seg || S < 0 || H <= 0 || H > 65535 || S > 65535 || D <= 0 ||
        D > DR_THREADS || Dv <= 0)
        return TM_ERR_ARG;
    if (S == 0) return TM_OK;
    const dim3 grid((Dv + DR_COLS - 1) / DR_COLS, H, S);
    const size_t lds = (size_t)D * DR_COLS * sizeof(float);
    if (D <= 64) delta_combine_kernel<64><<<grid, DR_THREADS, lds, stream>>>(trans, local, start, state, state_slots, first_seg, H, D, Dv);
    else if (D <= 128) delta_combine_kernel<128><<<grid, DR_THREADS, lds, stream>>>(trans, local, start, state, state_slots, first_seg, H, D, Dv);
    else delta_combine_kernel<256><<<grid, DR_THREADS, lds, stream>>>(trans, local, start, state, state_slots, first_seg, H, D, Dv);
    TM_CHECK_LAUNCH();
    return TM_OK;
}

// ------------------------------------------------------------------------------------------------ two sublayers side by side

// out[t] = (a[t] / rms(a[t]) * wa + b[t] / rms(b[t]) * wb) / 2 over the width W, statistics and sums in 32-bit, rounded once.
template <typename T>
__global__ __launch_bounds__(DP_THREADS) void pair_norm_mean_kernel(const T* __restrict__ a, const T* __restrict__ b,
                                                                    const float* __restrict__ wa, const float* __restrict__ wb,
                                                                    T* __restrict__ out, int W, float eps) {
    __shared__ float red[DP_THREADS / TM_WAVE];
    const size_t row = (size_t)blockIdx.x * W;
    float sa = 0.f, sb = 0.f;
    for (int c = threadIdx.x; c < W; c += DP_THREADS) {
        const float x = Elem<T>::load(a + row + c), y = Elem<T>::load(b + row + c);
        sa += x * x;
        sb += y * y;
    }
    const float ia = 1.0f / sqrtf(block_sum<DP_THREADS>(sa, red) / (float)W + eps);
    const float ib = 1.0f / sqrtf(block_sum<DP_THREADS>(sb, red) / (float)W + eps);
    for (int c = threadIdx.x; c < W; c += DP_THREADS)
        Elem<T>::store(out + row + c, 0.5f * (Elem<T>::load(a + row + c) * ia * wa[c] + Elem<T>::load(b + row + c) * ib * wb[c]));
}

extern "C" int tm_pair_norm_mean(const void* a, const void* b, const float* wa, const float* wb, void* out, int T, int W, float eps,
                                 int dtype, hipStream_t stream) {
    if (!a || !b || !wa || !wb || !out || T < 0 || W <= 0 || !(eps > 0.f)) return TM_ERR_ARG;
    if (dtype != TM_F32 && dtype != TM_BF16) return TM_ERR_ARG;
    if (T == 0) return TM_OK;
    if (dtype == TM_F32)
        pair_norm_mean_kernel<float><<<T, DP_THREADS, 0, stream>>>((const float*)a, (const float*)b, wa, wb, (float*)out, W, eps);
    else
        pair_norm_mean_kernel<bf16_t><<<T, DP_THREADS, 0, stream>>>((const bf16_t*)a, (const bf16_t*)b, wa, wb, (bf16_t*)out, W, eps);
    TM_CHECK_LAUNCH();
    return TM_OK;
}
