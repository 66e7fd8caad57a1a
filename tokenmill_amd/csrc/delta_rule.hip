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
//   tm_pair_norm_mean    out = (rms_norm(a; wa) + rms_norm(b; wb)) / 2: two sublayers side by side, each normed over the width
//
// The columns of S are independent of each other: with d_k = S^T k and d_q = S^T q taken on the state as the token finds it,
//   u = beta (v - g d_k),   o = g d_q + u (k . q),   S <- g S + k u^T
// is the same recurrence with one round of sums a token instead of two. The scan is dealt over (request, head, 16 columns)
// wavefronts; a lane keeps a quarter of a column's D rows in registers, and a column's four partial sums are added in a fixed
// order. A token's result depends on its request's state and tokens only, never on the step's other rows or on how the
// prompt was cut. Everything that enters the recurrence is 32-bit.
#include "common.h"
#include "api.h"

#define DP_THREADS 256
#define DR_MAX_TAPS 16

__device__ __forceinline__ float silu_f32(float z) { return z / (1.0f + expf(-z)); }

// grid T; a block is a token. LDS: C floats (the token's convolved channels).
template <typename T>
__global__ __launch_bounds__(DP_THREADS) void delta_prepare_kernel(const T* __restrict__ proj, int ld, const T* __restrict__ conv_w,
                                                                   const T* __restrict__ conv_state, const float* __restrict__ ba,
                                                                   int ldba, const float* __restrict__ a_log,
                                                                   const float* __restrict__ dt_bias, const int* __restrict__ cu,
                                                                   const int* __restrict__ slots, const int* __restrict__ seq_of_token,
                                                                   float* __restrict__ out, int ldo, int H, int G, int D, int Dv,
                                                                   int taps, float unit_eps) {
    extern __shared__ float ch[];
    const int t = blockIdx.x;
    const int s = seq_of_token[t];
    const int first = cu[s], i = t - first;                  // the token's place among its request's rows of this step
    const int C = 2 * G * D + H * Dv;
    const T* st = conv_state + (size_t)slots[s] * (taps - 1) * C;
    for (int c = threadIdx.x; c < C; c += DP_THREADS) {
        float acc = 0.f;
        for (int j = 0; j < taps; ++j) {
            const int at = i - (taps - 1) + j;               // < 0: before this step's rows, in the state
            const float x = at >= 0 ? Elem<T>::load(proj + (size_t)(first + at) * ld + c)
                                    : Elem<T>::load(st + (size_t)(taps - 1 + at) * C + c);
            acc += Elem<T>::load(conv_w + (size_t)c * taps + j) * x;
        }
        ch[c] = silu_f32(acc);
    }
    __syncthreads();
    float* o = out + (size_t)t * ldo;
    const int wave = threadIdx.x / TM_WAVE, lane = threadIdx.x % TM_WAVE;
    const float q_scale = 1.0f / sqrtf((float)D);
    for (int g = wave; g < G; g += DP_THREADS / TM_WAVE) {   // a wavefront a q/k head
        const float* q = ch + g * D;
        const float* k = ch + G * D + g * D;
        float sq = 0.f, sk = 0.f, qk = 0.f;
        for (int d = lane; d < D; d += TM_WAVE) {
            sq += q[d] * q[d];
            sk += k[d] * k[d];
            qk += q[d] * k[d];
        }
        sq = wave_sum(sq), sk = wave_sum(sk), qk = wave_sum(qk);
        const float iq = q_scale / sqrtf(sq + unit_eps), ik = 1.0f / sqrtf(sk + unit_eps);
        for (int d = lane; d < D; d += TM_WAVE) {
            o[g * D + d] = q[d] * iq;
            o[G * D + g * D + d] = k[d] * ik;
        }
        if (lane == 0) o[C + 2 * H + g] = qk * iq * ik;
    }
    for (int c = 2 * G * D + threadIdx.x; c < C; c += DP_THREADS) o[c] = ch[c];
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
        G <= 0 || H % G || D <= 0 || Dv <= 0 || taps < 1 || taps > DR_MAX_TAPS || (taps > 1 && !conv_state) || ldba < 2 * H ||
        !(unit_eps > 0.f))
        return TM_ERR_ARG;
    const long long C = 2LL * G * D + (long long)H * Dv;
    if (ld < C || ldo < C + 2 * H + G || C * 4 > 64 * 1024) return TM_ERR_ARG;
    if (dtype != TM_F32 && dtype != TM_BF16) return TM_ERR_ARG;
    if (T == 0) return TM_OK;
    const size_t lds = (size_t)C * sizeof(float);
    if (dtype == TM_F32)
        delta_prepare_kernel<float><<<T, DP_THREADS, lds, stream>>>((const float*)proj, ld, (const float*)conv_w, (const float*)conv_state,
                                                                    ba, ldba, a_log, dt_bias, cu_q_lens, state_slots, seq_of_token, out,
                                                                    ldo, H, G, D, Dv, taps, unit_eps);
    else
        delta_prepare_kernel<bf16_t><<<T, DP_THREADS, lds, stream>>>((const bf16_t*)proj, ld, (const bf16_t*)conv_w,
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

// grid (ceil(Dv / (64 / PARTS)), H, S); a block is one wavefront. PARTS (4, or 8 for keys of more than 128 channels) lanes share
// a column's rows: lane = column * PARTS + part; part p keeps rows p * R .. p * R + R - 1 of its column, R = ceil(D / PARTS) <= RMAX. The next token's operands are asked for before the
// current token is worked on. VEC: R is a multiple of 4 and the rows are 16-byte aligned, so a lane's q and k come as float4.
template <int RMAX, int PARTS, bool VEC>
__global__ __launch_bounds__(TM_WAVE) void delta_scan_kernel(const float* __restrict__ rows, int ld, float* __restrict__ o,
                                                            float* __restrict__ state, const int* __restrict__ cu_q_lens,
                                                            const int* __restrict__ state_slots, int H, int G, int D, int Dv) {
    const int lane = threadIdx.x, part = lane % PARTS;
    const int e = blockIdx.x * (TM_WAVE / PARTS) + lane / PARTS;
    const int h = blockIdx.y, s = blockIdx.z;
    const int g = h / (H / G);
    const int R = (D + PARTS - 1) / PARTS;
    const int d0 = part * R;
    const bool col = e < Dv;
    const int t0 = cu_q_lens[s], t1 = cu_q_lens[s + 1];
    if (t1 <= t0) return;
    const int C = 2 * G * D + H * Dv;
    const size_t q_at = (size_t)g * D + d0, k_at = (size_t)G * D + (size_t)g * D + d0, v_at = (size_t)2 * G * D + (size_t)h * Dv + (col ? e : 0);
    float* st = state + (((size_t)state_slots[s] * H + h) * D) * Dv + (col ? e : 0);
    float S[RMAX];
#pragma unroll
    for (int i = 0; i < RMAX; ++i) S[i] = (col && i < R && d0 + i < D) ? st[(size_t)(d0 + i) * Dv] : 0.f;
    float cq[RMAX], ck[RMAX], nq[RMAX], nk[RMAX];
    float cv, cb, cg, cx, nv, nb, ng, nx;
    auto fetch = [&](int t, float* q, float* k, float& v, float& b, float& gd, float& x) {
        const float* row = rows + (size_t)t * ld;
        if (VEC) {
#pragma unroll
            for (int i = 0; i < RMAX; i += 4)
                if (i < R) {
                    const float4 a = *(const float4*)(row + q_at + i), c = *(const float4*)(row + k_at + i);
                    q[i] = a.x, q[i + 1] = a.y, q[i + 2] = a.z, q[i + 3] = a.w;
                    k[i] = c.x, k[i + 1] = c.y, k[i + 2] = c.z, k[i + 3] = c.w;
                }
        } else {
#pragma unroll
            for (int i = 0; i < RMAX; ++i) {
                const bool in = i < R && d0 + i < D;
                q[i] = in ? row[q_at + i] : 0.f;
                k[i] = in ? row[k_at + i] : 0.f;
            }
        }
        v = row[v_at];
        b = row[C + h];
        gd = row[C + H + h];
        x = row[C + 2 * H + g];
    };
    fetch(t0, cq, ck, cv, cb, cg, cx);
    for (int t = t0; t < t1; ++t) {
        fetch(t + 1 < t1 ? t + 1 : t, nq, nk, nv, nb, ng, nx);            // the last token asks for itself again
        float dk = 0.f, dq = 0.f;
#pragma unroll
        for (int i = 0; i < RMAX; ++i)
            if (i < R) {
                dk += S[i] * ck[i];
                dq += S[i] * cq[i];
            }
        dk += __shfl_xor(dk, 1, TM_WAVE);
        dq += __shfl_xor(dq, 1, TM_WAVE);
        dk += __shfl_xor(dk, 2, TM_WAVE);
        dq += __shfl_xor(dq, 2, TM_WAVE);
        if (PARTS == 8) {
            dk += __shfl_xor(dk, 4, TM_WAVE);
            dq += __shfl_xor(dq, 4, TM_WAVE);
        }
        const float u = cb * (cv - cg * dk);
#pragma unroll
        for (int i = 0; i < RMAX; ++i)
            if (i < R) S[i] = cg * S[i] + ck[i] * u;
        if (col && part == 0) o[((size_t)t * H + h) * Dv + e] = cg * dq + u * cx;
#pragma unroll
        for (int i = 0; i < RMAX; ++i) cq[i] = nq[i], ck[i] = nk[i];
        cv = nv, cb = nb, cg = ng, cx = nx;
    }
#pragma unroll
    for (int i = 0; i < RMAX; ++i)
        if (col && i < R && d0 + i < D) st[(size_t)(d0 + i) * Dv] = S[i];
}

extern "C" int tm_delta_scan(const float* rows, int ld, float* o, float* state, const int* cu_q_lens, const int* state_slots, int S,
                             int H, int G, int D, int Dv, hipStream_t stream) {
    if (!rows || !o || !state || !cu_q_lens || !state_slots || S < 0 || H <= 0 || G <= 0 || H % G || D <= 0 || D > 256 || Dv <= 0 ||
        H > 65535 || S > 65535 || (long long)ld < 2LL * G * D + (long long)H * Dv + 2 * H + G)
        return TM_ERR_ARG;
    if (S == 0) return TM_OK;
    const int parts = D > 128 ? 8 : 4, cols = TM_WAVE / parts;
    const dim3 grid((Dv + cols - 1) / cols, H, S);
    const int R = (D + parts - 1) / parts;
    const bool vec = D % (4 * parts) == 0 && ld % 4 == 0 && ((uintptr_t)rows % 16) == 0;
#define DR_GO(RM, P)                                                                                                            \
    do {                                                                                                                        \
        if (vec) delta_scan_kernel<RM, P, true><<<grid, TM_WAVE, 0, stream>>>(rows, ld, o, state, cu_q_lens, state_slots, H, G, D, Dv); \
        else delta_scan_kernel<RM, P, false><<<grid, TM_WAVE, 0, stream>>>(rows, ld, o, state, cu_q_lens, state_slots, H, G, D, Dv);    \
    } while (0)
    if (parts == 8) DR_GO(32, 8);
    else if (R <= 8) DR_GO(8, 4);
    else if (R <= 16) DR_GO(16, 4);
    else DR_GO(32, 4);
#undef DR_GO
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
