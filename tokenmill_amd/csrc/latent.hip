// Attention over a shared latent: every token caches one row [Lk latent channels | Dr rotated key channels] and all
// query heads read the same rows (the per-head key and value matrices are applied to the query and to the result
// instead of to every cached row).
//
//   low[t] = [ q latent (Lq) | kv latent (Lk) | shared key (Dr) | ... ]           32-bit rows of the down projections
//   tm_latent_prepare   cq[t] = rms_norm(low[t, :Lq]; wq)                          -> the up projection of the queries
//                       row[t] = [ rms_norm(low[t, Lq:Lq+Lk]; wk) | rotate(low[t, Lq+Lk : Lq+Lk+Dr]) ] -> cache slot of t
//   tm_heads_matmul     C[t, h, :N] = A[t, h, :K] . B[h]  (B [H, K, N]), optionally times sigmoid(gate[t, h])
//   tm_rotate_heads     dst[t, h, :Dr] = rotate(src[t, h, :Dr])                    the rotated part of every query head
//   tm_attn_latent      out[t, h, :Lk] = softmax_j(scale * qa[t, h] . row[j]) . row[j, :Lk]   over the window's rows
//
// The rotation pairs channels (2i, 2i + 1), i < rot / 2, or with `half_pairs` channels (i, i + rot / 2), by the angle
// position * f_i (cos and sin from a 32-bit table [positions, rot / 2]); channels from rot on pass unchanged. Norm
// statistics, scores, softmax and all sums are 32-bit. A softmax may have a sink: one more term exp(sink[h]) in the
// denominator of head h, with no row behind it (sink null: none).
#include "common.h"
#include "api.h"

#define LP_THREADS 256

template <typename T>
__global__ __launch_bounds__(LP_THREADS) void latent_prepare_kernel(const float* __restrict__ low, int ld, int Lq, int Lk, int Dr,
                                                                    int rot, const float* __restrict__ wq,
                                                                    const float* __restrict__ wk, float eps,
                                                                    const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                                                    const int* __restrict__ positions, const int* __restrict__ slots,
                                                                    T* __restrict__ cq, T* __restrict__ pool, int half_pairs) {
    __shared__ float red[LP_THREADS / TM_WAVE];
    const int t = blockIdx.x;
    const float* row = low + (size_t)t * ld;
    float sq = 0.f, sk = 0.f;
    for (int c = threadIdx.x; c < Lq; c += LP_THREADS) sq += row[c] * row[c];
    for (int c = threadIdx.x; c < Lk; c += LP_THREADS) sk += row[Lq + c] * row[Lq + c];
    if (Lq > 0) {
        const float inv = 1.0f / sqrtf(block_sum<LP_THREADS>(sq, red) / (float)Lq + eps);
        for (int c = threadIdx.x; c < Lq; c += LP_THREADS) Elem<T>::store(cq + (size_t)t * Lq + c, row[c] * inv * wq[c]);
    }
    const int slot = slots ? slots[t] : -1;
    if (Lk == 0 || !slots) return;                            // a layer without a latent of its own: block-uniform
    const float invk = 1.0f / sqrtf(block_sum<LP_THREADS>(sk, red) / (float)Lk + eps);
    if (slot < 0) return;
    T* dst = pool + (size_t)slot * (Lk + Dr);
    for (int c = threadIdx.x; c < Lk; c += LP_THREADS) Elem<T>::store(dst + c, row[Lq + c] * invk * wk[c]);
    const float* kr = row + Lq + Lk;
    const int half = rot / 2;
    const int p = rot ? positions[t] : 0;
    for (int i = threadIdx.x; i < half; i += LP_THREADS) {
        float a, b;
        const int i1 = half_pairs ? i : 2 * i, i2 = half_pairs ? i + half : 2 * i + 1;
        rotate_pair(kr[i1], kr[i2], cos_t[(size_t)p * half + i], sin_t[(size_t)p * half + i], a, b);
        Elem<T>::store(dst + Lk + i1, a);
        Elem<T>::store(dst + Lk + i2, b);
    }
    for (int c = rot + threadIdx.x; c < Dr; c += LP_THREADS) Elem<T>::store(dst + Lk + c, kr[c]);
}

extern "C" int tm_latent_prepare(const float* low, int ld, int Lq, int Lk, int Dr, int rot, const float* wq, const float* wk,
                                 float eps, const float* cos_t, const float* sin_t, const int* positions, const int* slots,
                                 void* cq, void* pool, int dtype, int T, int half_pairs, hipStream_t stream) {
    if (!low || Lq < 0 || Lk < 0 || Lq + Lk <= 0 || Dr < 0 || rot < 0 || rot > Dr || rot % 2 || ld < Lq + Lk + Dr || (Lk && !wk) ||
        (!Lk && (slots || Dr)) || (Lq && (!wq || !cq)) ||
        (rot && (!cos_t || !sin_t || !positions)) || (slots && !pool) || !(eps > 0.f) || T < 0)
        return TM_ERR_ARG;
    if (dtype != TM_F32 && dtype != TM_BF16) return TM_ERR_ARG;
    if (T == 0) return TM_OK;
    if (dtype == TM_F32)
        latent_prepare_kernel<float><<<T, LP_THREADS, 0, stream>>>(low, ld, Lq, Lk, Dr, rot, wq, wk, eps, cos_t, sin_t, positions,
                                                                   slots, (float*)cq, (float*)pool, half_pairs);
    else
        latent_prepare_kernel<bf16_t><<<T, LP_THREADS, 0, stream>>>(low, ld, Lq, Lk, Dr, rot, wq, wk, eps, cos_t, sin_t, positions,
                                                                    slots, (bf16_t*)cq, (bf16_t*)pool, half_pairs);
    TM_CHECK_LAUNCH();
    return TM_OK;
}

// ------------------------------------------------------------------------------------------------ per-head products

#define HM_TM 32
#define HM_TN 64
#define HM_TK 16

// A block computes 32 tokens x 64 columns of one head; k ascends in steps of 16 through LDS, so an element's sum has one
// order whatever rows stand beside it.
template <typename T>
__global__ __launch_bounds__(256) void heads_matmul_kernel(const T* __restrict__ A, int lda, int a_head, const T* __restrict__ B,
                                                           T* __restrict__ C, int ldc, int c_head, const float* __restrict__ gate,
                                                           int ldg, int rows, int K, int N) {
    __shared__ float As[HM_TM][HM_TK + 1];
    __shared__ float Bs[HM_TK][HM_TN];
    const int h = blockIdx.z;
    const int t0 = blockIdx.x * HM_TM, n0 = blockIdx.y * HM_TN;
    const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;      // columns tx * 4 .. + 3, rows ty * 2, ty * 2 + 1
    const T* Bh = B + (size_t)h * K * N;
    float acc[2][4] = {};
    for (int k0 = 0; k0 < K; k0 += HM_TK) {
        for (int i = threadIdx.x; i < HM_TM * HM_TK; i += 256) {
            const int r = i / HM_TK, k = i % HM_TK;
            As[r][k] = (t0 + r < rows && k0 + k < K) ? Elem<T>::load(A + (size_t)(t0 + r) * lda + (size_t)h * a_head + k0 + k) : 0.f;
        }
        for (int i = threadIdx.x; i < HM_TK * HM_TN; i += 256) {
            const int k = i / HM_TN, n = i % HM_TN;
            Bs[k][n] = (k0 + k < K && n0 + n < N) ? Elem<T>::load(Bh + (size_t)(k0 + k) * N + n0 + n) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < HM_TK; ++k) {
            const float a0 = As[ty * 2][k], a1 = As[ty * 2 + 1][k];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float b = Bs[k][tx * 4 + j];
                acc[0][j] += a0 * b;
                acc[1][j] += a1 * b;
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int t = t0 + ty * 2 + i;
        if (t >= rows) continue;
        const float g = gate ? 1.0f / (1.0f + __expf(-gate[(size_t)t * ldg + h])) : 1.0f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n < N) Elem<T>::store(C + (size_t)t * ldc + (size_t)h * c_head + n, acc[i][j] * g);
        }
    }
}

extern "C" int tm_heads_matmul(const void* A, int lda, int a_head, const void* B, void* C, int ldc, int c_head, const float* gate,
                               int ldg, int T, int H, int K, int N, int dtype, hipStream_t stream) {
    if (!A || !B || !C || T < 0 || H <= 0 || H > 65535 || K <= 0 || N <= 0 || a_head < K || c_head < N ||
        (long long)lda < (long long)(H - 1) * a_head + K || (long long)ldc < (long long)(H - 1) * c_head + N || (gate && ldg < H))
        return TM_ERR_ARG;
    if (dtype != TM_F32 && dtype != TM_BF16) return TM_ERR_ARG;
    if (T == 0) return TM_OK;
    dim3 grid((T + HM_TM - 1) / HM_TM, (N + HM_TN - 1) / HM_TN, H);
    if (grid.y > 65535) return TM_ERR_ARG;
    if (dtype == TM_F32)
        heads_matmul_kernel<float><<<grid, 256, 0, stream>>>((const float*)A, lda, a_head, (const float*)B, (float*)C, ldc, c_head,
                                                             gate, ldg, T, K, N);
    else
        heads_matmul_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)A, lda, a_head, (const bf16_t*)B, (bf16_t*)C, ldc,
                                                              c_head, gate, ldg, T, K, N);
    TM_CHECK_LAUNCH();
    return TM_OK;
}

template <typename T>
__global__ __launch_bounds__(256) void rotate_heads_kernel(const T* __restrict__ src, int lds_, int s_head, T* __restrict__ dst,
                                                           int ldd, int d_head, int H, int Dr, int rot,
                                                           const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                                           const int* __restrict__ positions, int half_pairs) {
    const int t = blockIdx.x;
    const int half = rot / 2;
    const int p = rot ? positions[t] : 0;
    for (int i = threadIdx.x; i < H * half; i += 256) {
        const int h = i / half, c = i % half;
        const T* s = src + (size_t)t * lds_ + (size_t)h * s_head;
        T* d = dst + (size_t)t * ldd + (size_t)h * d_head;
        float a, b;
        const int c1 = half_pairs ? c : 2 * c, c2 = half_pairs ? c + half : 2 * c + 1;
        rotate_pair(Elem<T>::load(s + c1), Elem<T>::load(s + c2), cos_t[(size_t)p * half + c], sin_t[(size_t)p * half + c], a, b);
        Elem<T>::store(d + c1, a);
        Elem<T>::store(d + c2, b);
    }
    const int rest = Dr - rot;
    for (int i = threadIdx.x; i < H * rest; i += 256) {
        const int h = i / rest, c = rot + i % rest;
        dst[(size_t)t * ldd + (size_t)h * d_head + c] = src[(size_t)t * lds_ + (size_t)h * s_head + c];
    }
}

extern "C" int tm_rotate_heads(const void* src, int ld_src, int src_head, void* dst, int ld_dst, int dst_head, int T, int H, int Dr,
                               int rot, const float* cos_t, const float* sin_t, const int* positions, int dtype, int half_pairs,
                               hipStream_t stream) {
    if (!src || !dst || T < 0 || H <= 0 || Dr < 0 || rot < 0 || rot > Dr || rot % 2 || src_head < Dr || dst_head < Dr ||
        (rot && (!cos_t || !sin_t || !positions)))
        return TM_ERR_ARG;
    if (dtype != TM_F32 && dtype != TM_BF16) return TM_ERR_ARG;
    if (T == 0 || Dr == 0) return TM_OK;
    if (dtype == TM_F32)
        rotate_heads_kernel<float><<<T, 256, 0, stream>>>((const float*)src, ld_src, src_head, (float*)dst, ld_dst, dst_head, H, Dr, rot,
                                                          cos_t, sin_t, positions, half_pairs);
    else
        rotate_heads_kernel<bf16_t><<<T, 256, 0, stream>>>((const bf16_t*)src, ld_src, src_head, (bf16_t*)dst, ld_dst, dst_head, H, Dr,
                                                           rot, cos_t, sin_t, positions, half_pairs);
    TM_CHECK_LAUNCH();
    return TM_OK;
}

// ------------------------------------------------------------------------------------------------ attention

#define AL_WAVES 4

// what the lanes of one wavefront wrote to LDS is seen by its other lanes behind this
__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}
#define AL_MAX_DK 704           // cached row: latent + rotated channels
#define AL_MAX_ACC 8            // latent channels a lane adds up: Lk <= 8 * 64

// One wavefront per (token, head). Rows are visited in rounds of 64 from the first visible one: a lane takes one row's
// score, the round's weights go through LDS, then a lane per latent channel adds the round's rows in ascending order.
// The running maximum and sum follow the rounds, so a token's result depends on its own position and window only.
template <typename T>
__global__ __launch_bounds__(AL_WAVES * TM_WAVE) void attn_latent_kernel(const T* __restrict__ qa, int q_stride, T* __restrict__ out,
                                                                         int out_stride, const T* __restrict__ pool,
                                                                         const int* __restrict__ block_tables, int table_width,
                                                                         const int* __restrict__ seq_of_token,
                                                                         const int* __restrict__ positions, int T_tokens, int H,
                                                                         int Lk, int Dk, int page, float scale, int window,
                                                                         const float* __restrict__ sink) {
    __shared__ float q_s[AL_WAVES][AL_MAX_DK];
    __shared__ float p_s[AL_WAVES][TM_WAVE];
    __shared__ int slot_s[AL_WAVES][TM_WAVE];
    const int wave = threadIdx.x / TM_WAVE, lane = threadIdx.x % TM_WAVE;
    const long long w = (long long)blockIdx.x * AL_WAVES + wave;
    if (w >= (long long)T_tokens * H) return;                 // whole wavefronts leave; no block-wide barrier below
    const int t = (int)(w / H), h = (int)(w % H);
    const int s = seq_of_token[t];
    const int p = positions[t];
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int* table = block_tables + (size_t)s * table_width;
    float* qs = q_s[wave];
    const T* qrow = qa + (size_t)t * q_stride + (size_t)h * Dk;
    for (int d = lane; d < Dk; d += TM_WAVE) qs[d] = Elem<T>::load(qrow + d);
    wave_lds_sync();

    float m = -INFINITY, l = 0.f;
    float acc[AL_MAX_ACC];
#pragma unroll
    for (int i = 0; i < AL_MAX_ACC; ++i) acc[i] = 0.f;
    for (int j0 = lo; j0 <= p; j0 += TM_WAVE) {
        const int j = j0 + lane;
        const bool seen = j <= p;
        float sc = -INFINITY;
        int slot = 0;
        if (seen) {
            slot = table[j / page] * page + j % page;
            const T* krow = pool + (size_t)slot * Dk;
            float dot = 0.f;
            for (int d = 0; d < Dk; ++d) dot += qs[d] * Elem<T>::load(krow + d);
            sc = dot * scale;
        }
        const float m_new = fmaxf(m, wave_max(sc));
        const float pw = seen ? __expf(sc - m_new) : 0.f;
        const float alpha = __expf(m - m_new);                // 0 in the first round (m = -inf)
        l = l * alpha + wave_sum(pw);
        m = m_new;
        p_s[wave][lane] = pw;
        slot_s[wave][lane] = slot;
        wave_lds_sync();
        const int n = min(TM_WAVE, p - j0 + 1);
#pragma unroll
        for (int i = 0; i < AL_MAX_ACC; ++i) {
            const int c = lane + i * TM_WAVE;
            if (c < Lk) {
                float a = acc[i] * alpha;
                for (int k = 0; k < n; ++k) a += p_s[wave][k] * Elem<T>::load(pool + (size_t)slot_s[wave][k] * Dk + c);
                acc[i] = a;
            }
        }
        wave_lds_sync();
    }
    if (sink) l += __expf(sink[h] - m);                      // the sink: a term of the denominator without a row
    const float inv = 1.0f / l;
    T* o = out + (size_t)t * out_stride + (size_t)h * Lk;
#pragma unroll
    for (int i = 0; i < AL_MAX_ACC; ++i) {
        const int c = lane + i * TM_WAVE;
        if (c < Lk) Elem<T>::store(o + c, acc[i] * inv);
    }
}

extern "C" int tm_attn_latent(const void* qa, int q_stride, void* out, int out_stride, const void* pool, const int* block_tables,
                              int table_width, const int* seq_of_token, const int* positions, int T, int H, int Lk, int Dk, int page,
                              float scale, int window, const float* sink, int dtype, hipStream_t stream) {
    if (!qa || !out || !pool || !block_tables || !seq_of_token || !positions || T < 0 || H <= 0 || Lk <= 0 || Lk > Dk ||
        Dk > AL_MAX_DK || Lk > AL_MAX_ACC * TM_WAVE || page <= 0 || window < 0 || table_width <= 0 ||
        (long long)q_stride < (long long)H * Dk || (long long)out_stride < (long long)H * Lk)
        return TM_ERR_ARG;
    if (dtype != TM_F32 && dtype != TM_BF16) return TM_ERR_ARG;
    if (T == 0) return TM_OK;
    const long long pairs = (long long)T * H;
    const long long blocks = (pairs + AL_WAVES - 1) / AL_WAVES;
    if (blocks > 0x7fffffffLL) return TM_ERR_ARG;
    if (dtype == TM_F32)
        attn_latent_kernel<float><<<(unsigned)blocks, AL_WAVES * TM_WAVE, 0, stream>>>(
            (const float*)qa, q_stride, (float*)out, out_stride, (const float*)pool, block_tables, table_width, seq_of_token,
            positions, T, H, Lk, Dk, page, scale, window, sink);
    else
        attn_latent_kernel<bf16_t><<<(unsigned)blocks, AL_WAVES * TM_WAVE, 0, stream>>>(
            (const bf16_t*)qa, q_stride, (bf16_t*)out, out_stride, (const bf16_t*)pool, block_tables, table_width, seq_of_token,
            positions, T, H, Lk, Dk, page, scale, window, sink);
    TM_CHECK_LAUNCH();
    return TM_OK;
}
