// What stands between the projection of q, k and v and an attention over the paged cache, for mixers that norm q and k
// over the whole projection (all heads of a token at once) rather than head by head:
//
//   proj row (32-bit) = [H heads of q, D wide | G heads of k, D wide | G heads of v, Dv wide | ...]   (k and v absent for a
//                        layer that reads another layer's cache)
//   qn = w_q * q / sqrt(mean(q^2 over all H * D) + eps), kn likewise over G * D with w_k      (weights null: no norm)
//   with `per_head` every head of q and of k is normed by itself over its D channels, and w_q, w_k are [D], shared by the heads
//   the first `rot` channels of every head of qn and kn turn by the token's position: pairs (j, j + rot/2), or neighbours
//   (2j, 2j + 1) if `interleaved`; cos/sin [positions, rot/2] hold whatever frequencies and magnitude the model wants
//   q goes to q_out [T, H * D] in the storage type; kn and v to the token's cache slot
//   (K pool [pages, page, G, D], V pool [pages, G, Dv, page])
//
// Everything between the loads and the stores is 32-bit. A block a token: the two sums of squares have one order per
// (H * D, G * D) (a thread strides over the row, lanes and wavefronts are added by the fixed tree of block_sum).
#include "common.h"
#include "api.h"

#define AP_THREADS 256
#define AP_MAX_HEADS 1024         // heads of q and k together that a token's per-head norms take

template <typename T>
__global__ __launch_bounds__(AP_THREADS) void whole_norm_rope_store_kernel(
    const float* __restrict__ proj, int ld, T* __restrict__ q_out, int H, int G, int D, int Dv, int rot, int interleaved,
    const float* __restrict__ q_w, const float* __restrict__ k_w, float eps, const float* __restrict__ cos_t,
    const float* __restrict__ sin_t, const int* __restrict__ positions, const int* __restrict__ slots, T* __restrict__ k_pool,
    T* __restrict__ v_pool, int page, int has_kv, int per_head) {
    __shared__ float red[AP_THREADS / TM_WAVE];
    __shared__ float inv_head[AP_MAX_HEADS];
    const int t = blockIdx.x;
    const float* row = proj + (size_t)t * ld;
    const int Q = H * D, K = has_kv ? G * D : 0;
    const int slot = (has_kv && slots) ? slots[t] : -1;
    const bool store = has_kv && k_pool && slot >= 0;
    float rq = 1.f, rk = 1.f;
    const int heads = H + (has_kv ? G : 0);
    if (per_head && q_w) {                      // a wavefront a head; a head's sum has one order per D
        const int wave = threadIdx.x / TM_WAVE, lane = threadIdx.x % TM_WAVE;
        for (int hh = wave; hh < heads; hh += AP_THREADS / TM_WAVE) {
            float ss = 0.f;
            for (int d = lane; d < D; d += TM_WAVE) ss += row[hh * D + d] * row[hh * D + d];
            ss = wave_sum(ss);
            if (lane == 0) inv_head[hh] = 1.0f / sqrtf(ss / (float)D + eps);
        }
        __syncthreads();
    } else if (q_w) {
        float ss = 0.f;
        for (int c = threadIdx.x; c < Q; c += AP_THREADS) ss += row[c] * row[c];
        rq = 1.0f / sqrtf(block_sum<AP_THREADS>(ss, red) / (float)Q + eps);
    }
    if (!per_head && k_w && K) {
        float ss = 0.f;
        for (int c = threadIdx.x; c < K; c += AP_THREADS) ss += row[Q + c] * row[Q + c];
        rk = 1.0f / sqrtf(block_sum<AP_THREADS>(ss, red) / (float)K + eps);
    }
    const int half = cos_t ? rot / 2 : 0;
    const float* cs = half ? cos_t + (size_t)positions[t] * half : nullptr;
    const float* sn = half ? sin_t + (size_t)positions[t] * half : nullptr;
    T* qo = q_out + (size_t)t * Q;
    T* ko = store ? k_pool + (size_t)slot * G * D : nullptr;
    // the rotated pairs of every head of q and k
    for (int idx = threadIdx.x; idx < heads * half; idx += AP_THREADS) {
        const int hh = idx / half, j = idx % half;
        const int a = interleaved ? 2 * j : j, b = interleaved ? 2 * j + 1 : j + half;
        const int base = hh * D;                // q heads, then k heads, lie one behind the other in the row
        const bool is_q = hh < H;
        const float* w = is_q ? q_w : k_w;
        const float r = per_head ? inv_head[hh] : is_q ? rq : rk;
        const int wb = is_q ? base : base - Q;
        const int wi = per_head ? 0 : wb;       // where the head's weights start
        float x1 = row[base + a], x2 = row[base + b];
        if (w) {
            x1 = w[wi + a] * (x1 * r);
            x2 = w[wi + b] * (x2 * r);
        }
        float y1, y2;
        rotate_pair(x1, x2, cs[j], sn[j], y1, y2);
        if (is_q) {
            Elem<T>::store(qo + base + a, y1);
            Elem<T>::store(qo + base + b, y2);
        } else if (ko) {
            Elem<T>::store(ko + wb + a, y1);
            Elem<T>::store(ko + wb + b, y2);
        }
    }
    // the channels behind the rotated ones
    const int rest = D - 2 * half;
    for (int idx = threadIdx.x; idx < heads * rest; idx += AP_THREADS) {
        const int hh = idx / rest, d = 2 * half + idx % rest;
        const int base = hh * D;
        const bool is_q = hh < H;
        const float* w = is_q ? q_w : k_w;
        const int wb = is_q ? base : base - Q;
        float x = row[base + d];
        if (w) x = w[(per_head ? 0 : wb) + d] * (x * (per_head ? inv_head[hh] : is_q ? rq : rk));
        if (is_q) Elem<T>::store(qo + base + d, x);
        else if (ko) Elem<T>::store(ko + wb + d, x);
    }
    if (store) {
        const int pg = slot / page, in_page = slot % page;
        const float* v = row + Q + K;
        for (int idx = threadIdx.x; idx < G * Dv; idx += AP_THREADS)
            Elem<T>::store(v_pool + ((size_t)pg * G * Dv + idx) * page + in_page, v[idx]);
    }
}

extern "C" int tm_whole_norm_rope_store(const float* proj, int ld, void* q_out, int dtype, int T, int H, int G, int D, int Dv,
                                        int rot, int interleaved, const float* q_w, const float* k_w, float eps,
                                        const float* cos_t, const float* sin_t, const int* positions, const int* slots,
                                        void* k_pool, void* v_pool, int page, int has_kv, int per_head, hipStream_t stream) {
    if (T <= 0) return TM_OK;
    if (per_head && H + G > AP_MAX_HEADS) return TM_ERR_ARG;
    if (!proj || !q_out || H <= 0 || G <= 0 || D <= 0 || Dv <= 0 || rot < 0 || rot > D || (rot & 1)) return TM_ERR_ARG;
    if (ld < H * D + (has_kv ? G * (D + Dv) : 0)) return TM_ERR_ARG;
    if ((q_w || k_w) && !(eps > 0.f)) return TM_ERR_ARG;
    if (has_kv && (q_w == nullptr) != (k_w == nullptr)) return TM_ERR_ARG;
    if (cos_t && rot && (!sin_t || !positions)) return TM_ERR_ARG;
    if (k_pool && (!has_kv || !slots || !v_pool || page <= 0)) return TM_ERR_ARG;
    if (dtype == TM_F32)
        whole_norm_rope_store_kernel<float><<<T, AP_THREADS, 0, stream>>>(proj, ld, (float*)q_out, H, G, D, Dv, rot, interleaved, q_w,
                                                                          k_w, eps, cos_t, sin_t, positions, slots, (float*)k_pool,
                                                                          (float*)v_pool, page, has_kv, per_head);
    else if (dtype == TM_BF16)
        whole_norm_rope_store_kernel<bf16_t><<<T, AP_THREADS, 0, stream>>>(proj, ld, (bf16_t*)q_out, H, G, D, Dv, rot, interleaved,
                                                                           q_w, k_w, eps, cos_t, sin_t, positions, slots,
                                                                           (bf16_t*)k_pool, (bf16_t*)v_pool, page, has_kv, per_head);
    else
        return TM_ERR_ARG;
    TM_CHECK_LAUNCH();
    return TM_OK;
}

// x[t, h * Dv + d] *= sigmoid(gate[t * ldg + h]): a gate per (token, head) on an attention's result, for the kernels that
// do not take the gate themselves.
template <typename T>
__global__ void head_gate_kernel(T* __restrict__ x, const float* __restrict__ gate, int ldg, int H, int Dv, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        const size_t t = i / ((size_t)H * Dv);
        const int h = (int)((i / Dv) % H);
        const float g = 1.f / (1.f + expf(-gate[t * ldg + h]));
        Elem<T>::store(x + i, Elem<T>::load(x + i) * g);
    }
}

extern "C" int tm_head_gate(void* x, int dtype, const float* gate, int ldg, int T, int H, int Dv, hipStream_t stream) {
    if (T <= 0) return TM_OK;
    if (!x || !gate || H <= 0 || Dv <= 0 || ldg < H) return TM_ERR_ARG;
    const size_t n = (size_t)T * H * Dv, want = (n + 255) / 256;
    const int blocks = (int)(want < 16384 ? want : 16384);
    if (dtype == TM_F32) head_gate_kernel<float><<<blocks, 256, 0, stream>>>((float*)x, gate, ldg, H, Dv, n);
    else if (dtype == TM_BF16) head_gate_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)x, gate, ldg, H, Dv, n);
    else return TM_ERR_ARG;
    TM_CHECK_LAUNCH();
    return TM_OK;
}
